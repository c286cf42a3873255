"""Per-layer scales of an fp8-e4m3fn KV cache, read from the JSON file the reference's quantisation tools write.

Restates `kv_cache_scales_loader` (vllm/model_executor/model_loader/weight_utils.py:296-333) and the checks
of its schema (vllm/model_executor/layers/quantization/schema.py:19-84): the file holds
``{"model_type": ..., "kv_cache": {"dtype": "float8_e4m3fn", "scaling_factor": {tp_rank: {layer: scale}}}}``;
one scale per layer serves K and V alike (the model passes it as ``kv_scale`` to the attention layer,
vllm/model_executor/models/llama.py:484-505).  A file that cannot be used yields no scales and a warning,
which leaves every layer at 1.0, as in the reference.
"""
from __future__ import annotations

import json
import logging
from typing import Iterable, List, Optional, Tuple

logger = logging.getLogger(__name__)


class KVScalesError(ValueError):
    pass


def _validated(doc, tp_rank: int, tp_size: int, num_hidden_layers: int, model_type: Optional[str]):
    if not isinstance(doc, dict) or "kv_cache" not in doc:
        raise KVScalesError("no 'kv_cache' section")
    if model_type is not None and doc.get("model_type") != model_type:
        raise KVScalesError(f"scales belong to model type {doc.get('model_type')!r}, the model is {model_type!r}")
    kv = doc["kv_cache"]
    if kv.get("dtype") != "float8_e4m3fn":
        raise KVScalesError(f"scales are for KV cache dtype {kv.get('dtype')!r}, not float8_e4m3fn")
    by_rank = {int(r): {int(l): float(s) for l, s in layers.items()} for r, layers in kv["scaling_factor"].items()}
    if len(by_rank) != tp_size or any(r not in by_rank for r in range(tp_size)):
        raise KVScalesError(f"the file holds TP ranks {sorted(by_rank)}, the engine runs with TP size {tp_size}")
    for rank, layers in by_rank.items():
        if len(layers) != num_hidden_layers:
            raise KVScalesError(f"TP rank {rank} holds {len(layers)} layers, the model has {num_hidden_layers}")
    mine = by_rank[tp_rank]
    missing = [l for l in range(num_hidden_layers) if l not in mine]
    if missing:
        raise KVScalesError(f"no scale for layers {missing[:8]} of TP rank {tp_rank}")
    if any(not (s > 0.0) for s in mine.values()):
        raise KVScalesError("scales must be positive")
    return mine


def kv_cache_scales_loader(filename: str, tp_rank: int, tp_size: int, num_hidden_layers: int,
                           model_type: Optional[str]) -> Iterable[Tuple[int, float]]:
    """(layer, scale) pairs of `tp_rank`, or an empty list (with a warning) when the file is missing, is not JSON
    or does not fit the model: the caller then keeps 1.0 everywhere."""
    try:
        with open(filename) as f:
            doc = json.load(f)
        return list(_validated(doc, tp_rank, tp_size, num_hidden_layers, model_type).items())
    except FileNotFoundError:
        logger.error("File or directory '%s' not found.", filename)
    except json.JSONDecodeError:
        logger.error("Error decoding JSON in file '%s'.", filename)
    except Exception as e:  # noqa: BLE001 - as the reference: any failure falls back to 1.0
        logger.error("An error occurred while reading '%s': %s", filename, e)
    logger.warning("Defaulting to KV cache scaling factors = 1.0 for all layers in TP rank %d as an error occurred "
                   "during loading.", tp_rank)
    return []


def layer_scales(filename: str, num_hidden_layers: int, tp_rank: int = 0, tp_size: int = 1,
                 model_type: Optional[str] = None) -> List[float]:
    """One scale per layer, 1.0 where the file gave none."""
    out = [1.0] * num_hidden_layers
    for layer, scale in kv_cache_scales_loader(filename, tp_rank, tp_size, num_hidden_layers, model_type):
        out[layer] = scale
    return out
