"""Per-step vTensor bookkeeping that the reference does at the top of ``LlamaModel.forward``
(vllm/model_executor/models/llama.py:307-341): advance every scheduled sequence's range, map a
chunk where a sequence crosses a 2 MiB boundary, and hand the byte offsets to the kernels."""
from __future__ import annotations

from typing import List, Sequence

import torch

from .. import vmm_allocator as vmm


def prepare_step(attn_metadata, kv_caches: Sequence) -> None:
    """Fills ``attn_metadata.slot_m`` (and ``decode_seq_len``) for this step.

    kv_caches: per layer a (K, V) pair of ``KV_cache`` handles, or None entries during profiling.
    """
    if not kv_caches or kv_caches[0] is None:
        return
    k_cache = [k.kv_cache for k, _ in kv_caches]
    v_cache = [v.kv_cache for _, v in kv_caches]
    kv_size = attn_metadata.kv_num_heads * attn_metadata.kv_head_size * 2  # llama.py:315, bytes of a bf16 row
    n = len(attn_metadata.slot_mapping_list)
    if attn_metadata.num_prefills > 0:
        kv_size_list: List[int] = [seq_len * kv_size for seq_len in attn_metadata.seq_lens]  # llama.py:318-320
        decode_seq_len = None
    else:
        # llama.py:321-337: the reference spins on its background mapper here and then queues
        # eagerExtend requests; mapping is synchronous in this library, so only the requests remain
        decode_seq_len = torch.ones(n, dtype=torch.int32, device=attn_metadata.slot_mapping.device)
        kv_size_list = [kv_size] * n
        for idx, slot_id in enumerate(attn_metadata.extend_seq_list):
            if slot_id != -1:
                attn_metadata.kvcache_segment[idx].eagerExtend(kv_size, slot_id)
    attn_metadata.decode_seq_len = decode_seq_len
    slot_m = vmm.extend_kv_cache_batch(k_cache, v_cache, attn_metadata.slot_mapping_list, kv_size_list,
                                       attn_metadata.kvcache_segment, attn_metadata.set_used_size, kv_size,
                                       attn_metadata.num_prefills == 0)  # llama.py:340
    attn_metadata.slot_m = torch.tensor(slot_m, dtype=torch.int64, device=attn_metadata.slot_mapping.device)
