"""Cache and attention ops with the names, argument order and error behaviour of the
reference's ``vllm/_custom_ops.py`` (attention :34-77, cache ops :238-281), implemented by
the HIP kernels of ``libvtkv.so``.

All ops work in place on caller-owned tensors, run asynchronously on torch's current
stream and return ``None``; bad arguments raise ``RuntimeError`` (``VtkvError``), as the
reference's ``TORCH_CHECK`` does.  PyTorch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence, Union

import torch

from . import _C

_DTYPES = {torch.float32: _C.F32, torch.bfloat16: _C.BF16, torch.float16: _C.F16, torch.uint8: _C.FP8_E4M3}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPES[torch.float8_e4m3fn] = _C.FP8_E4M3

_PARTITION_SIZE = 512  # vllm/attention/ops/paged_attn.py:10


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t) -> C.c_void_p:
    """Device/host address of a tensor, a raw integer address, or NULL for None."""
    if t is None:
        return C.c_void_p(0)
    if isinstance(t, int):
        return C.c_void_p(t)
    return C.c_void_p(t.data_ptr())


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise _C.VtkvError(_C.EINVAL, f"unsupported dtype {t.dtype}") from None


def _kv_dtype(kv_cache_dtype: str, model_dtype: int) -> int:
    if kv_cache_dtype == "auto":
        return model_dtype
    if kv_cache_dtype in ("fp8", "fp8_e4m3"):
        return _C.FP8_E4M3
    raise _C.VtkvError(_C.EINVAL, f"Unsupported data type of kv cache: {kv_cache_dtype}")


def _require_cuda(*tensors) -> None:
    for t in tensors:
        if isinstance(t, torch.Tensor) and not t.is_cuda:
            raise _C.VtkvError(_C.EINVAL, "tensor must live on the GPU")


# Scratch for the attention's partial results, grown on demand: one per device and stream, because calls
# that run at the same time must not share it (they would mix their partial results and arrival counters).
# The library wants it zero-filled before its first use (it keeps the counters there and resets them itself).
_workspaces = {}


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None and torch.cuda.is_current_stream_capturing():
        # a graph is being recorded: use the scratch an eager call on this device has made before, so that the
        # graph neither allocates nor clears 35 MiB at every replay (replay it on that call's stream)
        for (dev, _), other in _workspaces.items():
            if dev == device and other.numel() >= nbytes:
                return other
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


# --------------------------------------------------------------------------------------- attention
def paged_attention_v1(
    out: torch.Tensor,
    query: torch.Tensor,
    key_cache: Union[int, torch.Tensor],
    value_cache: Union[int, torch.Tensor],
    num_kv_heads: int,
    scale: float,
    seq_lens: torch.Tensor,
    block_size: int,
    max_seq_len: int,
    alibi_slopes: Optional[torch.Tensor],
    kv_cache_dtype: str,
    kv_scale: float,
    slot_mapping: torch.Tensor,
    v_scale: Optional[float] = None,
    partition_tokens: int = 0,
) -> None:
    """Fork signature (csrc/ops.h:6-19): key_cache / value_cache are the device address of
    (or an int64 tensor holding) the per-slot base pointers, ``slot_mapping`` holds each
    sequence's slot; ``block_size`` must be 1 (vllm/attention/ops/paged_attn.py:105).
    ``kv_scale`` scales K (and V unless ``v_scale`` is given) for an fp8 cache.  ``out`` has the
    query's dtype, or float32 to receive the result before its final rounding."""
    if block_size != 1:
        raise _C.VtkvError(_C.EINVAL, f"Unsupported block size: {block_size} (contiguous ranges use 1)")
    _require_cuda(out, query, seq_lens, slot_mapping)
    num_seqs, num_heads, head_size = query.shape
    if not out.is_contiguous():
        raise _C.VtkvError(_C.EINVAL, "out must be contiguous")
    if seq_lens.dtype != torch.int32 or slot_mapping.dtype != torch.int64:
        raise _C.VtkvError(_C.EINVAL, "seq_lens must be int32 and slot_mapping int64")
    qd = _dt(query)
    lib = _C.lib()
    need = lib.vtkv_decode_attention_workspace_bytes(num_seqs, num_heads, head_size, max_seq_len, partition_tokens)
    ws = _workspace(need, query.device)
    if alibi_slopes is not None:
        alibi_slopes = alibi_slopes.to(device=query.device, dtype=torch.float32)
    _C.check(lib.vtkv_decode_attention(
        _ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), _ptr(slot_mapping), _ptr(seq_lens),
        num_seqs, num_heads, num_kv_heads, head_size, query.stride(0), float(scale), int(max_seq_len),
        _ptr(alibi_slopes), qd, _dt(out), _kv_dtype(kv_cache_dtype, qd), float(kv_scale),
        float(kv_scale if v_scale is None else v_scale), _ptr(ws), ws.numel(), int(partition_tokens), _stream()))


def decode_append_attention(
    out: torch.Tensor,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: Union[int, torch.Tensor],
    value_cache: Union[int, torch.Tensor],
    num_kv_heads: int,
    scale: float,
    seq_lens: Union[torch.Tensor, Sequence[int]],
    max_seq_len: int,
    alibi_slopes: Optional[torch.Tensor],
    slot_mapping: torch.Tensor,
    partition_tokens: int = 0,
    kv_cache_dtype: str = "auto",
    kv_scale: float = 1.0,
    v_scale: Optional[float] = None,
) -> None:
    """One launch for the two calls a decode step makes per layer, ``reshape_and_cache`` then
    ``paged_attention_v1`` (vllm/attention/backends/xformers.py:310-312 and :357-371): ``key`` /
    ``value`` hold one new row per sequence, ``seq_lens`` counts it, the row lands at position
    ``seq_lens[b] - 1`` of sequence b's ranges and attention runs over all ``seq_lens[b]`` rows.
    ``seq_lens`` is an int32 GPU tensor, or a host sequence of at most 512 ints (then nothing is
    uploaded).  The cache is bf16, or fp8 (``kv_cache_dtype="fp8"`` with ``kv_scale`` / ``v_scale``: the row is
    stored quantised exactly as ``reshape_and_cache`` stores it).  No counterpart as a single op in the
    reference."""
    _require_cuda(out, query, key, value, slot_mapping)
    num_seqs, num_heads, head_size = query.shape
    if not out.is_contiguous():
        raise _C.VtkvError(_C.EINVAL, "out must be contiguous")
    if slot_mapping.dtype != torch.int64:
        raise _C.VtkvError(_C.EINVAL, "slot_mapping must be int64")
    key = key.view(-1, num_kv_heads, head_size)
    value = value.view(-1, num_kv_heads, head_size)
    if key.shape[0] != num_seqs or value.shape[0] != num_seqs:
        raise _C.VtkvError(_C.EINVAL, "key/value must hold one row per sequence")
    if key.stride(2) != 1 or key.stride(1) != head_size or value.stride(2) != 1 or value.stride(1) != head_size:
        raise _C.VtkvError(_C.EINVAL, "key/value rows must be contiguous in (head, dim)")
    if isinstance(seq_lens, torch.Tensor):
        _require_cuda(seq_lens)
        if seq_lens.dtype != torch.int32:
            raise _C.VtkvError(_C.EINVAL, "seq_lens must be int32")
        dev_lens, host_lens = _ptr(seq_lens), None
    else:
        if len(seq_lens) != num_seqs:
            raise _C.VtkvError(_C.EINVAL, "one sequence length per query row")
        # (a ctypes int32 array made by an earlier call is taken as it is: a step's lengths serve every layer)
        dev_lens, host_lens = None, seq_lens if isinstance(seq_lens, C.Array) else (C.c_int32 * num_seqs)(*seq_lens)
    qd = _dt(query)
    lib = _C.lib()
    need = lib.vtkv_decode_attention_workspace_bytes(num_seqs, num_heads, head_size, max_seq_len, partition_tokens)
    ws = _workspace(need, query.device)
    if alibi_slopes is not None:
        alibi_slopes = alibi_slopes.to(device=query.device, dtype=torch.float32)
    _C.check(lib.vtkv_decode_append_attention(
        _ptr(out), _ptr(query), _ptr(key), _ptr(value), key.stride(0), value.stride(0), _ptr(key_cache),
        _ptr(value_cache), _ptr(slot_mapping), dev_lens, host_lens, num_seqs, num_heads, num_kv_heads, head_size,
        query.stride(0), float(scale), int(max_seq_len), _ptr(alibi_slopes), qd, _dt(out),
        _kv_dtype(kv_cache_dtype, _dt(key)), float(kv_scale), float(kv_scale if v_scale is None else v_scale),
        _ptr(ws), ws.numel(), int(partition_tokens), _stream()))


def prefill_units(query_lens: Sequence[int], seq_lens: Sequence[int], per_unit: int, order: str = "sequence"):
    """Cut each sequence's query tokens into runs of up to ``per_unit`` consecutive tokens: int32 rows
    [sequence index, first query row, tokens, position of the first token]; ``order`` is "sequence"
    (sequence by sequence, longest context first inside each) or "rows" (longest context first over the batch)."""
    import numpy as np

    parts, row = [], 0
    for b, (ql, sl) in enumerate(zip(query_lens, seq_lens)):
        if ql < 0 or sl < ql:
            raise _C.VtkvError(_C.EINVAL, f"sequence {b}: {ql} query tokens but {sl} rows")
        j = np.arange(0, ql, per_unit, dtype=np.int32)
        u = np.empty((j.size, 4), np.int32)
        u[:, 0] = b
        u[:, 1] = row + j
        u[:, 2] = np.minimum(per_unit, ql - j)
        u[:, 3] = sl - ql + j
        parts.append(u)
        row += ql
    if not parts:
        return np.empty((0, 4), np.int32)
    units = np.concatenate(parts)
    if order == "rows":
        idx = np.argsort(-(units[:, 2] + units[:, 3]), kind="stable")   # most rows first over the whole batch
    else:
        # Sequence by sequence, most rows first inside a sequence.  The workgroups that run at the same time then
        # read the rows of one or two sequences, which stay in the L2 of the XCD that serves their kv head: with
        # the batch-wide order the kernel fetched every row three times over (8 prompts of 2048 tokens: 618 MB
        # against 201 MB), with this one once (201.5 MB); the time is the same, the rows came from the last-level
        # cache either way.  The short units of the last sequence still close the launch.
        idx = np.lexsort((-(units[:, 2] + units[:, 3]), units[:, 0]))
    return np.ascontiguousarray(units[idx])


def prefill_attention(
    out: torch.Tensor,
    query: torch.Tensor,
    key_cache: Union[int, torch.Tensor],
    value_cache: Union[int, torch.Tensor],
    num_kv_heads: int,
    scale: float,
    query_lens: Sequence[int],
    seq_lens: Sequence[int],
    slot_mapping: torch.Tensor,
    alibi_slopes: Optional[torch.Tensor] = None,
    kv_cache_dtype: str = "auto",
    kv_scale: float = 1.0,
    v_scale: Optional[float] = None,
) -> None:
    """Causal attention of the prompt tokens of a batch over the contiguous ranges, which already
    hold the prompt's rows (``reshape_and_cache`` runs first, vllm/attention/backends/xformers.py:
    301-312).  Stands in for both prompt-run branches of the reference backend (:331-386): a plain
    prompt (``seq_lens[b] == query_lens[b]``) and a prompt chunk behind a cached prefix
    (``seq_lens[b] > query_lens[b]``: the last ``query_lens[b]`` positions are the queries).
    ``query`` / ``out`` are [num_query_tokens, num_heads, head_size], sequences packed in order;
    ``query_lens`` / ``seq_lens`` are host lists; ``slot_mapping`` holds each sequence's slot."""
    _require_cuda(out, query, slot_mapping)
    num_tokens, num_heads, head_size = query.shape
    if not out.is_contiguous() or out.shape != query.shape:
        raise _C.VtkvError(_C.EINVAL, "out must be contiguous and shaped like query")
    if slot_mapping.dtype != torch.int64 or len(query_lens) != len(seq_lens) or sum(query_lens) != num_tokens:
        raise _C.VtkvError(_C.EINVAL, "slot_mapping must be int64 and query_lens must add up to the query rows")
    qd = _dt(query)
    kvd = _kv_dtype(kv_cache_dtype, qd)
    lib = _C.lib()
    per_unit = lib.vtkv_prefill_unit_tokens_for(num_heads, num_kv_heads, head_size, kvd)
    if per_unit <= 0:
        raise _C.VtkvError(_C.EINVAL, f"unsupported head counts {num_heads}/{num_kv_heads} or head size {head_size}")
    units = prefill_units(query_lens, seq_lens, per_unit)
    if len(units) == 0:
        return
    if alibi_slopes is not None:
        alibi_slopes = alibi_slopes.to(device=query.device, dtype=torch.float32)
    # through pinned memory and without waiting: a copy from pageable memory would hold the host until the
    # GPU has caught up with everything queued before it
    units_t = torch.from_numpy(units).pin_memory().to(query.device, non_blocking=True)
    _C.check(lib.vtkv_prefill_attention(
        _ptr(out), _ptr(query), _ptr(key_cache), _ptr(value_cache), _ptr(slot_mapping), _ptr(units_t), len(units),
        num_heads, num_kv_heads, head_size, query.stride(0), float(scale), int(max(seq_lens)), _ptr(alibi_slopes), qd,
        _dt(out), kvd, float(kv_scale), float(kv_scale if v_scale is None else v_scale), _stream()))


def paged_attention_v2(
    out: torch.Tensor,
    exp_sum: Optional[torch.Tensor],
    max_logits: Optional[torch.Tensor],
    tmp_out: Optional[torch.Tensor],
    query: torch.Tensor,
    key_cache: Union[int, torch.Tensor],
    value_cache: Union[int, torch.Tensor],
    num_kv_heads: int,
    scale: float,
    seq_lens: torch.Tensor,
    block_size: int,
    max_seq_len: int,
    alibi_slopes: Optional[torch.Tensor],
    kv_cache_dtype: str,
    kv_scale: float,
    slot_mapping: torch.Tensor,
    v_scale: Optional[float] = None,
) -> None:
    """Split-K entry with the reference's 512-row partitions (csrc/attention/attention_kernels.cu:
    451-583,739-914, vllm/attention/ops/paged_attn.py:139-166).  With the caller's per-partition buffers
    (``exp_sum`` / ``max_logits`` float32 [num_seqs, num_heads, P], ``tmp_out`` [num_seqs, num_heads, P,
    head_size] of the query's dtype, P >= ceil(max_seq_len / 512)) every (sequence, kv head, partition)
    is one workgroup and the buffers are filled as the reference fills them; ``out`` is merged from fp32
    partials.  Without them (all three None) the same rows are cut into 512-row spans of the library's own
    scratch."""
    given = [t is not None for t in (exp_sum, max_logits, tmp_out)]
    if not any(given):
        return paged_attention_v1(out, query, key_cache, value_cache, num_kv_heads, scale, seq_lens, block_size,
                                  max_seq_len, alibi_slopes, kv_cache_dtype, kv_scale, slot_mapping, v_scale,
                                  partition_tokens=_PARTITION_SIZE)
    if not all(given):
        raise _C.VtkvError(_C.EINVAL, "exp_sum, max_logits and tmp_out come together or not at all")
    if block_size != 1:
        raise _C.VtkvError(_C.EINVAL, f"Unsupported block size: {block_size} (contiguous ranges use 1)")
    _require_cuda(out, exp_sum, max_logits, tmp_out, query, seq_lens, slot_mapping)
    num_seqs, num_heads, head_size = query.shape
    if seq_lens.dtype != torch.int32 or slot_mapping.dtype != torch.int64:
        raise _C.VtkvError(_C.EINVAL, "seq_lens must be int32 and slot_mapping int64")
    parts = exp_sum.shape[-1] if exp_sum.dim() == 3 else -1
    if (exp_sum.dtype != torch.float32 or max_logits.dtype != torch.float32 or tmp_out.dtype != query.dtype
            or tuple(exp_sum.shape) != (num_seqs, num_heads, parts) or max_logits.shape != exp_sum.shape
            or tuple(tmp_out.shape) != (num_seqs, num_heads, parts, head_size)
            or not (out.is_contiguous() and exp_sum.is_contiguous() and max_logits.is_contiguous()
                    and tmp_out.is_contiguous())):
        raise _C.VtkvError(_C.EINVAL, "exp_sum / max_logits must be contiguous float32 [num_seqs, num_heads, P] and "
                                      "tmp_out [num_seqs, num_heads, P, head_size] of the query's dtype")
    qd = _dt(query)
    lib = _C.lib()
    ws = _workspace(lib.vtkv_decode_attention_v2_workspace_bytes(num_seqs, num_heads, head_size, parts), query.device)
    if alibi_slopes is not None:
        alibi_slopes = alibi_slopes.to(device=query.device, dtype=torch.float32)
    _C.check(lib.vtkv_decode_attention_v2(
        _ptr(out), _ptr(exp_sum), _ptr(max_logits), _ptr(tmp_out), _ptr(query), _ptr(key_cache), _ptr(value_cache),
        _ptr(slot_mapping), _ptr(seq_lens), num_seqs, num_heads, num_kv_heads, head_size, query.stride(0),
        float(scale), int(max_seq_len), int(parts), _ptr(alibi_slopes), qd, _dt(out), _kv_dtype(kv_cache_dtype, qd),
        float(kv_scale), float(kv_scale if v_scale is None else v_scale), _ptr(ws), ws.numel(), _stream()))


# --------------------------------------------------------------------------------------- cache ops
def reshape_and_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: Union[int, torch.Tensor],
    value_cache: Union[int, torch.Tensor],
    slot_m: torch.Tensor,
    slot_mapping: torch.Tensor,
    seq_lens: Optional[torch.Tensor],
    cache_seq_lens: Optional[torch.Tensor],
    max_seq_len: int,
    num_kv_heads: int,
    head_size: int,
    kv_cache_dtype: str = "auto",
    k_scale: float = 1.0,
    v_scale: float = 1.0,
) -> None:
    """vTensor scatter (vllm/_custom_ops.py:238-252): ``key_cache`` / ``value_cache`` are
    int64 device tensors of per-slot base addresses, ``slot_m`` the byte offset of each
    sequence's next row, ``slot_mapping`` its slot."""
    _require_cuda(key, value, slot_m, slot_mapping)
    if slot_m.dtype != torch.int64 or slot_mapping.dtype != torch.int64:
        raise _C.VtkvError(_C.EINVAL, "slot_m and slot_mapping must be int64")
    for t in (seq_lens, cache_seq_lens):
        if t is not None and t.dtype != torch.int32:
            raise _C.VtkvError(_C.EINVAL, "seq_lens and cache_seq_lens must be int32")
    key = key.view(-1, num_kv_heads, head_size)
    value = value.view(-1, num_kv_heads, head_size)
    if key.stride(2) != 1 or key.stride(1) != head_size or value.stride(2) != 1 or value.stride(1) != head_size:
        raise _C.VtkvError(_C.EINVAL, "key/value rows must be contiguous in (head, dim)")
    sd = _dt(key)
    _C.check(_C.lib().vtkv_reshape_and_cache(
        _ptr(key), _ptr(value), _ptr(key_cache), _ptr(value_cache), _ptr(slot_m), _ptr(slot_mapping),
        _ptr(seq_lens), _ptr(cache_seq_lens), slot_mapping.shape[0], int(max_seq_len), num_kv_heads, head_size,
        key.stride(0), value.stride(0), sd, _kv_dtype(kv_cache_dtype, sd), float(k_scale), float(v_scale),
        _stream()))


def reshape_and_cache_paged(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    kv_cache_dtype: str = "auto",
    kv_scale: float = 1.0,
) -> None:
    """Upstream 7-argument form (tests/kernels/test_cache.py:161): K cache
    [num_blocks, H, D/x, block_size, x], V cache [num_blocks, H, D, block_size]."""
    if kv_cache_dtype != "auto" or kv_scale != 1.0:
        raise _C.VtkvError(_C.EINVAL, "the paged layout is kept for unquantised caches only")
    _require_cuda(key, value, key_cache, value_cache, slot_mapping)
    num_tokens, num_heads, head_size = key.shape
    block_size = key_cache.shape[3]
    _C.check(_C.lib().vtkv_reshape_and_cache_paged(
        _ptr(key), _ptr(value), _ptr(key_cache), _ptr(value_cache), _ptr(slot_mapping), num_tokens, num_heads,
        head_size, block_size, key.stride(0), value.stride(0), key.element_size(), _stream()))


def reshape_and_cache_flash(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    kv_cache_dtype: str,
) -> None:
    """vllm/_custom_ops.py:255-264: K and V caches [num_blocks, block_size, H, D]; "auto" caches only
    (csrc/cache_kernels.cu:307-310)."""
    if kv_cache_dtype != "auto":
        raise _C.VtkvError(_C.EINVAL, f"Unsupported data type of kv cache: {kv_cache_dtype}")
    _require_cuda(key, value, key_cache, value_cache, slot_mapping)
    num_tokens, num_heads, head_size = key.shape
    if key_cache.stride(0) != value_cache.stride(0):
        raise _C.VtkvError(_C.EINVAL, "key_cache and value_cache differ in their block stride")
    if key.stride(1) != head_size or key.stride(2) != 1 or value.stride(1) != head_size or value.stride(2) != 1:
        raise _C.VtkvError(_C.EINVAL, "key/value rows must be contiguous in (head, dim)")
    _C.check(_C.lib().vtkv_reshape_and_cache_flash(
        _ptr(key), _ptr(value), _ptr(key_cache), _ptr(value_cache), _ptr(slot_mapping), num_tokens, num_heads,
        head_size, key_cache.shape[1], key_cache.stride(0), key.stride(0), value.stride(0), key.element_size(),
        _stream()))


def copy_blocks(key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                block_mapping: torch.Tensor) -> None:
    """vllm/_custom_ops.py:266-268; block_mapping is an int64 [num_pairs, 2] GPU tensor."""
    n = len(key_caches)
    if n != len(value_caches):
        raise _C.VtkvError(_C.EINVAL, "key_caches and value_caches differ in length")
    if n == 0:
        return
    _require_cuda(block_mapping, *key_caches, *value_caches)
    block_mapping = block_mapping.contiguous()
    kp = (C.c_uint64 * n)(*[t.data_ptr() for t in key_caches])
    vp = (C.c_uint64 * n)(*[t.data_ptr() for t in value_caches])
    block_bytes = key_caches[0][0].numel() * key_caches[0].element_size()
    _C.check(_C.lib().vtkv_copy_blocks(kp, vp, n, _ptr(block_mapping), block_mapping.shape[0], block_bytes,
                                       _stream()))


def swap_blocks(src: torch.Tensor, dst: torch.Tensor, block_mapping: torch.Tensor) -> None:
    """vllm/_custom_ops.py:271-273; block_mapping must be a CPU int64 [n, 2] tensor
    (csrc/cache_kernels.cu:47)."""
    if block_mapping.device.type != "cpu":
        raise _C.VtkvError(_C.EINVAL, "block_mapping must be on CPU")
    if src.is_cuda and dst.is_cuda:
        if src.device != dst.device:
            raise _C.VtkvError(_C.EINVAL, "src and dst must be on the same GPU")
        direction = _C.D2D
    elif src.is_cuda and not dst.is_cuda:
        direction = _C.D2H
    elif not src.is_cuda and dst.is_cuda:
        direction = _C.H2D
    else:
        raise _C.VtkvError(_C.EINVAL, "Invalid device combination")
    mapping = block_mapping.to(torch.int64).contiguous()
    block_bytes = src[0].numel() * src.element_size()
    _C.check(_C.lib().vtkv_swap_blocks(_ptr(src), _ptr(dst), block_bytes, _ptr(mapping), mapping.shape[0],
                                       direction, _stream()))


def swap_ranges(src: Sequence[int], dst: Sequence[int], nbytes: Sequence[int], direction: str,
                piece_bytes: int = 0, num_streams: int = 0) -> None:
    """Move whole byte ranges (a sequence's mapped K or V range) between the GPU and pinned
    host memory; direction is "out" (GPU->host), "in" (host->GPU) or "d2d"."""
    n = len(src)
    if not (n == len(dst) == len(nbytes)):
        raise _C.VtkvError(_C.EINVAL, "src, dst and nbytes differ in length")
    kind = {"out": _C.D2H, "in": _C.H2D, "d2d": _C.D2D}[direction]
    s = (C.c_uint64 * n)(*src)
    d = (C.c_uint64 * n)(*dst)
    b = (C.c_int64 * n)(*nbytes)
    _C.check(_C.lib().vtkv_swap_ranges(s, d, b, n, kind, int(piece_bytes), int(num_streams), _stream()))


def convert_fp8(output: torch.Tensor, input: torch.Tensor, scale: float = 1.0, kv_dtype: str = "fp8") -> None:
    """vllm/_custom_ops.py:276-281: the 1-byte side is fp8 e4m3fn, direction from the dtypes."""
    if kv_dtype not in ("fp8", "fp8_e4m3", "auto"):
        raise _C.VtkvError(_C.EINVAL, f"Unsupported data type: {kv_dtype}")
    _require_cuda(output, input)
    if not (output.is_contiguous() and input.is_contiguous()) or output.numel() != input.numel():
        raise _C.VtkvError(_C.EINVAL, "convert_fp8 needs contiguous tensors of equal size")
    to_fp8 = output.element_size() == 1
    wide = input if to_fp8 else output
    if (input if not to_fp8 else output).element_size() != 1 or wide.element_size() == 1:
        raise _C.VtkvError(_C.EINVAL, "exactly one side must be a 1-byte fp8 tensor")
    _C.check(_C.lib().vtkv_convert_fp8(_ptr(output), _ptr(input), input.numel(), float(scale), int(to_fp8),
                                       _dt(wide), _stream()))
