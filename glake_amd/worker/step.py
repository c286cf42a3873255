"""Per-step vTensor bookkeeping that the reference does at the top of ``LlamaModel.forward``
(vllm/model_executor/models/llama.py:307-341): advance every scheduled sequence's range, map a
chunk where a sequence crosses a 2 MiB boundary, and hand the byte offsets to the kernels."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .. import vmm_allocator as vmm


def kv_row_bytes(num_kv_heads: int, head_size: int, kv_cache_dtype: str = "auto", model_elem_bytes: int = 2) -> int:
    """Bytes of one K (or V) row of one token in a sequence's range: one byte per element for an fp8 cache,
    otherwise the model's element size (the reference hard-codes 2, llama.py:315)."""
    elem = 1 if kv_cache_dtype in ("fp8", "fp8_e4m3") else int(model_elem_bytes)
    return int(num_kv_heads) * int(head_size) * elem


def prepare_step(attn_metadata, kv_caches: Sequence, kv_cache_dtype: Optional[str] = None,
                 model_elem_bytes: int = 2) -> None:
    """Fills ``attn_metadata.slot_m`` (and ``decode_seq_len``, ``query_lens_tensor``, ``cache_seq_lens``)
    for this step.

    kv_caches: per layer a (K, V) pair of ``KV_cache`` handles, or None entries during profiling.
    kv_cache_dtype: "auto" (rows of the model's element size) or "fp8" (one byte per element); by default
    what the ``CacheEngine`` that made the handles says (``KV_cache.kv_cache_dtype``), else "auto".

    The batch holds ``num_prefills`` prompts first, then the decode sequences (one new row each).  A prompt
    writes ``query_lens[i]`` rows when ``attn_metadata.query_lens`` is given (a prompt, or a chunk of one, behind
    rows that are already cached: ``seq_lens[i]`` then counts the cached rows too), otherwise ``seq_lens[i]``.
    """
    if not kv_caches or kv_caches[0] is None:
        return
    k_cache = [k.kv_cache for k, _ in kv_caches]
    v_cache = [v.kv_cache for _, v in kv_caches]
    if kv_cache_dtype is None:
        kv_cache_dtype = getattr(kv_caches[0][0], "kv_cache_dtype", "auto")
    kv_size = kv_row_bytes(attn_metadata.kv_num_heads, attn_metadata.kv_head_size, kv_cache_dtype,
                           model_elem_bytes)  # llama.py:315
    n = len(attn_metadata.slot_mapping_list)
    n_pre = attn_metadata.num_prefills
    device = attn_metadata.slot_mapping.device
    segs = attn_metadata.kvcache_segment
    slots = attn_metadata.slot_mapping_list
    used = attn_metadata.set_used_size
    slot_m: List[int] = []
    if n_pre > 0:
        rows = list(attn_metadata.query_lens[:n_pre]) if attn_metadata.query_lens is not None \
            else list(attn_metadata.seq_lens[:n_pre])
        kv_size_list: List[int] = [r * kv_size for r in rows]  # llama.py:318-320
        slot_m += vmm.extend_kv_cache_batch(k_cache, v_cache, slots[:n_pre], kv_size_list, segs[:n_pre],
                                            used[:n_pre], kv_size, False)  # llama.py:340, prompt form
        if attn_metadata.query_lens is not None:
            attn_metadata.query_lens_tensor = torch.tensor(rows, dtype=torch.int32, device=device)
        if attn_metadata.query_lens is not None or attn_metadata.cache_seq_lens is None:
            # where each prompt's rows start in the packed key/value tensors (the reference's cache_seq_lens,
            # model_runner.py:366-370, which it builds from seq_lens: right only without cached rows)
            starts = [0] * n_pre
            for i in range(1, n_pre):
                starts[i] = starts[i - 1] + rows[i - 1]
            attn_metadata.cache_seq_lens = torch.tensor(starts, dtype=torch.int32, device=device)
    decode_seq_len = None
    if n > n_pre:
        # llama.py:321-337: the reference spins on its background mapper here and then queues
        # eagerExtend requests; here a row that needs a chunk which is still being mapped waits inside
        # extend_kv_cache_batch, so only the requests remain
        nd = n - n_pre
        decode_seq_len = torch.ones(nd, dtype=torch.int32, device=device)
        ext = attn_metadata.extend_seq_list or []
        for idx, slot_id in enumerate(ext):
            if slot_id != -1 and idx >= n_pre:
                segs[idx].eagerExtend(kv_size, slot_id)
        try:
            slot_m += vmm.extend_kv_cache_batch(k_cache, v_cache, slots[n_pre:], [kv_size] * nd, segs[n_pre:],
                                                used[n_pre:], kv_size, True)  # llama.py:340, decode form
        except Exception:
            # the step did not happen: the prompts' rows are given back too (the decode half has undone itself)
            for seg, before in zip(segs[:n_pre], slot_m):
                seg.set_used_size(before)
            raise
    attn_metadata.decode_seq_len = decode_seq_len
    attn_metadata.slot_m = torch.tensor(slot_m, dtype=torch.int64, device=device)
    # The decode sequences' lengths for the fused append + attention launch, which takes up to 512 of them with
    # its kernel arguments (model_runner.py:607 hands the lengths over on the host as well as on the device).
    # Made here, once per step and for all layers, from this step's seq_lens; not for a step that is recorded
    # into a graph, whose replays must read the lengths of their own step from the device.
    host_lens = None
    seq_lens = attn_metadata.seq_lens
    if (n > n_pre and seq_lens is not None and len(seq_lens) == n and n - n_pre <= 512
            and not getattr(attn_metadata, "use_cuda_graph", False)):
        import ctypes

        host_lens = (ctypes.c_int32 * (n - n_pre))(*seq_lens[n_pre:])
    if hasattr(attn_metadata, "_host_decode_lens"):
        attn_metadata._host_decode_lens = host_lens


class DecodeStepPlan:
    """One decode step of one layer for a fixed set of sequences, with the per-step host work cut down.

    ``run`` does what the reference does per step and layer through separate Python calls
    (vllm/model_executor/models/llama.py:307-341 then vllm/attention/backends/xformers.py:301-371):
    advance each sequence's range by one token row (mapping a chunk at a 2 MiB boundary), upload the
    byte offsets and the new sequence lengths, append the step's K/V rows and run decode attention
    over the whole context.  The same C entry points are used as by the separate ops
    (``vtkv_extend_kv_cache_batch``, ``vtkv_reshape_and_cache``, ``vtkv_decode_attention``); what the
    plan saves is per-call Python: argument arrays, the device tables and the pinned staging ring are
    made once, the bookkeeping writes its offsets straight into pinned memory, and both metadata arrays
    travel in one asynchronous copy.  With ``fused=True`` (bf16 or fp8 cache) the append and the attention
    are one launch (``vtkv_decode_append_attention``) and, up to 512 sequences, the lengths travel with the
    kernel arguments, so a step is two kernels (attention and its merge) and no copy.  Build a new plan
    when the set of running sequences changes.  ``run`` does host-side bookkeeping every step and hands the lengths
    over by value: it is not something to record into a HIP graph (a captured step calls the separate
    operators with device-side lengths).
    """

    def __init__(self, segments: Sequence, slot_ids: Sequence[int], key_cache, value_cache, num_heads: int,
                 num_kv_heads: int, head_size: int, scale: float, kv_cache_dtype: str = "auto", k_scale: float = 1.0,
                 v_scale: float = 1.0, model_dtype: torch.dtype = torch.bfloat16, device=None, ring: int = 128,
                 fused: bool = True, map_ahead_rows: int = 64):
        import ctypes as C

        import numpy as np

        from .. import _C, _custom_ops as ops

        if len(segments) != len(slot_ids) or not segments:
            raise _C.VtkvError(_C.EINVAL, "DecodeStepPlan: one slot id per segment, at least one sequence")
        if ring < 2 or ring % 2:
            raise _C.VtkvError(_C.EINVAL, "DecodeStepPlan: ring must be even and at least 2")
        if model_dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise _C.VtkvError(_C.EINVAL, f"DecodeStepPlan: the attention kernels take bfloat16, float16 and float32 "
                                          f"queries, not {model_dtype}")
        self._C, self._lib, self._np = _C, _C.lib(), np
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        n = self.n = len(segments)
        self.num_heads, self.num_kv_heads, self.head_size = int(num_heads), int(num_kv_heads), int(head_size)
        self.scale = float(scale)
        self._src_dt = ops._DTYPES[model_dtype]
        self._kv_dt = ops._kv_dtype(kv_cache_dtype, self._src_dt)
        self.k_scale, self.v_scale = float(k_scale), float(v_scale)
        self.kv_size = self.num_kv_heads * self.head_size * {_C.FP8_E4M3: 1, _C.F32: 4}.get(self._kv_dt, 2)  # bytes per row
        self._segments = list(segments)  # keeps the handles alive
        self._segs = (C.c_void_p * n)(*[s._h for s in segments])
        self._tok = (C.c_int64 * n)(*([self.kv_size] * n))
        self._k_table, self._v_table = ops._ptr(key_cache), ops._ptr(value_cache)
        self._tables = (key_cache, value_cache)
        self._slot_t = torch.tensor(list(slot_ids), dtype=torch.int64, device=self.device)
        self._slot_p = C.c_void_p(self._slot_t.data_ptr())
        # per step: n int64 byte offsets then n int32 lengths; a ring of pinned rows, guarded by one event
        # per half so that a row is rewritten only after its previous upload has run
        self._ring = ring
        self._stage = torch.empty(ring, 3 * n, dtype=torch.int32).pin_memory()
        stage_np = self._stage.numpy()
        self._offs = [stage_np[i, :2 * n].view(np.int64) for i in range(ring)]
        self._lens = [stage_np[i, 2 * n:] for i in range(ring)]
        self._row_p = [C.c_void_p(self._stage[i].data_ptr()) for i in range(ring)]
        self._meta = torch.empty(3 * n, dtype=torch.int32, device=self.device)
        self._meta_addr = self._meta.data_ptr()
        self._offs_p = C.c_void_p(self._meta_addr)
        self._lens_p = C.c_void_p(self._meta_addr + 8 * n)
        self._events = [torch.cuda.Event(), torch.cuda.Event()]
        self._recorded = [False, False]
        self._row = 0
        # Every 16th step the sequences that have come within `map_ahead_rows` rows of the end of what is mapped
        # are announced to the map-ahead worker (what the scheduler's extend_seq_list does for an engine), so
        # that no step maps a chunk in the calling thread: a synchronous mapping costs 0.1 ms, which an empty
        # launch queue (the first steps after a wait) passes on to the GPU.  0 switches it off.
        self._ahead_bytes = int(map_ahead_rows) * self.kv_size
        self._steps = 0
        need = self._lib.vtkv_decode_attention_workspace_bytes(n, self.num_heads, self.head_size, 1, 0)
        # its own scratch (zero-filled once, as the library asks): plans may run on different streams at once
        self._ws = torch.zeros(max(int(need), 1 << 20), dtype=torch.uint8, device=self.device)
        self._ws_p, self._ws_n = C.c_void_p(self._ws.data_ptr()), self._ws.numel()
        self.seq_lens = None  # numpy view of the last step's lengths (valid until the ring wraps)
        # one launch per step: any cache type at head size 128; 16-bit caches at the other head sizes
        self.fused = bool(fused) and self._src_dt != _C.F32 and (self.head_size == 128 or self._kv_dt == self._src_dt)
        self._inline = self.fused and n <= 512
        self._host_lens_p = [C.c_void_p(self._stage[i].data_ptr() + 8 * n) for i in range(ring)]

    def run(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, out: torch.Tensor,
            alibi_slopes=None) -> int:
        """query [n, num_heads, head_size]; key/value [n, num_kv_heads*head_size] (or 3-d), the step's new
        rows; out like query (or float32).  Returns the longest sequence length after the step."""
        C_void_p = type(self._slot_p)
        lib, check, n = self._lib, self._C.check, self.n
        i, half = self._row, self._ring // 2
        if i == 0 or i == half:
            h = 0 if i == 0 else 1
            if self._recorded[h]:
                self._events[h].synchronize()
        if self._ahead_bytes and self._steps % 16 == 0:
            check(lib.vtkv_map_ahead_batch(self._segs, n, self._ahead_bytes))
        self._steps += 1
        check(lib.vtkv_extend_kv_cache_batch(self._segs, n, self._tok, None, self.kv_size, 1, self._row_p[i]))
        lens = self._lens[i]
        self._np.floor_divide(self._offs[i], self.kv_size, out=lens, casting="unsafe")
        lens += 1
        max_len = int(lens.max())
        stream = C_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        self._row = (i + 1) % self._ring
        self.seq_lens = lens
        out_dt = self._C.F32 if out.dtype == torch.float32 else self._src_dt
        alibi_p = None if alibi_slopes is None else C_void_p(alibi_slopes.data_ptr())
        if self._inline:
            # nothing on the GPU reads the staging row: the lengths are copied into the kernel arguments
            check(lib.vtkv_decode_append_attention(
                C_void_p(out.data_ptr()), C_void_p(query.data_ptr()), C_void_p(key.data_ptr()),
                C_void_p(value.data_ptr()), key.stride(0), value.stride(0), self._k_table, self._v_table,
                self._slot_p, None, self._host_lens_p[i], n, self.num_heads, self.num_kv_heads, self.head_size,
                query.stride(0), self.scale, max_len, alibi_p, self._src_dt, out_dt, self._kv_dt, self.k_scale,
                self.v_scale, self._ws_p, self._ws_n, 0, stream))
            return max_len
        check(lib.vtkv_memcpy_h2d_async(self._meta_addr, self._row_p[i], 12 * n, stream))
        if i == half - 1 or i == self._ring - 1:
            h = 0 if i == half - 1 else 1
            self._events[h].record()
            self._recorded[h] = True
        if self.fused:
            check(lib.vtkv_decode_append_attention(
                C_void_p(out.data_ptr()), C_void_p(query.data_ptr()), C_void_p(key.data_ptr()),
                C_void_p(value.data_ptr()), key.stride(0), value.stride(0), self._k_table, self._v_table,
                self._slot_p, self._lens_p, None, n, self.num_heads, self.num_kv_heads, self.head_size,
                query.stride(0), self.scale, max_len, alibi_p, self._src_dt, out_dt, self._kv_dt, self.k_scale,
                self.v_scale, self._ws_p, self._ws_n, 0, stream))
            return max_len
        kstride = key.stride(0)
        vstride = value.stride(0)
        check(lib.vtkv_reshape_and_cache(
            C_void_p(key.data_ptr()), C_void_p(value.data_ptr()), self._k_table, self._v_table, self._offs_p,
            self._slot_p, None, None, n, 1, self.num_kv_heads, self.head_size, kstride, vstride, self._src_dt,
            self._kv_dt, self.k_scale, self.v_scale, stream))
        check(lib.vtkv_decode_attention(
            C_void_p(out.data_ptr()), C_void_p(query.data_ptr()), self._k_table, self._v_table, self._slot_p,
            self._lens_p, n, self.num_heads, self.num_kv_heads, self.head_size, query.stride(0), self.scale, max_len,
            alibi_p, self._src_dt, out_dt, self._kv_dt,
            self.k_scale, self.v_scale, self._ws_p, self._ws_n, 0, stream))
        return max_len
