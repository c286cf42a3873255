"""KV cache owner for the vTensor layout: one address-range segment per sequence slot, per-layer
pointer tables, and the host arena that swapped-out sequences live in.

Counterpart of the reference's ``CacheEngine`` (vllm/worker/cache_engine.py:19-142), taking plain
sizes instead of vLLM config objects.  Swap works on whole sequences: the reference's block-wise
``swap_in/swap_out`` (:131-139) is vestigial for vTensor (its ``gpu_cache`` holds pointer
tables, not tensors, and it runs with zero CPU blocks), so the unit here is "the used bytes of a
slot's K and V ranges in every layer", moved with chunked multi-stream copies.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import _C, _custom_ops as ops, vmm_allocator as vmm



def _dtype_size(dtype: torch.dtype) -> int:
    return torch.tensor([], dtype=dtype).element_size()


class _HostArena:
    """First-fit allocator over one pinned host buffer."""

    def __init__(self, nbytes: int):
        self.nbytes = nbytes
        self.base = int(_C.check_ptr(_C.lib().vtkv_host_alloc(nbytes), "pinned host arena")) if nbytes > 0 else 0
        self.free: List[Tuple[int, int]] = [(0, nbytes)] if nbytes > 0 else []

    def alloc(self, n: int) -> int:
        n = (n + 255) // 256 * 256
        for i, (off, size) in enumerate(self.free):
            if size >= n:
                if size == n:
                    self.free.pop(i)
                else:
                    self.free[i] = (off + n, size - n)
                return off
        raise _C.VtkvOutOfChunks(_C.ENOMEM, f"host swap arena exhausted: need {n} bytes")

    def release(self, off: int, n: int) -> None:
        n = (n + 255) // 256 * 256
        self.free.append((off, n))
        self.free.sort()
        merged: List[Tuple[int, int]] = []
        for o, s in self.free:
            if merged and merged[-1][0] + merged[-1][1] == o:
                merged[-1] = (merged[-1][0], merged[-1][1] + s)
            else:
                merged.append((o, s))
        self.free = merged

    def close(self) -> None:
        if self.base:
            _C.check(_C.lib().vtkv_host_free(C.c_void_p(self.base)))
            self.base = 0


class CacheEngine:
    def __init__(self, num_layers: int, num_kv_heads: int, head_size: int, dtype: torch.dtype, max_num_seqs: int,
                 max_num_batched_tokens: int, cache_seqs: int = 0, cache_tokens: int = 0,
                 swap_space_bytes: int = 0, device: int = 0, value_skew: int = 256) -> None:
        self.num_layers = num_layers
        self.num_kv_heads = num_kv_heads
        self.head_size = head_size
        self.dtype = dtype
        self.device = device
        self.token_size = num_kv_heads * head_size * _dtype_size(dtype)  # bytes of one K (or V) row
        # cache_engine.py:53-57: every slot reserves room for max_num_batched_tokens rows
        # (plus the bytes by which the V rows are set off from the base of their range)
        self.value_skew = int(value_skew)
        ctx = max_num_batched_tokens * self.token_size + self.value_skew
        gran = self.chunk_bytes = vmm.chunkBytes()  # 2 MiB (cache_engine.py:54) unless the pool was given larger chunks
        self.max_context_size = gran * ((ctx + gran - 1) // gran)
        self.kv_batch_stride = self.max_context_size
        # cache_engine.py:58-71: the first cache_seqs slots keep cache_tokens chunks mapped
        keep = gran * cache_tokens if cache_seqs > 0 else 0
        self.vmm_kvcache_segment = [
            vmm.KVcacheSegment(num_layers, self.max_context_size, keep, cache_seqs > 0 and i < cache_seqs)
            for i in range(max_num_seqs)
        ]
        if self.value_skew:  # before any pointer is fetched
            for seg in self.vmm_kvcache_segment:
                seg.set_value_skew(self.value_skew)
        # cache_engine.py:111-129: per layer one pointer table for K and one for V
        self.kv_cache_dtype = "fp8" if _dtype_size(dtype) == 1 else "auto"
        self.gpu_cache = [(vmm.KV_cache(max_num_seqs, l, self.kv_cache_dtype),
                           vmm.KV_cache(max_num_seqs, l, self.kv_cache_dtype)) for l in range(num_layers)]
        vmm.copy_kv_cache([k.kv_cache for k, _ in self.gpu_cache], [v.kv_cache for _, v in self.gpu_cache],
                          self.vmm_kvcache_segment)
        # cache_engine.py:98-109: the same pointers as int64 device tensors, one per layer
        self.k_cache_ptr: List[torch.Tensor] = []
        self.v_cache_ptr: List[torch.Tensor] = []
        dev = torch.device("cuda", device)
        for l in range(num_layers):
            self.k_cache_ptr.append(torch.tensor([s.getKeyDevicePtr(l) for s in self.vmm_kvcache_segment],
                                                 dtype=torch.long, device=dev))
            self.v_cache_ptr.append(torch.tensor([s.getValueDevicePtr(l) for s in self.vmm_kvcache_segment],
                                                 dtype=torch.long, device=dev))
        self._arena = _HostArena(swap_space_bytes)
        self.swap_in_map_bytes = 32 << 20     # swap_in maps this much of every range, queues its copies, maps on
        self.swap_in_flush_bytes = 64 << 20   # ... and hands the queued copies over when they add up to this
        self._swapped: Dict[int, Tuple[int, int]] = {}  # slot -> (arena offset, used bytes per range)

    # ------------------------------------------------------------------ swap (whole sequences)
    def swap_out(self, slots: Sequence[int], keys: Optional[Sequence] = None) -> int:
        """Copy the used part of every K and V range of `slots` to pinned host memory on the current
        stream, then unmap the slots (their chunks return to the pool).  Returns bytes moved.
        `keys` name the saved sequences (by default the slot numbers): with keys of its own a sequence can
        come back into another slot while its old one serves someone else."""
        src, dst, nbytes = [], [], []
        total = 0
        keys = list(slots) if keys is None else list(keys)
        if len(set(slots)) != len(slots) or len(keys) != len(slots) or len(set(keys)) != len(keys):
            raise _C.VtkvError(_C.EINVAL, "swap_out: a slot or a key is listed twice, or keys and slots differ in number")
        for key in keys:
            if key in self._swapped:
                raise _C.VtkvError(_C.ESTATE, f"sequence {key} is already swapped out")
        # room for all of them first: a full arena must leave every slot as it was
        placed: List[Tuple[int, int, int]] = []
        try:
            for slot in slots:
                used = self.vmm_kvcache_segment[slot].used_size
                placed.append((slot, self._arena.alloc(2 * self.num_layers * used) if used else 0, used))
        except _C.VtkvError:
            for _, off, used in placed:
                if used:
                    self._arena.release(off, 2 * self.num_layers * used)
            raise
        for (slot, off, used), key in zip(placed, keys):
            seg = self.vmm_kvcache_segment[slot]
            self._swapped[key] = (off, used)
            for l in range(self.num_layers):
                for which, base in ((0, seg.getKeyDevicePtr(l)), (1, seg.getValueDevicePtr(l))):
                    if used:
                        src.append(base)
                        dst.append(self._arena.base + off + (2 * l + which) * used)
                        nbytes.append(used)
                        total += used
        ops.swap_ranges(src, dst, nbytes, "out")
        # the copies must have read the ranges before their chunks go back to the pool
        torch.cuda.current_stream().synchronize()
        for slot in slots:
            self.vmm_kvcache_segment[slot].preempt_seq(slot)
        return total

    def swap_in(self, slots: Sequence[int], keys: Optional[Sequence] = None) -> int:
        """Map chunks for `slots` again and copy the KV saved under `keys` (by default the slot numbers) back
        from host memory; a slot that receives another slot's sequence must hold no rows.
        Mapping and copying take turns on the host and overlap on the device: the ranges are mapped
        ``swap_in_map_bytes`` at a time, and the copies into what is mapped are handed over (one asynchronous
        call) whenever ``swap_in_flush_bytes`` are queued, so they run while the host maps on.  Mapping a chunk
        takes about as long as copying it (42 us against 38 us), so a swap-in of unmapped sequences stays bound
        by the mapping: 32 to 34 GB/s for one 347 MB sequence against 27 GB/s with everything mapped first.
        The overlap needs the current stream to be a non-blocking one: this runtime's mapping calls wait for
        everything queued on the null stream, the copies included, and the two then run one after the other."""
        total = 0
        keys = list(slots) if keys is None else list(keys)
        if len(keys) != len(slots):
            raise _C.VtkvError(_C.EINVAL, "swap_in: keys and slots differ in number")
        for key in keys:
            if key not in self._swapped:
                raise _C.VtkvError(_C.ESTATE, f"sequence {key} is not swapped out")
        try:
            total = self._swap_in_copies(slots, keys)
        except Exception:
            # (the pool ran dry part of the way, most likely) the sequences stay swapped out, whole: copies already
            # queued finish, and every slot of this call gives back what was mapped for it
            torch.cuda.current_stream().synchronize()
            for slot in slots:
                self.vmm_kvcache_segment[slot].preempt_seq(slot)
            raise
        torch.cuda.current_stream().synchronize()  # the arena space is reused after this
        for key in keys:
            off, used = self._swapped.pop(key)
            if used:
                self._arena.release(off, 2 * self.num_layers * used)
        return total

    def _swap_in_copies(self, slots: Sequence[int], keys: Sequence) -> int:
        total = 0
        src, dst, nbytes, queued = [], [], [], 0
        step = max(1, self.swap_in_map_bytes // self.chunk_bytes)   # chunks per range mapped between two rounds of copies
        for slot, key in zip(slots, keys):
            off, used = self._swapped[key]
            seg = self.vmm_kvcache_segment[slot]
            if not used:
                seg.set_used_size(0)
                continue
            # the V rows start value_skew bytes into their range, so that much more must be mapped
            need = (used + self.value_skew + self.chunk_bytes - 1) // self.chunk_bytes
            mapped = seg.actual_size // self.chunk_bytes
            ptrs = [(seg.getKeyDevicePtr(l), seg.getValueDevicePtr(l)) for l in range(self.num_layers)]
            done_k = done_v = 0
            while True:
                if mapped < need:
                    grow = min(step, need - mapped)
                    seg.expandMultiSegment(grow)
                    mapped += grow
                ready_k = min(used, mapped * self.chunk_bytes)
                ready_v = min(used, max(0, mapped * self.chunk_bytes - self.value_skew))
                for l, (kp, vp) in enumerate(ptrs):
                    for which, base, lo, hi in ((0, kp, done_k, ready_k), (1, vp, done_v, ready_v)):
                        if hi > lo:
                            src.append(self._arena.base + off + (2 * l + which) * used + lo)
                            dst.append(base + lo)
                            nbytes.append(hi - lo)
                            total += hi - lo
                            queued += hi - lo
                done_k, done_v = ready_k, ready_v
                if queued >= self.swap_in_flush_bytes:
                    ops.swap_ranges(src, dst, nbytes, "in")
                    src, dst, nbytes, queued = [], [], [], 0
                if mapped >= need:
                    break
            seg.set_used_size(used)
        if src:
            ops.swap_ranges(src, dst, nbytes, "in")
        return total

    # ------------------------------------------------------------------ block-wise API of the reference
    def copy(self, src_to_dsts: torch.Tensor) -> None:
        raise NotImplementedError("block copies have no meaning for per-sequence contiguous ranges; "
                                  "use _custom_ops.copy_blocks on paged tensors")

    @staticmethod
    def get_cache_block_size(block_size: int, num_kv_heads: int, head_size: int, num_layers: int,
                             dtype: torch.dtype) -> int:
        # cache_engine.py:144-162
        return _dtype_size(dtype) * num_layers * 2 * block_size * num_kv_heads * head_size

    def close(self) -> None:
        for seg in self.vmm_kvcache_segment:
            seg.destroy()
        for k, v in self.gpu_cache:
            k.kv_cache.destroy()
            v.kv_cache.destroy()
        self._arena.close()
