"""Facade with the names of the reference's ``vmmAllocator`` pybind module
(vmm_allocator/vmm_allocator.h:190-219) and of its ``KV_cache`` wrapper
(vmm_allocator/vmm_allocator.py:5-19), over the HIP virtual-memory pool of ``libvtkv.so``.

Differences a caller can observe, all deliberate:
  * ``eagerExtend`` hands its request to a worker thread that sleeps on a condition variable (the
    reference's thread spins on its queue and signals through POSIX shared memory); a row that needs
    the chunk before the worker is done simply waits inside ``extend_kv_cache_batch``, so the spin
    on ``query_shm`` at llama.py:322-326 is not needed (it still works);
  * growth that was not requested ahead is done by the calling thread inside ``extend_kv_cache_batch``;
  * unmapping is lazy: a released chunk stays mapped ("retired") until another sequence needs it;
  * pool exhaustion raises ``VtkvOutOfChunks`` instead of printing and carrying on
    (vmm_allocator.cpp:232-235,330-333);
  * segments can be destroyed (the reference never frees address ranges).
"""
from __future__ import annotations

import ctypes as C
import sys
from typing import List, Sequence

import numpy as np

from . import _C

granularitySize = 2 * 1024 * 1024  # vmm_allocator.h:45


def chunkBytes() -> int:
    """Bytes of one physical chunk: ``granularitySize`` unless ``set_chunk_bytes`` asked for more."""
    return int(_C.lib().vtkv_chunk_bytes())


def set_chunk_bytes(nbytes: int) -> None:
    """Chunks of ``nbytes`` (a power of two from 2 MiB to 1 GiB) from the next ``init_physical_handle`` on; only
    while the pool is empty.  The reference's granularity is fixed; with this HIP runtime a pool holds at most
    30000 chunks, so a cache above 58 GiB needs larger ones.  No counterpart in the reference."""
    _C.check(_C.lib().vtkv_pool_set_chunk_bytes(int(nbytes)))


def init_physical_handle(num_blocks: int, device_id: int) -> bool:
    """Create ``num_blocks`` physical chunks (2 MiB each by default) on ``device_id`` (vmm_allocator.cpp:113-151)."""
    _C.check(_C.lib().vtkv_pool_init(int(device_id), int(num_blocks)))
    return True


def showFreeBlocks() -> int:
    return int(_C.check(_C.lib().vtkv_pool_free_chunks()))


def totalBlocks() -> int:
    return int(_C.check(_C.lib().vtkv_pool_total_chunks()))


def sharedBlocks() -> int:
    """Physical chunks that are mapped into more than one segment (shared prefixes)."""
    return int(_C.check(_C.lib().vtkv_pool_shared_chunks()))


def recreatedBlocks() -> int:
    """Physical chunks replaced by new ones so far (each after 256 map/unmap cycles)."""
    return int(_C.check(_C.lib().vtkv_pool_recreated_chunks()))


def retiredBlocks() -> int:
    """Free chunks that are still mapped at the top of a shrunken segment (unmapping is lazy)."""
    return int(_C.check(_C.lib().vtkv_pool_retired_chunks()))


def trim(max_chunks: int = -1) -> int:
    """Unmap up to ``max_chunks`` retired chunks now (all by default); returns how many."""
    return int(_C.check(_C.lib().vtkv_pool_trim(int(max_chunks))))


def destroy_pool() -> None:
    _C.check(_C.lib().vtkv_pool_destroy())


class KVcacheSegment:
    """One sequence slot: per layer a K and a V virtual range (vmm_allocator.cpp:177-456)."""

    def __init__(self, layer_num: int, context_max_size: int, expand_size: int, expand: bool):
        self._h = _C.check_ptr(
            _C.lib().vtkv_seg_create(int(layer_num), int(context_max_size), int(expand_size), int(bool(expand))),
            "KVcacheSegment")
        self.layer_num = int(layer_num)
        self.context_max_size = int(context_max_size)
        self.expand_size = int(expand_size)

    # --- pointers
    def getKeyDevicePtr(self, layer_index: int) -> int:
        return int(_C.check_ptr(_C.lib().vtkv_seg_key_ptr(self._h, int(layer_index)), "getKeyDevicePtr"))

    def getValueDevicePtr(self, layer_index: int) -> int:
        return int(_C.check_ptr(_C.lib().vtkv_seg_value_ptr(self._h, int(layer_index)), "getValueDevicePtr"))

    @property
    def value_skew(self) -> int:
        """Bytes between the base of a V range and its first row (0 unless set); ``getValueDevicePtr`` includes
        them and the segment keeps ``used_size + value_skew <= actual_size``.  With 256 the K and the V row
        of a token lie in different memory channels.  No counterpart in the reference."""
        return int(_C.check(_C.lib().vtkv_seg_value_skew(self._h)))

    def set_value_skew(self, nbytes: int) -> None:
        """Set that offset (a multiple of 256 up to 4096); only while the segment holds no rows.  Pointers
        fetched before are stale afterwards."""
        _C.check(_C.lib().vtkv_seg_set_value_skew(self._h, int(nbytes)))

    def ensure_mapped(self, nbytes: int) -> None:
        """Map what ``nbytes`` more bytes per range behind ``used_size`` need, the V offset included
        (``vtkv_seg_ensure``); for callers that write rows through the pointers themselves."""
        _C.check(_C.lib().vtkv_seg_ensure(self._h, int(nbytes)))

    # --- accounting
    def get_used_slot(self) -> int:
        return int(_C.check(_C.lib().vtkv_seg_get_used(self._h)))

    def set_used_size(self, used_size: int) -> None:
        _C.check(_C.lib().vtkv_seg_set_used(self._h, int(used_size)))

    @property
    def used_size(self) -> int:
        return self.get_used_slot()

    @property
    def actual_size(self) -> int:
        return int(_C.check(_C.lib().vtkv_seg_mapped_bytes(self._h)))

    # --- growth / shrink
    def expandMultiSegment(self, expand_num: int) -> bool:
        _C.check(_C.lib().vtkv_seg_expand(self._h, int(expand_num)))
        return True

    def copy_kv_cache(self, token_size: int, kv_size: int) -> None:
        _C.check(_C.lib().vtkv_seg_reserve(self._h, int(token_size), int(kv_size)))

    def eagerExtend(self, token_size: int, seq_id: int) -> None:
        """Ask the map-ahead worker for one more chunk per range and return at once
        (vmm_allocator.cpp:307-320); ``query_shm([seq_id])`` tells when it is there."""
        _eager_segments[int(seq_id)] = self
        _C.check(_C.lib().vtkv_seg_eager_extend(self._h, 1))

    def share_prefix(self, src: "KVcacheSegment", nbytes: int, stream: int = 0) -> None:
        """Begin this (empty) sequence with the first ``nbytes`` bytes of every range of ``src``: whole
        chunks are mapped a second time instead of copied, the partly filled one is copied on ``stream``
        (a raw HIP stream handle, 0 = the null stream)."""
        _C.check(_C.lib().vtkv_seg_share_prefix(self._h, src._h, int(nbytes), C.c_void_p(stream)))

    @property
    def pending(self) -> int:
        """Map-ahead requests of this segment that have not finished."""
        return int(_C.check(_C.lib().vtkv_seg_pending(self._h)))

    def preempt_seq(self, seq_id: int = -1) -> None:
        _C.check(_C.lib().vtkv_seg_preempt(self._h))

    def release_seq(self, seq_id: int = -1) -> None:
        _C.check(_C.lib().vtkv_seg_release(self._h))

    def show_info(self, seq_id: int) -> List[int]:
        # [seq_id, actual_size, used_size, ready flag, cycle] (vmm_allocator.cpp:448-456)
        return [int(seq_id), self.actual_size, self.used_size, 1, 0]

    # --- debugging helpers (vmm_allocator.cpp:423-446), layer 0 K range
    def write_string(self, s: str) -> None:
        data = s.encode()
        used = self.get_used_slot()
        _C.check(_C.lib().vtkv_seg_ensure(self._h, len(data)))
        _C.check(_C.lib().vtkv_memcpy_h2d(self.getKeyDevicePtr(0) + used, data, len(data)))
        self.set_used_size(used + len(data))

    def read_string(self) -> str:
        used = self.get_used_slot()
        buf = C.create_string_buffer(max(used, 1))
        if used:
            _C.check(_C.lib().vtkv_memcpy_d2h(buf, self.getKeyDevicePtr(0), used))
        return buf.raw[:used].decode()

    def destroy(self) -> None:
        if self._h:
            for k in [k for k, v in _eager_segments.items() if v is self]:
                del _eager_segments[k]
            _C.check(_C.lib().vtkv_seg_destroy(self._h))
            self._h = None

    def __del__(self):  # best effort; at interpreter exit the HIP runtime may be gone already, and the
        try:            # process gives everything back anyway
            if not sys.is_finalizing():
                self.destroy()
        except Exception:
            pass


class KVCache:
    """Device array of per-slot base pointers (vmm_allocator.cpp:458-470)."""

    def __init__(self, num_seqs: int):
        self.num_seqs = int(num_seqs)
        self._table = int(_C.check_ptr(_C.lib().vtkv_ptr_table_create(self.num_seqs), "KVCache"))

    def getKVCachePtr(self) -> int:
        return self._table

    def AddKVCache(self, slot: int, kv_cache: int) -> None:
        if not 0 <= slot < self.num_seqs:
            raise _C.VtkvError(_C.EINVAL, f"slot {slot} outside [0, {self.num_seqs})")
        _C.check(_C.lib().vtkv_ptr_table_set(self._table, int(slot), int(kv_cache)))

    def to_numpy(self) -> np.ndarray:
        out = np.zeros(self.num_seqs, np.int64)
        _C.check(_C.lib().vtkv_memcpy_d2h(out.ctypes.data_as(C.c_void_p), self._table, out.nbytes))
        return out

    def destroy(self) -> None:
        if self._table:
            _C.check(_C.lib().vtkv_ptr_table_destroy(self._table))
            self._table = 0

    def __del__(self):
        try:
            if not sys.is_finalizing():
                self.destroy()
        except Exception:
            pass


class KV_cache:
    """Per-layer handle the model code passes around (vmm_allocator/vmm_allocator.py:5-19)."""

    def __init__(self, max_seqs: int, layer_index: int, kv_cache_dtype: str = "auto") -> None:
        self.max_seqs = max_seqs
        self.layer_index = layer_index
        # "auto" (rows of the model's element size) or "fp8" (one byte per element): what the ranges behind this
        # table hold, so that the step prologue can size a row; no counterpart in the reference, whose rows
        # are always two bytes per element (vllm/model_executor/models/llama.py:315)
        self.kv_cache_dtype = kv_cache_dtype
        self.kv_cache = KVCache(self.max_seqs)
        self.vmm_ptr = self.kv_cache.getKVCachePtr()


def _seg_array(segments: Sequence[KVcacheSegment]):
    return (C.c_void_p * len(segments))(*[s._h for s in segments])


def extend_kv_cache_batch(k_cache_batch, v_cache_batch, slot_mapping: Sequence[int], token_size: Sequence[int],
                          segment: Sequence[KVcacheSegment], set_used_size: Sequence[int], kv_size: int,
                          gen: bool) -> List[int]:
    """Per-step bookkeeping (vmm_allocator.h:138-168): returns each sequence's byte offset
    before this step's rows, then advances it.  ``k_cache_batch`` / ``v_cache_batch`` are
    accepted and ignored, as in the reference (its table refresh is commented out)."""
    n = len(slot_mapping)
    if not (len(token_size) == len(segment) == len(set_used_size) == n):
        raise _C.VtkvError(_C.EINVAL, "extend_kv_cache_batch: argument lists differ in length")
    tok = (C.c_int64 * n)(*[int(t) for t in token_size])
    used = (C.c_int64 * n)(*[int(u) for u in set_used_size])
    out = (C.c_int64 * n)()
    _C.check(_C.lib().vtkv_extend_kv_cache_batch(_seg_array(segment), n, tok, used, int(kv_size), int(bool(gen)),
                                                 out))
    return list(out)


def copy_kv_cache(k_cache_batch: Sequence[KVCache], v_cache_batch: Sequence[KVCache],
                  segment: Sequence[KVcacheSegment]) -> None:
    """Fill every layer's K and V pointer table from the segments (vmm_allocator.h:170-182)."""
    segs = _seg_array(segment)
    for layer, (k, v) in enumerate(zip(k_cache_batch, v_cache_batch)):
        _C.check(_C.lib().vtkv_ptr_table_fill(k.getKVCachePtr(), segs, len(segment), layer, 0))
        _C.check(_C.lib().vtkv_ptr_table_fill(v.getKVCachePtr(), segs, len(segment), layer, 1))


# Readiness queries of the reference's background mapper (vmm_allocator.cpp:74-111), answered from the
# segments that eagerExtend was called on under these sequence ids.
_eager_segments = {}


def query_shm(seq_ids: Sequence[int]) -> bool:
    """True when no map-ahead request of these sequences is outstanding."""
    for i in seq_ids:
        seg = _eager_segments.get(int(i))
        if seg is not None and seg._h and seg.pending:
            return False
    return True


def query_cycle(seq_ids: Sequence[int]) -> bool:
    """The reference's "waited long enough, check again" signal; here simply: something is outstanding."""
    return not query_shm(seq_ids)


def map_ahead_batch(segments: Sequence["KVcacheSegment"], ahead_bytes: int) -> int:
    """``eagerExtend`` for every segment whose rows have come within ``ahead_bytes`` of the end of what is mapped,
    that has no request under way and that the pool can serve now (``vtkv_map_ahead_batch``); returns how many
    requests were queued.  No counterpart in the reference, whose scheduler names the sequences one by one."""
    arr = (C.c_void_p * len(segments))(*[s._h for s in segments])
    return int(_C.check(_C.lib().vtkv_map_ahead_batch(arr, len(segments), int(ahead_bytes))))


def wait_map_ahead() -> None:
    """Block until every map-ahead request has been carried out."""
    _C.check(_C.lib().vtkv_map_ahead_wait())


def query_unmap(seq_ids: Sequence[int]) -> List[bool]:
    return [True for _ in seq_ids]


def print_shm_state(seq_ids: Sequence[int]) -> List[int]:
    return [1 for _ in seq_ids]
