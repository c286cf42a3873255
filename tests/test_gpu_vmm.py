"""The HIP virtual-memory chunk pool and per-sequence ranges: integer invariants of the reference's
allocator (vmm_allocator/vmm_allocator.cpp:214-421) plus what it silently gets wrong (pool
exhaustion, growth past the reserved range)."""
import ctypes as C

import numpy as np
import pytest

from kvharness import CHUNK

pytestmark = pytest.mark.gpu


def accounted(vmm, segs):
    mapped = sum(2 * s.layer_num * (s.actual_size // CHUNK) for s in segs)
    return vmm.showFreeBlocks() + mapped


def test_grow_release_preempt_keep_the_books_balanced(gpu_pool):
    vmm = gpu_pool
    free0 = vmm.showFreeBlocks()
    layers = 3
    a = vmm.KVcacheSegment(layers, 8 * CHUNK, 2 * CHUNK, True)    # pre-mapped, keeps 2 chunks on release
    b = vmm.KVcacheSegment(layers, 8 * CHUNK, 0, False)
    assert a.actual_size == 2 * CHUNK and b.actual_size == 0
    assert vmm.showFreeBlocks() == free0 - 2 * layers * 2
    b.expandMultiSegment(3)
    assert accounted(vmm, [a, b]) == free0
    a.expandMultiSegment(4)
    assert a.actual_size == 6 * CHUNK and accounted(vmm, [a, b]) == free0
    a.set_used_size(5 * CHUNK + 17)
    a.release_seq(0)                                               # keeps the first expand_size bytes
    assert a.actual_size == 2 * CHUNK and a.used_size == 0 and accounted(vmm, [a, b]) == free0
    a.release_seq(0)                                               # res == 0: nothing to do (cpp:393-396)
    assert a.actual_size == 2 * CHUNK
    b.release_seq(1)                                               # expand_size 0: everything goes back
    assert b.actual_size == 0
    a.preempt_seq(0)
    assert a.actual_size == 0 and vmm.showFreeBlocks() == free0
    c = vmm.KVcacheSegment(layers, 8 * CHUNK, 4 * CHUNK, False)
    c.expandMultiSegment(1)
    c.release_seq(2)                                               # fewer bytes mapped than expand_size: unmap all (cpp:391-392)
    assert c.actual_size == 0
    for s in (a, b, c):
        s.destroy()
    assert vmm.showFreeBlocks() == free0


def test_pointers_are_stable_and_data_survives_growth(gpu_pool):
    from glake_amd import _C

    vmm = gpu_pool
    seg = vmm.KVcacheSegment(2, 6 * CHUNK, 0, False)
    ptrs = [(seg.getKeyDevicePtr(l), seg.getValueDevicePtr(l)) for l in range(2)]
    assert len({p for pair in ptrs for p in pair}) == 4 and all(p % CHUNK == 0 for pair in ptrs for p in pair)
    seg.expandMultiSegment(1)
    rng = np.random.default_rng(0)
    blob = rng.integers(0, 256, CHUNK, dtype=np.uint8)
    _C.check(_C.lib().vtkv_memcpy_h2d(ptrs[1][0], blob.ctypes.data_as(C.c_void_p), CHUNK))
    seg.expandMultiSegment(2)
    assert [(seg.getKeyDevicePtr(l), seg.getValueDevicePtr(l)) for l in range(2)] == ptrs
    # a write spanning the old/new chunk boundary, then read everything back through one pointer
    tail = rng.integers(0, 256, 2 * CHUNK, dtype=np.uint8)
    _C.check(_C.lib().vtkv_memcpy_h2d(ptrs[1][0] + CHUNK, tail.ctypes.data_as(C.c_void_p), 2 * CHUNK))
    got = np.empty(3 * CHUNK, np.uint8)
    _C.check(_C.lib().vtkv_memcpy_d2h(got.ctypes.data_as(C.c_void_p), ptrs[1][0], 3 * CHUNK))
    assert np.array_equal(got[:CHUNK], blob) and np.array_equal(got[CHUNK:], tail)
    seg.destroy()


def test_extend_kv_cache_batch_follows_the_reference_bookkeeping(gpu_pool):
    vmm = gpu_pool
    kv = 8 * 128 * 2
    segs = [vmm.KVcacheSegment(1, 4 * CHUNK, 0, False) for _ in range(3)]
    # prefill: used += prompt bytes, mapped covers prompt + 100 rows of slack (cpp:322-337)
    prompt = [10 * kv, 1000 * kv, 1024 * kv]
    slot_m = vmm.extend_kv_cache_batch(None, None, [0, 1, 2], prompt, segs, [0, 0, 0], kv, False)
    assert slot_m == [0, 0, 0]
    assert [s.used_size for s in segs] == prompt
    assert [s.actual_size for s in segs] == [CHUNK, 2 * CHUNK, 2 * CHUNK]
    # decode: returns the offset of the new row, then advances by one row (vmm_allocator.h:150-157)
    slot_m = vmm.extend_kv_cache_batch(None, None, [0, 1, 2], [kv] * 3, segs, [0, 0, 0], kv, True)
    assert slot_m == prompt and [s.used_size for s in segs] == [p + kv for p in prompt]
    # set_used_size (in rows) rewinds a slot first (h:146-148)
    slot_m = vmm.extend_kv_cache_batch(None, None, [0, 1, 2], [kv] * 3, segs, [0, 7, 0], kv, True)
    assert slot_m[1] == 7 * kv and segs[1].used_size == 8 * kv
    # a decode row that crosses the mapped size maps the next chunk by itself
    segs[0].set_used_size(CHUNK)
    free = vmm.showFreeBlocks()
    slot_m = vmm.extend_kv_cache_batch(None, None, [0], [kv], segs[:1], [0], kv, True)
    assert slot_m == [CHUNK] and segs[0].actual_size == 2 * CHUNK and vmm.showFreeBlocks() == free - 2
    for s in segs:
        s.destroy()


def test_exhaustion_and_overflow_fail_cleanly(gpu_pool):
    from glake_amd import _C

    vmm = gpu_pool
    free0 = vmm.showFreeBlocks()
    layers = 4
    big = vmm.KVcacheSegment(layers, (free0 // (2 * layers) + 8) * CHUNK, 0, False)
    with pytest.raises(_C.VtkvOutOfChunks):
        big.expandMultiSegment(free0 // (2 * layers) + 1)          # more chunks than the pool holds
    assert big.actual_size == 0 and vmm.showFreeBlocks() == free0  # nothing half-mapped
    small = vmm.KVcacheSegment(1, 2 * CHUNK, 0, False)
    small.expandMultiSegment(2)
    with pytest.raises(_C.VtkvError):
        small.expandMultiSegment(1)                                # beyond the reserved range
    with pytest.raises(_C.VtkvError):
        vmm.KVcacheSegment(1, CHUNK + 1, 0, False)                 # not a multiple of the chunk
    small.destroy()
    big.destroy()
    with pytest.raises(_C.VtkvError):
        small.getKeyDevicePtr(0)                                   # use after destroy is caught
    assert vmm.showFreeBlocks() == free0


def test_write_string_read_string_round_trip(gpu_pool):
    # the reference's only self-check of the allocator (vmm_allocator/radix_cache.py:256-304)
    seg = gpu_pool.KVcacheSegment(1, 2 * CHUNK, 0, False)
    seg.write_string("hello ")
    seg.write_string("contiguous world")
    assert seg.read_string() == "hello contiguous world"
    seg.destroy()


def test_pointer_tables(gpu_pool):
    vmm = gpu_pool
    segs = [vmm.KVcacheSegment(2, 2 * CHUNK, 0, False) for _ in range(5)]
    kt, vt = [vmm.KVCache(5) for _ in range(2)], [vmm.KVCache(5) for _ in range(2)]
    vmm.copy_kv_cache(kt, vt, segs)
    for l in range(2):
        assert kt[l].to_numpy().tolist() == [s.getKeyDevicePtr(l) for s in segs]
        assert vt[l].to_numpy().tolist() == [s.getValueDevicePtr(l) for s in segs]
    kt[0].AddKVCache(3, 12345)
    assert kt[0].to_numpy()[3] == 12345
    for s in segs:
        s.destroy()
    for t in kt + vt:
        t.destroy()


def test_lazy_unmap_retire_revive_trim_reclaim(gpu_pool):
    """A shrinking segment keeps its chunks mapped ("retired", counted as free); the same segment takes
    them back with their contents, vtkv_pool_trim unmaps them, and another segment's growth reclaims
    them when the free list runs dry."""
    from glake_amd import _C

    vmm = gpu_pool
    vmm.trim()
    assert vmm.retiredBlocks() == 0
    free0 = vmm.showFreeBlocks()
    layers = 2
    a = vmm.KVcacheSegment(layers, 8 * CHUNK, 0, False)
    a.expandMultiSegment(3)
    blob = np.random.default_rng(3).integers(0, 256, 3 * CHUNK, dtype=np.uint8)
    _C.check(_C.lib().vtkv_memcpy_h2d(a.getValueDevicePtr(1), blob.ctypes.data_as(C.c_void_p), blob.nbytes))
    a.preempt_seq(0)
    assert a.actual_size == 0 and vmm.showFreeBlocks() == free0 and vmm.retiredBlocks() == 3 * 2 * layers
    # revival: same chunks, same place, no driver call; the bytes are still there
    a.expandMultiSegment(2)
    assert a.actual_size == 2 * CHUNK and vmm.retiredBlocks() == 1 * 2 * layers
    back = np.empty(2 * CHUNK, np.uint8)
    _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), a.getValueDevicePtr(1), back.nbytes))
    assert np.array_equal(back, blob[:2 * CHUNK])
    # growing past the retired part mixes revived and fresh chunks
    a.expandMultiSegment(3)
    assert a.actual_size == 5 * CHUNK and vmm.retiredBlocks() == 0 and vmm.showFreeBlocks() == free0 - 5 * 2 * layers
    a.preempt_seq(0)
    assert vmm.retiredBlocks() == 5 * 2 * layers
    # trim unmaps whole rows (one chunk of every range of a segment)
    assert vmm.trim(1) == 2 * layers and vmm.retiredBlocks() == 4 * 2 * layers and vmm.showFreeBlocks() == free0
    # reclaim: b needs more chunks than the free list holds, so a's retired chunks are unmapped for it
    on_list = vmm.showFreeBlocks() - vmm.retiredBlocks()
    n = on_list // 2 + 2                                           # 2 chunks per row of a 1-layer segment
    b = vmm.KVcacheSegment(1, (n + 1) * CHUNK, 0, False)
    b.expandMultiSegment(n)
    assert b.actual_size == n * CHUNK and vmm.retiredBlocks() < 4 * 2 * layers
    assert vmm.showFreeBlocks() == free0 - 2 * n
    # a can still grow: whatever is left of its retired chunks is revived, the rest is fresh
    a.expandMultiSegment(1)
    assert a.actual_size == CHUNK
    b.destroy()
    a.destroy()
    assert vmm.showFreeBlocks() == free0 and vmm.retiredBlocks() == 0


def test_map_ahead_requests_run_on_the_worker_and_settle(gpu_pool):
    """eagerExtend returns at once; the chunk appears without further calls; operations on the segment
    and rows that need the chunk wait for it; data written before and after is intact; a request that
    cannot be served is reported by the next operation on the segment."""
    import time

    from glake_amd import _C

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    layers, row = 2, 2048
    segs = [vmm.KVcacheSegment(layers, 6 * CHUNK, 0, False) for _ in range(8)]
    for i, s in enumerate(segs):
        s.expandMultiSegment(1)
        s.set_used_size(CHUNK - 3 * row)              # three rows short of the first chunk's end
        s.eagerExtend(row, 100 + i)
    deadline = time.time() + 10
    while not vmm.query_shm(range(100, 108)):
        assert time.time() < deadline, "map-ahead requests did not finish"
        time.sleep(0.001)
    assert not vmm.query_cycle(range(100, 108))
    assert all(s.actual_size == 2 * CHUNK and s.pending == 0 for s in segs)
    assert vmm.showFreeBlocks() == free0 - 8 * 2 * layers * 2
    # rows crossing into the chunk that was mapped ahead: no growth in the calling thread
    for _ in range(6):
        slot_m = vmm.extend_kv_cache_batch(None, None, list(range(8)), [row] * 8, segs, [0] * 8, row, True)
    assert slot_m == [CHUNK + 2 * row] * 8 and all(s.actual_size == 2 * CHUNK for s in segs)
    blob = np.random.default_rng(5).integers(0, 256, 2 * CHUNK, dtype=np.uint8)
    _C.check(_C.lib().vtkv_memcpy_h2d(segs[3].getKeyDevicePtr(1), blob.ctypes.data_as(C.c_void_p), blob.nbytes))
    # a burst of requests followed at once by operations that must wait for them
    for s in segs:
        s.eagerExtend(row, 0)
        s.eagerExtend(row, 0)
    segs[0].preempt_seq(0)                            # waits for both requests, then gives everything up
    assert segs[0].actual_size == 0
    segs[1].expandMultiSegment(1)                     # waits, then grows in the calling thread
    assert segs[1].actual_size == 5 * CHUNK
    vmm.wait_map_ahead()
    assert all(s.actual_size == 4 * CHUNK for s in segs[2:])
    back = np.empty(2 * CHUNK, np.uint8)
    _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), segs[3].getKeyDevicePtr(1), back.nbytes))
    assert np.array_equal(back, blob)
    # fully mapped ranges: a request is a no-op (vmm_allocator.cpp:310)
    segs[2].expandMultiSegment(2)
    segs[2].eagerExtend(row, 0)
    vmm.wait_map_ahead()
    assert segs[2].actual_size == 6 * CHUNK
    # a request the pool cannot serve leaves nothing half-mapped and no error behind; growth that the pool
    # still cannot serve fails by itself
    hog = vmm.KVcacheSegment(1, (vmm.showFreeBlocks() // 2 + 2) * CHUNK, 0, False)
    hog.expandMultiSegment((vmm.showFreeBlocks() - 2) // 2)      # leaves fewer chunks than segs[4] needs
    segs[4].eagerExtend(row, 0)
    vmm.wait_map_ahead()
    with pytest.raises(_C.VtkvOutOfChunks):
        segs[4].expandMultiSegment(1)
    assert segs[4].actual_size == 4 * CHUNK
    hog.destroy()
    for s in segs:
        s.destroy()
    assert vmm.showFreeBlocks() == free0


def test_map_ahead_batch_asks_for_what_is_about_to_be_needed(gpu_pool):
    """One call names every sequence that has come within the given distance of the end of its mapped part:
    those get a chunk per range from the worker, the others nothing; a second call asks for nothing more; with
    the pool too empty to serve a request it is not made (and no error is left behind)."""
    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    layers, row = 2, 2048
    # used bytes: 3 rows, 39 rows and 40 rows short of the chunk's end, far from it, one row short with the V offset
    near = [CHUNK - 3 * row, CHUNK - 39 * row, CHUNK - 40 * row, 5 * row, CHUNK - 256 - row]
    segs = [vmm.KVcacheSegment(layers, 4 * CHUNK, 0, False) for _ in near]
    segs[4].set_value_skew(256)
    for s, used in zip(segs, near):
        s.expandMultiSegment(1)
        s.set_used_size(used)
    assert vmm.map_ahead_batch(segs, 40 * row) == 3
    vmm.wait_map_ahead()
    assert [s.actual_size // CHUNK for s in segs] == [2, 2, 1, 1, 2] and all(s.pending == 0 for s in segs)
    assert vmm.showFreeBlocks() == free0 - (5 + 3) * 2 * layers
    assert vmm.map_ahead_batch(segs, 40 * row) == 0          # nothing is that close any more
    # rows crossing into the chunks that were mapped ahead: no growth in the calling thread
    for _ in range(5):
        vmm.extend_kv_cache_batch(None, None, [0, 4], [row] * 2, [segs[0], segs[4]], [0] * 2, row, True)
    assert segs[0].used_size == CHUNK + 2 * row and segs[0].actual_size == 2 * CHUNK and segs[4].actual_size == 2 * CHUNK
    # a pool that cannot serve the request: nothing is asked, nothing fails later
    spare = vmm.showFreeBlocks()
    hog = vmm.KVcacheSegment(1, (spare // 2 + 2) * CHUNK, 0, False)
    hog.expandMultiSegment((spare - 2) // 2)                 # leaves 2 or 3 chunks: fewer than one per range of a segment
    segs[2].set_used_size(CHUNK - 2 * row)
    assert vmm.map_ahead_batch(segs[2:3], 40 * row) == 0
    hog.preempt_seq(0)
    assert vmm.map_ahead_batch(segs[2:3], 40 * row) == 1
    vmm.wait_map_ahead()
    assert segs[2].actual_size == 2 * CHUNK
    vmm.extend_kv_cache_batch(None, None, [2], [3 * row], segs[2:3], [0], row, True)   # no stale error
    for s in segs + [hog]:
        s.destroy()
    vmm.trim()
    assert vmm.showFreeBlocks() == free0


def test_failed_map_ahead_does_not_stop_a_preemption(gpu_pool):
    """Pool exhausted, a map-ahead request fails: calls that shrink the segment still do their work (that is how
    the scheduler gets chunks back), the failed request is advisory (a step whose rows fit what is mapped runs,
    a row that needs the chunk maps it in the calling thread), and a step that fails part of the way because the
    pool really is empty leaves every sequence's used size as it was."""
    from glake_amd import _C

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    row = 2048
    segs = [vmm.KVcacheSegment(1, 4 * CHUNK, 0, False) for _ in range(3)]
    for s in segs:
        s.expandMultiSegment(1)
        s.set_used_size(CHUNK - 2 * row)
    hog = vmm.KVcacheSegment(1, (vmm.showFreeBlocks() // 2 + 2) * CHUNK, 0, False)
    hog.expandMultiSegment(vmm.showFreeBlocks() // 2)            # at most one chunk left: no room for a K+V pair
    assert vmm.showFreeBlocks() < 2
    for s in segs:
        s.eagerExtend(row, 0)
    vmm.wait_map_ahead()
    assert all(s.actual_size == CHUNK for s in segs)              # nothing half-mapped
    # shrinking calls carry on and give the chunks back
    segs[0].preempt_seq(0)
    assert segs[0].actual_size == 0 and segs[0].used_size == 0
    assert vmm.showFreeBlocks() >= 2
    segs[0].expandMultiSegment(1)                                # the old failure is forgotten, not reported here
    segs[0].preempt_seq(0)
    # rows that fit what is mapped: the failed requests of segs[1] and segs[2] do not fail the step
    used = [s.used_size for s in segs[1:]]
    slot_m = vmm.extend_kv_cache_batch(None, None, [1, 2], [row, row], segs[1:], [0, 0], row, True)
    assert slot_m == used and [s.used_size for s in segs[1:]] == [u + row for u in used]
    # the next rows cross the chunk boundary.  The pool holds exactly the two chunks of one sequence (K and V):
    # the first sequence maps them in the calling thread, the second finds the pool empty, and the step is
    # rolled back as a whole (the first sequence keeps its chunk, not its row)
    assert 2 <= vmm.showFreeBlocks() < 4
    used = [s.used_size for s in segs[1:]]
    with pytest.raises(_C.VtkvOutOfChunks):
        vmm.extend_kv_cache_batch(None, None, [1, 2], [2 * row, 2 * row], segs[1:], [0, 0], row, True)
    assert [s.used_size for s in segs[1:]] == used and segs[1].actual_size == 2 * CHUNK
    # the caller preempts the second sequence and runs the step again with what is left
    segs[2].preempt_seq(2)
    slot_m = vmm.extend_kv_cache_batch(None, None, [1], [2 * row], segs[1:2], [0], row, True)
    assert slot_m == used[:1] and segs[1].used_size == used[0] + 2 * row
    segs[1].release_seq(1)
    hog.destroy()
    for s in segs:
        s.destroy()
    assert vmm.showFreeBlocks() == free0


def test_map_ahead_that_loses_the_race_for_the_last_chunks_is_not_an_error(gpu_pool):
    """A pool with exactly the chunks the step itself needs: requests made ahead of need count what earlier
    requests in the queue will take, one that comes too late leaves no error, and the rows that need a chunk now
    get it from the calling thread."""
    vmm = gpu_pool
    vmm.trim()
    row, layers = 2048, 2
    segs = [vmm.KVcacheSegment(layers, 4 * CHUNK, 0, False) for _ in range(3)]
    for s in segs:
        s.expandMultiSegment(1)
        s.set_used_size(CHUNK - 3 * row)
    spare = vmm.showFreeBlocks()
    hog = vmm.KVcacheSegment(1, (spare // 2 + 2) * CHUNK, 0, False)
    hog.expandMultiSegment((spare - 2 * layers) // 2)             # leaves the chunks of ONE growth step (4 or 5)
    assert 2 * layers <= vmm.showFreeBlocks() < 4 * layers
    # an explicit request takes them; the batch call that follows knows and asks for nothing
    segs[0].eagerExtend(row, 0)
    assert vmm.map_ahead_batch(segs[1:], 40 * row) == 0
    vmm.wait_map_ahead()
    assert segs[0].actual_size == 2 * CHUNK and segs[1].actual_size == CHUNK
    # a request that cannot be served any more fails in the worker and is forgotten
    segs[1].eagerExtend(row, 0)
    vmm.wait_map_ahead()
    assert segs[1].actual_size == CHUNK
    for _ in range(3):                                            # rows that still fit: no error
        vmm.extend_kv_cache_batch(None, None, [1], [row], segs[1:2], [0], row, True)
    hog.preempt_seq(0)                                            # chunks come back; the row that crosses maps in the caller
    vmm.extend_kv_cache_batch(None, None, [1], [row], segs[1:2], [0], row, True)
    assert segs[1].actual_size == 2 * CHUNK and segs[1].used_size == CHUNK + row
    assert vmm.map_ahead_batch(segs[2:], 40 * row) == 1           # and a later request is made again
    vmm.wait_map_ahead()
    assert segs[2].actual_size == 2 * CHUNK
    for s in segs + [hog]:
        s.destroy()


def test_shared_prefix_maps_whole_chunks_twice_and_copies_the_tail(gpu_pool):
    """A new sequence that starts with another one's prefix: whole chunks become visible at a second
    address without taking chunks from the pool, the partly filled chunk is copied, both sequences go on
    independently, and a shared chunk returns to the pool only when its last user lets go."""
    import torch

    from glake_amd import _C

    def read(ptr, n):
        out = np.empty(n, np.uint8)
        _C.check(_C.lib().vtkv_memcpy_d2h(out.ctypes.data_as(C.c_void_p), ptr, n))
        return out

    def write(ptr, data):
        _C.check(_C.lib().vtkv_memcpy_h2d(ptr, data.ctypes.data_as(C.c_void_p), data.nbytes))

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    layers = 2
    rng = np.random.default_rng(9)
    src = vmm.KVcacheSegment(layers, 8 * CHUNK, 0, False)
    src.expandMultiSegment(3)
    used = 2 * CHUNK + 12345 * 16
    blobs = {}
    for l in range(layers):
        for which, ptr in (("k", src.getKeyDevicePtr(l)), ("v", src.getValueDevicePtr(l))):
            blobs[(l, which)] = rng.integers(0, 256, used, dtype=np.uint8)
            write(ptr, blobs[(l, which)])
    src.set_used_size(used)
    prefix = 2 * CHUNK + 4000 * 16                       # two whole chunks and a partly filled one
    dst = vmm.KVcacheSegment(layers, 8 * CHUNK, 0, False)
    dst.share_prefix(src, prefix, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert dst.used_size == prefix and dst.actual_size == 3 * CHUNK
    assert vmm.sharedBlocks() == 2 * 2 * layers           # two chunks of each of the 2*layers ranges
    assert vmm.showFreeBlocks() == free0 - 3 * 2 * layers - 1 * 2 * layers   # only the tail chunks are new
    for l in range(layers):
        for which, ptr in (("k", dst.getKeyDevicePtr(l)), ("v", dst.getValueDevicePtr(l))):
            assert np.array_equal(read(ptr, prefix), blobs[(l, which)][:prefix])
    # both go on writing behind the prefix without seeing each other
    mine = rng.integers(0, 256, 4096, dtype=np.uint8)
    write(dst.getKeyDevicePtr(0) + prefix, mine)
    assert np.array_equal(read(src.getKeyDevicePtr(0) + prefix, 4096), blobs[(0, "k")][prefix:prefix + 4096])
    dst.expandMultiSegment(1)
    assert dst.actual_size == 4 * CHUNK
    # a third sequence shares with the second one: the first two chunks now have three users
    third = vmm.KVcacheSegment(layers, 8 * CHUNK, 0, False)
    third.share_prefix(dst, 2 * CHUNK)
    assert third.actual_size == 2 * CHUNK and vmm.sharedBlocks() == 2 * 2 * layers
    free_before = vmm.showFreeBlocks()
    src.preempt_seq(0)                                     # the owner leaves first
    assert src.actual_size == 0 and vmm.retiredBlocks() == 0
    assert vmm.showFreeBlocks() == free_before + 1 * 2 * layers     # only its unshared third chunk came back
    for seg in (dst, third):
        assert np.array_equal(read(seg.getValueDevicePtr(1), 2 * CHUNK), blobs[(1, "v")][:2 * CHUNK])
    assert np.array_equal(read(dst.getKeyDevicePtr(0) + prefix, 4096), mine)
    dst.destroy()
    assert vmm.sharedBlocks() == 0 and np.array_equal(read(third.getKeyDevicePtr(1), 2 * CHUNK), blobs[(1, "k")][:2 * CHUNK])
    third.release_seq(0)
    with pytest.raises(_C.VtkvError):
        third.share_prefix(src, 1)                         # the source holds no rows any more
    src.destroy()
    third.destroy()
    assert vmm.showFreeBlocks() == free0 and vmm.retiredBlocks() == 0


def test_value_rows_set_off_from_the_base_of_their_range(gpu_pool):
    """A segment whose V rows start 256 bytes into their ranges (so that the K and the V row of a token lie in
    different memory channels): the V pointer moves, the K pointer does not, mapping counts the offset (a chunk
    boundary is reached one row early, a range filled to the last byte of a chunk owns the next one), and a
    shared prefix that ends on a chunk boundary gets a chunk of its own for the V rows' last 256 bytes."""
    import torch

    from glake_amd import _C

    def read(ptr, n):
        out = np.empty(n, np.uint8)
        _C.check(_C.lib().vtkv_memcpy_d2h(out.ctypes.data_as(C.c_void_p), ptr, n))
        return out

    def write(ptr, data):
        _C.check(_C.lib().vtkv_memcpy_h2d(ptr, data.ctypes.data_as(C.c_void_p), data.nbytes))

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    row = 8 * 128 * 2
    rng = np.random.default_rng(11)
    seg = vmm.KVcacheSegment(1, 4 * CHUNK, 0, False)
    k0, v0 = seg.getKeyDevicePtr(0), seg.getValueDevicePtr(0)
    assert seg.value_skew == 0
    with pytest.raises(_C.VtkvError):
        seg.set_value_skew(100)                            # not a multiple of 256
    with pytest.raises(_C.VtkvError):
        seg.set_value_skew(8192)
    seg.set_value_skew(256)
    assert seg.value_skew == 256 and seg.getKeyDevicePtr(0) == k0 and seg.getValueDevicePtr(0) == v0 + 256
    kt, vt = vmm.KV_cache(1, 0), vmm.KV_cache(1, 0)
    vmm.copy_kv_cache([kt.kv_cache], [vt.kv_cache], [seg])                # the pointer tables carry the offset too
    assert int(read(kt.vmm_ptr, 8).view(np.int64)[0]) == k0 and int(read(vt.vmm_ptr, 8).view(np.int64)[0]) == v0 + 256
    # rows 0..1022 fit the first chunk with the offset, row 1023 does not
    seg.ensure_mapped(1022 * row)
    assert seg.actual_size == CHUNK
    seg.set_used_size(1022 * row)
    assert vmm.extend_kv_cache_batch(None, None, [0], [row], [seg], [0], row, True) == [1022 * row]
    assert seg.actual_size == CHUNK
    assert vmm.extend_kv_cache_batch(None, None, [0], [row], [seg], [0], row, True) == [1023 * row]
    assert seg.actual_size == 2 * CHUNK and seg.used_size == CHUNK
    blobs = {}
    for which, ptr in (("k", seg.getKeyDevicePtr(0)), ("v", seg.getValueDevicePtr(0))):
        blobs[which] = rng.integers(0, 256, CHUNK, dtype=np.uint8)   # the V rows end 256 bytes into the second chunk
        write(ptr, blobs[which])
        assert np.array_equal(read(ptr, CHUNK), blobs[which])
    with pytest.raises(_C.VtkvError):
        seg.set_value_skew(0)                              # it holds rows
    with pytest.raises(_C.VtkvError):
        seg.set_used_size(4 * CHUNK)                       # the V rows would end beyond the range
    # a prefix of exactly one chunk: that chunk is shared, the V rows' last 256 bytes are copied
    dst = vmm.KVcacheSegment(1, 4 * CHUNK, 0, False)
    with pytest.raises(_C.VtkvError):
        dst.share_prefix(seg, CHUNK)                       # the two place their V rows differently
    dst.set_value_skew(256)
    dst.share_prefix(seg, CHUNK, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert dst.used_size == CHUNK and dst.actual_size == 2 * CHUNK and vmm.sharedBlocks() == 2
    assert vmm.showFreeBlocks() == free0 - 2 * 2 - 1 * 2
    for which, ptr in (("k", dst.getKeyDevicePtr(0)), ("v", dst.getValueDevicePtr(0))):
        assert np.array_equal(read(ptr, CHUNK), blobs[which])
    # the copied tail is the destination's own
    mine = rng.integers(0, 256, 256, dtype=np.uint8)
    write(dst.getValueDevicePtr(0) + CHUNK - 256, mine)
    assert np.array_equal(read(seg.getValueDevicePtr(0) + CHUNK - 256, 256), blobs["v"][CHUNK - 256:])
    # a prefix whose V rows end in the chunk behind the one its K rows end in: two chunks of its own
    seg.ensure_mapped(CHUNK - 128)
    assert seg.actual_size == 3 * CHUNK
    more = {}
    for which, ptr in (("k", seg.getKeyDevicePtr(0)), ("v", seg.getValueDevicePtr(0))):
        more[which] = rng.integers(0, 256, CHUNK - 128, dtype=np.uint8)
        write(ptr + CHUNK, more[which])
    seg.set_used_size(2 * CHUNK - 128)
    third = vmm.KVcacheSegment(1, 4 * CHUNK, 0, False)
    third.set_value_skew(256)
    third.share_prefix(seg, 2 * CHUNK - 128)
    torch.cuda.synchronize()
    assert third.actual_size == 3 * CHUNK and third.used_size == 2 * CHUNK - 128
    for which, ptr in (("k", third.getKeyDevicePtr(0)), ("v", third.getValueDevicePtr(0))):
        assert np.array_equal(read(ptr, 2 * CHUNK - 128), np.concatenate([blobs[which], more[which]]))
    for s in (dst, third, seg):
        s.destroy()
    assert vmm.showFreeBlocks() == free0 and vmm.sharedBlocks() == 0


def test_slots_are_created_and_destroyed_over_and_over(gpu_pool):
    """Churn: sets of slots of one size are created, some of them written and read, and all destroyed,
    hundreds of times.  The address ranges of destroyed slots are handed to the next slots of that size,
    so a slot that was never mapped follows one that was at the same addresses and the other way round
    (freeing and reserving the ranges anew instead ran into stale bookkeeping of the HIP runtime: a
    crash inside hipMemAddressFree or a failing hipMemMap after a few cycles)."""
    from glake_amd import _C

    vmm = gpu_pool
    free0 = vmm.showFreeBlocks()
    rng = np.random.default_rng(5)
    bases = set()
    for cycle in range(300):
        size = int(rng.integers(1, 4)) * CHUNK
        segs = [vmm.KVcacheSegment(1, size, 0, False) for _ in range(6)]
        for s in segs:
            bases.add((size, s.getKeyDevicePtr(0)))
            bases.add((size, s.getValueDevicePtr(0)))
        used = rng.permutation(6)[:3]
        for i in used:
            segs[i].expandMultiSegment(size // CHUNK)
            payload = rng.integers(0, 256, 4096, dtype=np.uint8)
            dst = segs[i].getValueDevicePtr(0) + size - 4096
            _C.check(_C.lib().vtkv_memcpy_h2d(dst, payload.ctypes.data_as(C.c_void_p), 4096))
            back = np.empty(4096, np.uint8)
            _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), dst, 4096))
            assert np.array_equal(back, payload)
        for s in segs:
            s.destroy()
        assert vmm.showFreeBlocks() == free0
    # three sizes, six slots, two ranges each: the same 36 ranges (at most) served all 300 cycles
    assert len(bases) <= 36


def test_chunks_are_replaced_after_many_map_unmap_cycles(gpu_pool):
    """One slot grows by a chunk and gives it back to the driver 700 times: the chunk on top of the free
    list goes through all of these cycles and is replaced by a newly created one after every 256 (the
    HIP runtime runs out of per-chunk state otherwise, after some 10^5 mappings at changing addresses).
    The books stay balanced and the memory works."""
    from glake_amd import _C

    vmm = gpu_pool
    free0, total0, made0 = vmm.showFreeBlocks(), vmm.totalBlocks(), vmm.recreatedBlocks()
    seg = vmm.KVcacheSegment(1, 2 * CHUNK, 0, False)
    payload = np.arange(4096, dtype=np.uint8)
    back = np.empty_like(payload)
    for cycle in range(700):
        seg.expandMultiSegment(1)
        if cycle % 50 == 0:
            dst = seg.getKeyDevicePtr(0) + CHUNK - 4096
            _C.check(_C.lib().vtkv_memcpy_h2d(dst, payload.ctypes.data_as(C.c_void_p), 4096))
            _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), dst, 4096))
            assert np.array_equal(back, payload)
        seg.preempt_seq(0)
        assert vmm.trim() == 2            # the K chunk and the V chunk really go back to the driver
    assert vmm.recreatedBlocks() - made0 >= 4     # two chunks per cycle, each replaced at 256 and 512 cycles
    seg.destroy()
    assert vmm.showFreeBlocks() == free0 and vmm.totalBlocks() == total0


def test_mappings_at_ever_new_addresses_stay_within_what_the_runtime_can_hold(gpu_pool):
    """48 slots grow by changing numbers of chunks and give them back, round after round, so that the
    chunks on top of the free list keep meeting addresses they have not been mapped at before: 75 000
    mappings, no chunk through more than some 150.  The HIP runtime holds 65 536 entries per process, one
    per chunk and one per (chunk, address) pair of a live chunk, and fails with "invalid argument" beyond;
    the pool counts the mappings of its live chunks and re-creates chunks on their way back to the free
    list once the count is above its share.  The books stay balanced and the memory works."""
    from glake_amd import _C

    vmm = gpu_pool
    free0, total0, made0 = vmm.showFreeBlocks(), vmm.totalBlocks(), vmm.recreatedBlocks()
    nseg, per = 48, 10
    segs = [vmm.KVcacheSegment(1, per * CHUNK, 0, False) for _ in range(nseg)]
    payload = np.arange(4096, dtype=np.uint8)
    back = np.empty_like(payload)
    maps = rounds = 0
    while maps < 75000:
        for i, seg in enumerate(segs):
            n = 1 + (i * 7 + rounds * 3) % per
            seg.expandMultiSegment(n)
            maps += 2 * n
        if rounds % 20 == 0:
            for seg in segs[::7]:
                dst = seg.getValueDevicePtr(0) + seg.actual_size - 4096
                _C.check(_C.lib().vtkv_memcpy_h2d(dst, payload.ctypes.data_as(C.c_void_p), 4096))
                _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), dst, 4096))
                assert np.array_equal(back, payload)
        for seg in segs:
            seg.preempt_seq(0)
        vmm.trim()
        rounds += 1
    assert vmm.recreatedBlocks() > made0
    for seg in segs:
        seg.destroy()
    assert vmm.showFreeBlocks() == free0 and vmm.totalBlocks() == total0
