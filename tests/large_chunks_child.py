"""Run by tests/test_gpu_large_chunks.py in a process of its own (the chunk size is a property of the
process-wide pool): a pool of 8 MiB chunks serves the same calls as the default 2 MiB one."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def main():
    import torch

    from glake_amd import _C, vmm_allocator as vmm
    from glake_amd.worker.cache_engine import CacheEngine
    import test_gpu_attention as A
    import test_gpu_attention_fp8 as F

    torch.cuda.set_device(0)
    big = 8 << 20
    with_error = 0
    try:
        vmm.set_chunk_bytes(3 << 20)          # not a power of two
    except _C.VtkvError:
        with_error += 1
    vmm.set_chunk_bytes(big)
    assert vmm.chunkBytes() == big
    vmm.init_physical_handle(40, 0)
    try:
        vmm.set_chunk_bytes(2 << 20)          # the pool holds chunks
    except _C.VtkvError as e:
        assert e.code == _C.ESTATE
        with_error += 1
    try:
        vmm.KVcacheSegment(1, 2 << 20, 0, False)   # not a multiple of the chunk
    except _C.VtkvError:
        with_error += 1
    assert with_error == 3

    # accounting in 8 MiB units, data across a chunk boundary
    seg = vmm.KVcacheSegment(2, 3 * big, 0, False)
    seg.expandMultiSegment(2)
    assert seg.actual_size == 2 * big and vmm.showFreeBlocks() == 40 - 2 * 2 * 2
    blob = np.random.default_rng(0).integers(0, 256, big + 4096, dtype=np.uint8)
    import ctypes as C
    _C.check(_C.lib().vtkv_memcpy_h2d(seg.getValueDevicePtr(1) + big - 2048, blob.ctypes.data_as(C.c_void_p), 4096))
    back = np.empty(4096, np.uint8)
    _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), seg.getValueDevicePtr(1) + big - 2048, 4096))
    assert np.array_equal(back, blob[:4096])
    # a decode row that crosses the mapped size maps the next (8 MiB) chunk by itself
    row = 8 * 128 * 2
    seg.set_used_size(2 * big)
    off = vmm.extend_kv_cache_batch(None, None, [0], [row], [seg], [0], row, True)
    assert off == [2 * big] and seg.actual_size == 3 * big
    seg.destroy()
    assert vmm.showFreeBlocks() == 40

    # attention parity over ranges made of 8 MiB chunks (4096 bf16 rows of 8 heads per chunk): sequences
    # inside one chunk, across two, ragged ends; bf16 and fp8 caches
    A.run_case(vmm, 5, [1, 17, 4095, 4096, 4097, 6000], 32, 8)
    F.run_case(vmm, 6, [33, 8191, 8193, 9000], 64, 8)

    # the cache engine sizes its slots in the pool's chunks and swaps whole sequences
    eng = CacheEngine(1, 8, 128, torch.bfloat16, 3, 5000, swap_space_bytes=64 << 20)
    assert eng.max_context_size % big == 0 and eng.chunk_bytes == big
    seg = eng.vmm_kvcache_segment[1]
    seg.expandMultiSegment(2)
    payload = np.random.default_rng(1).integers(0, 256, big + 777 * row, dtype=np.uint8)
    for ptr in (seg.getKeyDevicePtr(0), seg.getValueDevicePtr(0)):
        _C.check(_C.lib().vtkv_memcpy_h2d(ptr, payload.ctypes.data_as(C.c_void_p), payload.nbytes))
    seg.set_used_size(payload.nbytes)
    eng.swap_out([1])
    assert seg.actual_size == 0
    eng.swap_in([1])
    torch.cuda.synchronize()
    got = np.empty_like(payload)
    for ptr in (seg.getKeyDevicePtr(0), seg.getValueDevicePtr(0)):
        _C.check(_C.lib().vtkv_memcpy_d2h(got.ctypes.data_as(C.c_void_p), ptr, payload.nbytes))
        assert np.array_equal(got, payload)
    print("large chunks ok", flush=True)


if __name__ == "__main__":
    main()
