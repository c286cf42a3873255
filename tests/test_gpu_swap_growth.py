"""Dynamic growth plus swap (BASELINE config 5): sequences append one token per step, map a new
2 MiB chunk when they cross a boundary, and a seeded quarter of them is swapped out to pinned host
memory and back every 16 steps.  Every KV byte is checked exactly; attention is checked against
the oracle on a sample of sequences at the end."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import CHUNK, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


def download(seg, nbytes, which):
    from glake_amd import _C

    out = np.empty(nbytes // 2, np.uint16)
    src = seg.getKeyDevicePtr(0) if which == 0 else seg.getValueDevicePtr(0)
    _C.check(_C.lib().vtkv_memcpy_d2h(out.ctypes.data_as(C.c_void_p), src, nbytes))
    return out


@pytest.mark.parametrize("num_seqs,steps", [(32, 20), (256, 64)])
def test_growth_and_swap_round_trips_are_bit_exact(gpu_pool, num_seqs, steps):
    import torch

    from glake_amd import _custom_ops as ops, vmm_allocator as vmm
    from glake_amd.worker.cache_engine import CacheEngine

    hq, hkv, d = 32, 8, 128
    row = hkv * d * 2
    gen = torch.Generator().manual_seed(1004)
    ctx = torch.randint(256, 2049, (num_seqs,), generator=gen).tolist()
    # make sure some sequences cross a chunk boundary (1024 rows) during the run
    ctx[0], ctx[1], ctx[2] = 1024 - 3, 1024, 2048 - steps // 2
    free0 = vmm.showFreeBlocks()
    eng = CacheEngine(1, hkv, d, torch.bfloat16, num_seqs, 2048 + steps + 8, swap_space_bytes=num_seqs // 4 * 2 * 3 * CHUNK)
    segs = eng.vmm_kvcache_segment
    dev = torch.device("cuda")
    ggen = torch.Generator(device=dev).manual_seed(7)
    expect_k, expect_v = [], []
    for b in range(num_seqs):
        nbytes = ctx[b] * row
        segs[b].ensure_mapped(nbytes)   # counts the engine's V offset (sequence 1 fills its chunk to the last byte)
        for which, keep in ((0, expect_k), (1, expect_v)):
            t = torch.randn(ctx[b], hkv, d, generator=ggen, device=dev).to(torch.bfloat16)
            base = segs[b].getKeyDevicePtr(0) if which == 0 else segs[b].getValueDevicePtr(0)
            ops.swap_ranges([t.data_ptr()], [base], [nbytes], "d2d")
            torch.cuda.synchronize()
            keep.append([bits_from_torch_bf16(t).reshape(-1)])
        segs[b].set_used_size(nbytes)
    slot_t = torch.arange(num_seqs, dtype=torch.int64, device=dev)
    lens = list(ctx)
    moved_out = moved_in = 0
    maps = 0
    for step in range(1, steps + 1):
        mapped_before = [s.actual_size for s in segs]
        slot_m = vmm.extend_kv_cache_batch(None, None, list(range(num_seqs)), [row] * num_seqs, segs,
                                           [0] * num_seqs, row, True)
        assert slot_m == [n * row for n in lens]
        maps += sum(a.actual_size > m for a, m in zip(segs, mapped_before))
        nk = torch.randn(num_seqs, hkv, d, generator=ggen, device=dev).to(torch.bfloat16)
        nv = torch.randn(num_seqs, hkv, d, generator=ggen, device=dev).to(torch.bfloat16)
        ops.reshape_and_cache(nk, nv, eng.k_cache_ptr[0], eng.v_cache_ptr[0],
                              torch.tensor(slot_m, dtype=torch.int64, device=dev), slot_t, None, None, 1, hkv, d)
        hk, hv = bits_from_torch_bf16(nk), bits_from_torch_bf16(nv)
        for b in range(num_seqs):
            expect_k[b].append(hk[b].reshape(-1))
            expect_v[b].append(hv[b].reshape(-1))
        lens = [n + 1 for n in lens]
        if step % 16 == 0 or (steps < 16 and step == steps // 2):
            subset = torch.randperm(num_seqs, generator=gen)[:num_seqs // 4].tolist()
            free_before = vmm.showFreeBlocks()
            moved_out += eng.swap_out(subset)
            assert all(segs[s].actual_size == 0 for s in subset)
            assert vmm.showFreeBlocks() > free_before           # their chunks are back in the pool
            moved_in += eng.swap_in(subset)
            assert vmm.showFreeBlocks() == free_before
            assert all(segs[s].used_size == lens[s] * row for s in subset)
    assert maps >= 2 and moved_out == moved_in > 0
    torch.cuda.synchronize()
    for b in range(num_seqs):
        want_k, want_v = np.concatenate(expect_k[b]), np.concatenate(expect_v[b])
        assert np.array_equal(download(segs[b], lens[b] * row, 0), want_k), f"K of sequence {b} differs"
        assert np.array_equal(download(segs[b], lens[b] * row, 1), want_v), f"V of sequence {b} differs"
    # attention on a sample (sequence 0 and 1 crossed a chunk boundary) against the oracle
    sample = [0, 1, 2, num_seqs // 2, num_seqs - 1]
    q = O.f32_to_bf16(np.random.default_rng(0).standard_normal((num_seqs, hq, d)).astype(np.float32))
    out = torch.empty(num_seqs, hq, d, dtype=torch.float32, device=dev)
    ops.paged_attention_v1(out, torch_bf16_from_bits(q), eng.k_cache_ptr[0], eng.v_cache_ptr[0], hkv, d ** -0.5,
                           torch.tensor(lens, dtype=torch.int32, device=dev), 1, max(lens), None, "auto", 1.0, slot_t)
    got = out.cpu().numpy()[sample]
    kb = [np.concatenate(expect_k[b]).reshape(-1, hkv, d) for b in sample]
    vb = [np.concatenate(expect_v[b]).reshape(-1, hkv, d) for b in sample]
    want = O.paged_attention_v1(O.bf16_to_f32(q[sample]), O.VTensorCache(kb, vb, np.arange(len(sample)), hkv, d),
                                d ** -0.5, [lens[b] for b in sample])
    assert np.all(np.abs(got - want) <= 2e-3 + 2e-3 * np.abs(want))
    eng.close()
    assert vmm.showFreeBlocks() == free0


def test_swap_ranges_piece_and_stream_variants_are_exact(gpu_pool):
    import torch

    from glake_amd import _C, _custom_ops as ops

    n = 37 * (1 << 20) + 4096 + 16
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
    host = int(_C.check_ptr(_C.lib().vtkv_host_alloc(n), "host"))
    for piece, streams in ((0, 0), (1 << 20, 4), (3 << 20, 8), (n, 1)):
        back = torch.zeros_like(src)
        ops.swap_ranges([src.data_ptr(), src.data_ptr() + n // 2], [host, host + n // 2], [n // 2, n - n // 2], "out",
                        piece, streams)
        ops.swap_ranges([host], [back.data_ptr()], [n], "in", piece, streams)
        torch.cuda.synchronize()
        assert torch.equal(src, back)
    _C.check(_C.lib().vtkv_host_free(C.c_void_p(host)))


def test_swap_out_into_a_full_arena_changes_nothing(gpu_pool):
    """The host arena holds one of two sequences: swapping both out fails as a whole, both stay resident
    with their bytes, the arena stays empty, and each can still be swapped out (and in) alone."""
    import torch

    from glake_amd import _C
    from glake_amd.worker.cache_engine import CacheEngine

    hkv, d = 8, 128
    row = hkv * d * 2
    eng = CacheEngine(num_layers=2, num_kv_heads=hkv, head_size=d, dtype=torch.bfloat16, max_num_seqs=2,
                      max_num_batched_tokens=600, swap_space_bytes=2 * 2 * 300 * row + 4096)
    rng = np.random.default_rng(3)
    data = {}
    for slot, tokens in ((0, 300), (1, 250)):
        seg = eng.vmm_kvcache_segment[slot]
        seg.expandMultiSegment(1)
        seg.set_used_size(tokens * row)
        for l in range(2):
            for which, base in (("k", seg.getKeyDevicePtr(l)), ("v", seg.getValueDevicePtr(l))):
                buf = rng.integers(0, 256, tokens * row, dtype=np.uint8)
                _C.check(_C.lib().vtkv_memcpy_h2d(base, buf.ctypes.data, buf.nbytes))
                data[(slot, l, which)] = buf

    def resident_bytes_intact():
        for (slot, l, which), buf in data.items():
            seg = eng.vmm_kvcache_segment[slot]
            base = seg.getKeyDevicePtr(l) if which == "k" else seg.getValueDevicePtr(l)
            back = np.empty_like(buf)
            _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data, base, buf.nbytes))
            assert np.array_equal(back, buf), (slot, l, which)

    with pytest.raises(_C.VtkvOutOfChunks):
        eng.swap_out([0, 1])
    assert eng._swapped == {} and eng._arena.free == [(0, eng._arena.nbytes)]
    assert [s.actual_size for s in eng.vmm_kvcache_segment] == [2 << 20, 2 << 20]
    resident_bytes_intact()
    with pytest.raises(_C.VtkvError):
        eng.swap_out([0, 0])
    for slot in (0, 1):
        eng.swap_out([slot])
        assert eng.vmm_kvcache_segment[slot].actual_size == 0
        eng.swap_in([slot])
    resident_bytes_intact()
    eng.close()


def test_swap_in_that_finds_the_pool_empty_leaves_the_sequences_swapped_out(gpu_pool):
    """Two sequences are swapped out and somebody else takes the chunks in between: swapping both in fails part
    of the way, both stay in host memory and their slots hold nothing, and once the chunks are back the same call
    succeeds with every byte in place."""
    import torch

    from glake_amd import _C
    from glake_amd.worker.cache_engine import CacheEngine

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    hkv, d, layers = 8, 128, 2
    row = hkv * d * 2
    tokens = {0: 2500, 1: 1800}                            # 3 and 2 chunks per range
    eng = CacheEngine(num_layers=layers, num_kv_heads=hkv, head_size=d, dtype=torch.bfloat16, max_num_seqs=2,
                      max_num_batched_tokens=3000, swap_space_bytes=64 << 20)
    rng = np.random.default_rng(4)
    data = {}
    for slot, n in tokens.items():
        seg = eng.vmm_kvcache_segment[slot]
        seg.ensure_mapped(n * row)
        seg.set_used_size(n * row)
        for l in range(layers):
            for which, base in (("k", seg.getKeyDevicePtr(l)), ("v", seg.getValueDevicePtr(l))):
                buf = rng.integers(0, 256, n * row, dtype=np.uint8)
                _C.check(_C.lib().vtkv_memcpy_h2d(base, buf.ctypes.data, buf.nbytes))
                data[(slot, l, which)] = buf
    eng.swap_out([0, 1])
    assert vmm.showFreeBlocks() == free0
    # a hog leaves enough for the first sequence (3 chunks x 2 ranges x 2 layers) but not for the second
    spare = vmm.showFreeBlocks()
    hog = vmm.KVcacheSegment(1, (spare // 2 + 2) * CHUNK, 0, False)
    hog.expandMultiSegment((spare - 14) // 2)
    with pytest.raises(_C.VtkvOutOfChunks):
        eng.swap_in([0, 1])
    assert sorted(eng._swapped) == [0, 1]
    assert [s.actual_size for s in eng.vmm_kvcache_segment] == [0, 0] and [s.used_size for s in eng.vmm_kvcache_segment] == [0, 0]
    hog.destroy()
    eng.swap_in([0, 1])
    assert eng._swapped == {}
    for (slot, l, which), buf in data.items():
        seg = eng.vmm_kvcache_segment[slot]
        base = seg.getKeyDevicePtr(l) if which == "k" else seg.getValueDevicePtr(l)
        back = np.empty_like(buf)
        _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data, base, buf.nbytes))
        assert np.array_equal(back, buf), (slot, l, which)
    eng.close()
    vmm.trim()
    assert vmm.showFreeBlocks() == free0
