"""GPU parity of the cache ops through the C ABI: bit-exact against the oracle."""
import ctypes as C
import random

import numpy as np
import pytest

from golden import gen_inputs as G
from oracle import oracle as O

from kvharness import CHUNK, GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


def host_ranges(num_slots, nbytes):
    ks = [np.zeros(nbytes, np.uint8) for _ in range(num_slots)]
    vs = [np.zeros(nbytes, np.uint8) for _ in range(num_slots)]
    return ks, vs, np.array([b.ctypes.data for b in ks], np.int64), np.array([b.ctypes.data for b in vs], np.int64)


@pytest.mark.parametrize("hkv,d", [(8, 128), (2, 64), (5, 80)])
def test_vtensor_scatter_decode_bit_exact(gpu_pool, hkv, d):
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(0)
    b, slots_n, row = 9, 12, hkv * d * 2
    gpu = GpuSeqs(gpu_pool, slots_n, hkv, d, 2, 2048)
    gpu.map_zeroed(600 * row)
    fused = rng.integers(0, 65536, (b, 3, hkv, d)).astype(np.uint16)   # key/value are strided views
    slot_ids = rng.permutation(slots_n)[:b].astype(np.int64)
    slot_m = (rng.integers(0, 500, b) * row).astype(np.int64)
    slot_m[3] = -1                                                       # skipped row
    ks, vs, kp, vp = host_ranges(slots_n, 600 * row)
    O.reshape_and_cache_vtensor(fused[:, 1], fused[:, 2], kp, vp, slot_m, slot_ids, np.ones(b), np.zeros(b), 1, hkv, d)
    f_t = torch_bf16_from_bits(fused)
    kt, vt = gpu.table_tensors()
    ops.reshape_and_cache(f_t[:, 1], f_t[:, 2], kt, vt, torch.from_numpy(slot_m).cuda(),
                          torch.from_numpy(slot_ids).cuda(), None, None, 1, hkv, d)
    torch.cuda.synchronize()
    for s in range(slots_n):
        assert np.array_equal(gpu.download(s, 600 * row, which="k"), ks[s])
        assert np.array_equal(gpu.download(s, 600 * row, which="v"), vs[s])
    gpu.close()


@pytest.mark.parametrize("eb", [2, 4])
@pytest.mark.parametrize("d", [64, 80, 96, 112, 128, 256])
def test_vtensor_scatter_over_the_reference_matrix(gpu_pool, d, eb):
    """tests/kernels/test_cache.py:10-18: 42 tokens, 8 heads, head sizes 64..256, half / bfloat16 (any 16-bit
    pattern is moved as it is) and float; one new row per sequence, rows taken from a fused qkv tensor."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(d + eb)
    b, hkv = 42, 8
    row = hkv * d * eb
    np_t, t_t = (np.uint16, torch.bfloat16) if eb == 2 else (np.uint32, torch.float32)
    gpu = GpuSeqs(gpu_pool, b, hkv, d, eb, 1024)
    gpu.map_zeroed(300 * row)
    fused = rng.integers(0, 1 << (8 * eb), (b, 3, hkv, d), dtype=np.uint64).astype(np_t)
    if eb == 4:                                           # keep the patterns finite floats: NaN payloads need not survive a .cuda()
        fused &= np.uint32(0xBF7FFFFF)
    slot_ids = rng.permutation(b).astype(np.int64)
    slot_m = (rng.integers(0, 299, b) * row).astype(np.int64)
    ks, vs, kp, vp = host_ranges(b, 300 * row)
    O.reshape_and_cache_vtensor(fused[:, 1], fused[:, 2], kp, vp, slot_m, slot_ids, np.ones(b), np.zeros(b), 1, hkv, d)
    f_t = torch.from_numpy(fused.view(np.int16 if eb == 2 else np.int32)).cuda().view(t_t)
    kt, vt = gpu.table_tensors()
    ops.reshape_and_cache(f_t[:, 1], f_t[:, 2], kt, vt, torch.from_numpy(slot_m).cuda(),
                          torch.from_numpy(slot_ids).cuda(), None, None, 1, hkv, d)
    torch.cuda.synchronize()
    for s_ in range(b):
        assert np.array_equal(gpu.download(s_, 300 * row, which="k"), ks[s_])
        assert np.array_equal(gpu.download(s_, 300 * row, which="v"), vs[s_])
    gpu.close()


@pytest.mark.parametrize("d,src", [(64, "f16"), (80, "bf16"), (96, "f32"), (112, "f16"), (256, "bf16"), (128, "f16")])
def test_vtensor_scatter_fp8_over_head_sizes_and_source_types(gpu_pool, d, src):
    """kv_cache_dtype fp8 of the same matrix (test_cache.py:24): codes e4m3fn(x / scale) from half, bfloat16 and
    float rows; an fp16 value is exact in fp32, so the oracle is given the fp32 values."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(3 * d)
    b, hkv = 42, 8
    row = hkv * d
    x_k = (rng.standard_normal((b, hkv, d)) * 2.0).astype(np.float32)
    x_v = (rng.standard_normal((b, hkv, d)) * 2.0).astype(np.float32)
    k_scale, v_scale = float(np.abs(x_k).max() / 448), 0.0171
    if src == "bf16":
        hk, hv = O.f32_to_bf16(x_k), O.f32_to_bf16(x_v)
        tk, tv = torch_bf16_from_bits(hk), torch_bf16_from_bits(hv)
    elif src == "f16":
        hk, hv = x_k.astype(np.float16).astype(np.float32), x_v.astype(np.float16).astype(np.float32)
        tk, tv = torch.from_numpy(hk).cuda().to(torch.float16), torch.from_numpy(hv).cuda().to(torch.float16)
    else:
        hk, hv = x_k, x_v
        tk, tv = torch.from_numpy(x_k).cuda(), torch.from_numpy(x_v).cuda()
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 1, 2048)
    gpu.map_zeroed(500 * row)
    slot_ids = rng.permutation(b).astype(np.int64)
    slot_m = (rng.integers(0, 499, b) * row).astype(np.int64)
    ks, vs, kp, vp = host_ranges(b, 500 * row)
    O.reshape_and_cache_vtensor_fp8(hk, hv, kp, vp, slot_m, slot_ids, hkv, d, k_scale, v_scale)
    kt, vt = gpu.table_tensors()
    ops.reshape_and_cache(tk, tv, kt, vt, torch.from_numpy(slot_m).cuda(), torch.from_numpy(slot_ids).cuda(), None,
                          None, 1, hkv, d, "fp8", k_scale, v_scale)
    torch.cuda.synchronize()
    for s_ in range(b):
        assert np.array_equal(gpu.download(s_, 500 * row, which="k"), ks[s_])
        assert np.array_equal(gpu.download(s_, 500 * row, which="v"), vs[s_])
    gpu.close()


def test_vtensor_scatter_prefill_form_bit_exact(gpu_pool):
    """grid (batch, max_query_len): rows cache_seq_lens[b]+t of the packed prompt go to consecutive rows."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(1)
    hkv, d, row = 8, 128, 8 * 128 * 2
    lens = [5, 1, 300, 64]
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    n = sum(lens)
    key, value = rng.integers(0, 65536, (n, hkv, d)).astype(np.uint16), rng.integers(0, 65536, (n, hkv, d)).astype(np.uint16)
    gpu = GpuSeqs(gpu_pool, 4, hkv, d, 2, 2048)
    gpu.map_zeroed(450 * row)
    slot_ids = np.array([3, 0, 1, 2], np.int64)
    slot_m = (np.array([0, 7, 2, 100]) * row).astype(np.int64)
    ks, vs, kp, vp = host_ranges(4, 450 * row)
    O.reshape_and_cache_vtensor(key, value, kp, vp, slot_m, slot_ids, lens, starts, max(lens), hkv, d)
    kt, vt = gpu.table_tensors()
    ops.reshape_and_cache(torch_bf16_from_bits(key), torch_bf16_from_bits(value), kt, vt,
                          torch.from_numpy(slot_m).cuda(), torch.from_numpy(slot_ids).cuda(),
                          torch.tensor(lens, dtype=torch.int32, device="cuda"), torch.from_numpy(starts).cuda(),
                          max(lens), hkv, d)
    torch.cuda.synchronize()
    for s in range(4):
        assert np.array_equal(gpu.download(s, 450 * row, which="k"), ks[s])
        assert np.array_equal(gpu.download(s, 450 * row, which="v"), vs[s])
    gpu.close()


@pytest.mark.parametrize("src", ["bf16", "f32"])
def test_vtensor_scatter_fp8_bit_exact(gpu_pool, src):
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(2)
    b, hkv, d = 16, 8, 128
    row = hkv * d  # one byte per element
    x_k = (rng.standard_normal((b, hkv, d)) * 1.5).astype(np.float32)
    x_v = (rng.standard_normal((b, hkv, d)) * 1.5).astype(np.float32)
    x_k[0, 0, :8] = [0, -0.0, 1e-9, 500.0, -500.0, 2.0 ** -9, 2.0 ** -10, 0.0146484375]  # zeros, overflow, subnormals, tie
    k_scale, v_scale = float(np.abs(x_k).max() / 448), 0.0123
    if src == "bf16":
        hk, hv = O.f32_to_bf16(x_k), O.f32_to_bf16(x_v)
        tk, tv = torch_bf16_from_bits(hk), torch_bf16_from_bits(hv)
    else:
        hk, hv = x_k, x_v
        tk, tv = torch.from_numpy(x_k).cuda(), torch.from_numpy(x_v).cuda()
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 1, 4096)
    gpu.map_zeroed(1001 * row)
    slot_ids = rng.permutation(b).astype(np.int64)
    slot_m = (rng.integers(0, 1000, b) * row).astype(np.int64)
    ks, vs, kp, vp = host_ranges(b, 1001 * row)
    O.reshape_and_cache_vtensor_fp8(hk, hv, kp, vp, slot_m, slot_ids, hkv, d, k_scale, v_scale)
    kt, vt = gpu.table_tensors()
    ops.reshape_and_cache(tk, tv, kt, vt, torch.from_numpy(slot_m).cuda(), torch.from_numpy(slot_ids).cuda(), None,
                          None, 1, hkv, d, "fp8", k_scale, v_scale)
    torch.cuda.synchronize()
    for s in range(b):
        assert np.array_equal(gpu.download(s, 1001 * row, which="k"), ks[s])
        assert np.array_equal(gpu.download(s, 1001 * row, which="v"), vs[s])
    gpu.close()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_paged_scatter_matches_reference_fixture_inputs(dtype):
    """The upstream paged layout on the golden inputs: equal to the oracle (itself pinned to the
    reference's CPU kernel on exactly these inputs)."""
    import torch

    from glake_amd import _custom_ops as ops

    c = G.cache_case(dtype)
    kc, vc = c["k_cache"].copy(), c["v_cache"].copy()
    O.reshape_and_cache_paged(c["qkv"][:, 1], c["qkv"][:, 2], kc, vc, c["slot_mapping"])
    if dtype == "bf16":
        to_t = lambda a: torch_bf16_from_bits(a)
        back = bits_from_torch_bf16
    else:
        to_t = lambda a: torch.from_numpy(a).cuda()
        back = lambda t: t.cpu().numpy()
    qkv, gk, gv = to_t(c["qkv"]), to_t(c["k_cache"]), to_t(c["v_cache"])
    ops.reshape_and_cache_paged(qkv[:, 1], qkv[:, 2], gk, gv, torch.from_numpy(c["slot_mapping"]).cuda(), "auto", 1.0)
    torch.cuda.synchronize()
    assert np.array_equal(back(gk), kc) and np.array_equal(back(gv), vc)


@pytest.mark.parametrize("num_heads,head_size,block_size,dtype",
                         [(8, 64, 8, "bf16"), (8, 80, 16, "f32"), (8, 128, 32, "bf16"), (8, 256, 16, "f16"), (3, 66, 16, "bf16")])
def test_flash_layout_scatter_like_the_reference_test(num_heads, head_size, block_size, dtype):
    """tests/kernels/test_cache.py:206-270: 42 tokens of a fused qkv tensor to random slots of K and V caches
    [num_blocks, block_size, H, D]; the expectation is the reference test's own closed form
    cache[slot // block_size, slot % block_size] = row, a padded token (slot -1) is skipped, bytes exact.
    (3 heads of 66 make rows that are no multiple of 16 bytes: the 2-byte path.)"""
    import torch

    from glake_amd import _custom_ops as ops

    random.seed(0)
    rng = np.random.default_rng(head_size)
    num_tokens, num_blocks = 42, 1024
    slots = random.sample(range(block_size * num_blocks), num_tokens)
    slots[5] = -1
    np_t, t_t = {"bf16": (np.uint16, torch.bfloat16), "f16": (np.uint16, torch.float16), "f32": (np.uint32, torch.float32)}[dtype]
    bits = 8 * np.dtype(np_t).itemsize
    qkv = rng.integers(0, 1 << bits, (num_tokens, 3, num_heads, head_size), dtype=np.uint64).astype(np_t)
    kc = rng.integers(0, 1 << bits, (num_blocks, block_size, num_heads, head_size), dtype=np.uint64).astype(np_t)
    vc = rng.integers(0, 1 << bits, (num_blocks, block_size, num_heads, head_size), dtype=np.uint64).astype(np_t)
    if dtype == "f32":  # keep the patterns finite floats: NaN payloads need not survive a .cuda()
        qkv &= np.uint32(0xBF7FFFFF); kc &= np.uint32(0xBF7FFFFF); vc &= np.uint32(0xBF7FFFFF)
    signed = np.int16 if bits == 16 else np.int32
    to_t = lambda a: torch.from_numpy(a.view(signed)).cuda().view(t_t)
    back = lambda t: t.view(torch.int16 if bits == 16 else torch.int32).cpu().numpy().view(np_t)
    g_qkv, g_k, g_v = to_t(qkv), to_t(kc), to_t(vc)
    ops.reshape_and_cache_flash(g_qkv[:, 1], g_qkv[:, 2], g_k, g_v, torch.tensor(slots, dtype=torch.int64, device="cuda"),
                                "auto")
    torch.cuda.synchronize()
    for i, s_ in enumerate(slots):
        if s_ < 0:
            continue
        kc[s_ // block_size, s_ % block_size] = qkv[i, 1]
        vc[s_ // block_size, s_ % block_size] = qkv[i, 2]
    assert np.array_equal(back(g_k), kc) and np.array_equal(back(g_v), vc)
    with pytest.raises(Exception):
        ops.reshape_and_cache_flash(g_qkv[:, 1], g_qkv[:, 2], g_k, g_v, torch.tensor(slots, dtype=torch.int64, device="cuda"),
                                    "fp8")


def test_copy_blocks_takes_more_layers_than_one_launch_holds():
    """160 layers (two launches of the layer table), small blocks, and the call returns without waiting."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(8)
    layers, num_blocks = 160, 12
    mapping = [(0, 5), (3, 7), (3, 11), (9, 1)]
    ks = [rng.integers(0, 65536, (num_blocks, 2, 4, 8)).astype(np.uint16) for _ in range(layers)]
    vs = [rng.integers(0, 65536, (num_blocks, 2, 4, 8)).astype(np.uint16) for _ in range(layers)]
    gk, gv = [torch_bf16_from_bits(k) for k in ks], [torch_bf16_from_bits(v) for v in vs]
    ops.copy_blocks(gk, gv, torch.tensor(mapping, dtype=torch.int64, device="cuda"))
    O.copy_blocks(ks, vs, np.array(mapping))
    torch.cuda.synchronize()
    for a, b in zip(gk + gv, ks + vs):
        assert np.array_equal(bits_from_torch_bf16(a), b)


def test_copy_blocks_like_the_reference_test():
    """tests/kernels/test_cache.py:31-102: every source block copied to two destinations, 3 layers."""
    import torch

    from glake_amd import _custom_ops as ops

    random.seed(0)
    num_blocks, num_mappings, layers = 1024, 256, 3
    src = random.sample(range(num_blocks), num_mappings)
    rest = sorted(set(range(num_blocks)) - set(src))
    dst = random.sample(rest, 2 * num_mappings)
    mapping = [(src[i], dst[2 * i + j]) for i in range(num_mappings) for j in range(2)]
    rng = np.random.default_rng(3)
    ks = [rng.integers(0, 65536, (num_blocks, 8, 16, 16, 8)).astype(np.uint16) for _ in range(layers)]
    vs = [rng.integers(0, 65536, (num_blocks, 8, 128, 16)).astype(np.uint16) for _ in range(layers)]
    gk, gv = [torch_bf16_from_bits(k) for k in ks], [torch_bf16_from_bits(v) for v in vs]
    ops.copy_blocks(gk, gv, torch.tensor(mapping, dtype=torch.int64, device="cuda"))
    O.copy_blocks(ks, vs, np.array(mapping))
    torch.cuda.synchronize()
    for a, b in zip(gk + gv, ks + vs):
        assert np.array_equal(bits_from_torch_bf16(a), b)


@pytest.mark.parametrize("direction", [("cuda", "cpu"), ("cuda", "cuda"), ("cpu", "cuda")])
def test_swap_blocks_like_the_reference_tests(direction):
    """tests/kernels/test_cache.py:274-344 (random pairs) and tests/worker/test_swap.py:57-89 (fixed pairs)."""
    import torch

    from glake_amd import _custom_ops as ops

    random.seed(0)
    num_blocks, num_mappings = 1024, 256
    src_blocks = random.sample(range(num_blocks), num_mappings)
    if direction[0] == direction[1]:
        dst_blocks = random.sample(sorted(set(range(num_blocks)) - set(src_blocks)), num_mappings)
    else:
        dst_blocks = random.sample(range(num_blocks), num_mappings)
    fixed = [(3, 72), (56, 35), (84, 34)] if direction[0] == "cuda" else [(19, 45), (67, 23), (12, 78), (40, 99), (1, 71)]
    for mapping in (list(zip(src_blocks, dst_blocks)), fixed, [(10, 500), (11, 501), (12, 502), (13, 503)]):
        rng = np.random.default_rng(4)
        shape = (num_blocks, 8 * 128 * 16)
        a = torch.from_numpy(rng.integers(-32768, 32767, shape).astype(np.int16)).view(torch.bfloat16)
        b = torch.from_numpy(rng.integers(-32768, 32767, shape).astype(np.int16)).view(torch.bfloat16)
        src = a.cuda() if direction[0] == "cuda" else a.pin_memory()
        dst = b.cuda() if direction[1] == "cuda" else b.pin_memory()
        want = b.view(torch.int16).numpy().copy()
        O.swap_blocks(a.view(torch.int16).numpy(), want, np.array(mapping))
        ops.swap_blocks(src, dst, torch.tensor(mapping, dtype=torch.int64))
        torch.cuda.synchronize()
        assert np.array_equal(dst.cpu().view(torch.int16).numpy(), want)


def test_swap_blocks_rejects_gpu_mapping():
    import torch

    from glake_amd import _C, _custom_ops as ops

    a = torch.zeros(4, 64, device="cuda")
    with pytest.raises(_C.VtkvError, match="block_mapping must be on CPU"):
        ops.swap_blocks(a, a, torch.zeros(1, 2, dtype=torch.int64, device="cuda"))


@pytest.mark.parametrize("wide", ["f32", "bf16", "f16"])
def test_convert_fp8_bit_exact_and_round_trip(wide):
    """tests/kernels/test_cache.py:347-380 plus exact agreement with the oracle in both directions."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(5)
    x = rng.uniform(-224, 224, (64, 8, 128, 16)).astype(np.float32)
    dt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[wide]
    xt = torch.from_numpy(x).cuda().to(dt)
    codes = torch.empty(x.shape, dtype=torch.uint8, device="cuda")
    for scale in (1.0, 0.61):   # 224 / 0.61 stays inside the +-448 range
        ops.convert_fp8(codes, xt, scale)
        back = torch.empty_like(xt)
        ops.convert_fp8(back, codes, scale)
        torch.cuda.synchronize()
        x_wide = xt.float().cpu().numpy()
        want_codes = O.fp8_encode(x_wide, scale)
        assert np.array_equal(codes.cpu().numpy(), want_codes)
        want_back = O.fp8_decode(want_codes, scale)
        if wide == "f32":
            assert np.array_equal(back.cpu().numpy(), want_back)
        elif wide == "bf16":
            assert np.array_equal(bits_from_torch_bf16(back), O.f32_to_bf16(want_back))
        ok = bool(torch.allclose(xt.float(), back.float(), atol=1e-3, rtol=0.1))
        assert ok, "round trip outside atol 1e-3 / rtol 0.1"
