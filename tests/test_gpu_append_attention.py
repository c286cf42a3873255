"""The fused decode-step launch (vtkv_decode_append_attention, through the C ABI): the new K/V rows
land in the cache bit for bit where reshape_and_cache would put them, and the attention output over
old rows + new row is within 2e-3 abs + 2e-3 rel of the oracle (fp32 output, see test_gpu_attention.py
for why the comparison is made before the final bf16 store), for lengths from the host (kernel
arguments) and from the device, for a bf16 cache and for an fp8 cache (the new row is then quantised
inside the launch, to the same codes as reshape_and_cache writes)."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu

TOL = 2e-3


def run_case(vmm, seed, seq_lens, hq, hkv, lens_from="host", alibi=False, partition_tokens=0, d=128, fp8=False,
             value_skew=0):
    """seq_lens count the new token; value_skew: bytes between the base of a V range and its first row."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(seq_lens)
    num_slots = b + 2
    slots = rng.permutation(num_slots)[:b]
    eb = 1 if fp8 else 2
    row = hkv * d * eb
    k_scale, v_scale = (0.021, 0.033) if fp8 else (1.0, 1.0)
    code_t = np.uint8 if fp8 else np.uint16

    def stored(bits, sc):  # what the cache holds for bf16 source rows
        return O.fp8_encode(O.bf16_to_f32(bits), sc) if fp8 else bits

    gpu = GpuSeqs(vmm, num_slots, hkv, d, eb, max(seq_lens) + 1, value_skew=value_skew)
    k_host, v_host = {}, {}
    for i, t in enumerate(seq_lens):
        s = int(slots[i])
        k_host[s] = stored(bf16_randn(rng, (t - 1, hkv, d)), k_scale)
        v_host[s] = stored(bf16_randn(rng, (t - 1, hkv, d)), v_scale)
        gpu.upload(s, k_host[s], v_host[s])
    # the step's bookkeeping maps the chunk a new row needs, as in the engine
    used = vmm.extend_kv_cache_batch(None, None, [int(s) for s in slots], [row] * b, [gpu.segs[int(s)] for s in slots],
                                     [0] * b, row, True)
    assert used == [(t - 1) * row for t in seq_lens]
    q = bf16_randn(rng, (b, hq, d))
    nk, nv = bf16_randn(rng, (b, hkv, d)), bf16_randn(rng, (b, hkv, d))
    slopes = rng.standard_normal(hq).astype(np.float32) if alibi else None
    scale = float(d) ** -0.5

    kt, vt = gpu.table_tensors()
    out32 = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    out16 = torch.empty(b, hq, d, dtype=torch.bfloat16, device="cuda")
    q_t, nk_t, nv_t = (torch_bf16_from_bits(x) for x in (q, nk, nv))
    lens_arg = list(seq_lens) if lens_from == "host" else torch.tensor(seq_lens, dtype=torch.int32, device="cuda")
    slot_t = torch.tensor(slots, dtype=torch.int64, device="cuda")
    al_t = None if slopes is None else torch.from_numpy(slopes).cuda()
    for o in (out32, out16):  # the second call appends the same rows again: idempotent
        ops.decode_append_attention(o, q_t, nk_t, nv_t, kt, vt, hkv, scale, lens_arg, max(seq_lens), al_t, slot_t,
                                    partition_tokens=partition_tokens, kv_cache_dtype="fp8" if fp8 else "auto",
                                    kv_scale=k_scale, v_scale=v_scale)
    torch.cuda.synchronize()

    # cache: old rows untouched, new row in place
    full_k = [np.zeros((1, hkv, d), code_t)] * num_slots
    full_v = [np.zeros((1, hkv, d), code_t)] * num_slots
    for i, t in enumerate(seq_lens):
        s = int(slots[i])
        full_k[s] = np.concatenate([k_host[s], stored(nk[i:i + 1], k_scale)])
        full_v[s] = np.concatenate([v_host[s], stored(nv[i:i + 1], v_scale)])
        assert np.array_equal(gpu.download(s, t * row, which="k", dtype=code_t), full_k[s].reshape(-1)), f"K of seq {i}"
        assert np.array_equal(gpu.download(s, t * row, which="v", dtype=code_t), full_v[s].reshape(-1)), f"V of seq {i}"
    if fp8:  # exact dequantisation in fp32, which is what the kernel computes with
        full_k = [O.fp8_decode(c, k_scale) for c in full_k]
        full_v = [O.fp8_decode(c, v_scale) for c in full_v]
    cache = O.VTensorCache(full_k, full_v, slots, hkv, d)
    expect32 = O.paged_attention_v1(O.bf16_to_f32(q), cache, scale, seq_lens, slopes)
    got = out32.cpu().numpy()
    gpu.close()
    assert np.array_equal(bits_from_torch_bf16(out16), O.f32_to_bf16(got)), "bf16 output is not RNE(fp32 output)"
    err = np.abs(got - expect32)
    bound = TOL + TOL * np.abs(expect32)
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert np.all(err <= bound), (f"max err {err.max():.3e} at (seq, head, d)={worst}: got {got[worst]!r} "
                                  f"want {expect32[worst]!r}, len {seq_lens[worst[0]]}")
    return got


EDGE = [1, 2, 3, 16, 17, 18, 33, 64, 65, 66, 256, 257, 258, 1025, 1026]


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (8, 8), (16, 1)])
@pytest.mark.parametrize("lens_from", ["host", "device"])
def test_edge_lengths(gpu_pool, hq, hkv, lens_from):
    run_case(gpu_pool, 11, EDGE, hq, hkv, lens_from=lens_from)


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (16, 1)])
@pytest.mark.parametrize("lens_from", ["host", "device"])
def test_fp8_cache_edge_lengths(gpu_pool, hq, hkv, lens_from):
    run_case(gpu_pool, 13, EDGE + [2049, 2050], hq, hkv, lens_from=lens_from, fp8=True)


def test_fp8_cache_alibi_and_partitions(gpu_pool):
    run_case(gpu_pool, 14, [1, 34, 401, 1000], 32, 8, alibi=True, fp8=True)
    run_case(gpu_pool, 15, [700, 65, 1, 1500, 2049, 17], 32, 8, partition_tokens=512, fp8=True, lens_from="device")


def test_config2_shape(gpu_pool):
    rng = np.random.default_rng(1001)
    run_case(gpu_pool, 1001, rng.integers(512, 4097, 64).tolist(), 32, 8)


def test_alibi(gpu_pool):
    run_case(gpu_pool, 5, [1, 34, 401, 1000], 32, 8, alibi=True)


@pytest.mark.parametrize("pt", [64, 512])
def test_fixed_partitions_agree(gpu_pool, pt):
    lens = [700, 65, 1, 1500, 2049, 17]
    got = run_case(gpu_pool, 7, lens, 32, 8, partition_tokens=pt)
    base = run_case(gpu_pool, 7, lens, 32, 8)
    assert np.abs(got - base).max() <= 2e-3


@pytest.mark.parametrize("lens_from", ["host", "device"])
def test_very_many_short_sequences(gpu_pool, lens_from):
    # 512 sequences x 8 kv heads = 4096 segments: the variants that stream a pair of kv heads per workgroup
    rng = np.random.default_rng(5)
    lens = [int(x) for x in rng.integers(1, 50, 509)] + [900, 1, 17]
    run_case(gpu_pool, 21, lens, 32, 8, lens_from=lens_from)
    run_case(gpu_pool, 22, lens, 16, 8, lens_from=lens_from, alibi=True)


@pytest.mark.parametrize("fp8", [False, True])
def test_value_rows_offset_from_their_range_base_around_chunk_ends(gpu_pool, fp8):
    """The engine's placement (V rows 256 bytes into their range): sequences whose new row is the last one that
    fits the first chunk with the offset, the first one that does not, and rows on either side of the 2 MiB and
    4 MiB marks; cache bytes exact, attention within tolerance."""
    per = (2 << 20) // (8 * 128 * (1 if fp8 else 2))       # rows per chunk
    lens = [per - 1, per, per + 1, per + 2, 2 * per - 1, 2 * per, 2 * per + 1, 5, 700, 1]
    run_case(gpu_pool, 31, lens, 32, 8, fp8=fp8, value_skew=256)
    run_case(gpu_pool, 32, lens, 64, 8, lens_from="device", fp8=fp8, value_skew=256, alibi=True)


def test_long_sequence_many_workgroups_per_segment(gpu_pool):
    # one sequence spread over many workgroups plus short ones: the new row's tile is a segment of its own for some
    run_case(gpu_pool, 9, [40000, 1, 2, 5000], 32, 8, lens_from="device")


def test_more_host_lengths_than_one_launch_carries(gpu_pool):
    """512 lengths fit the kernel arguments of one launch; 700 sequences with host lengths run as two launches
    inside the one call (cache rows exact, attention within tolerance, as for every other case)."""
    rng = np.random.default_rng(6)
    lens = [int(x) for x in rng.integers(1, 50, 697)] + [900, 1, 17]
    lens[511], lens[512] = 333, 2
    run_case(gpu_pool, 23, lens, 16, 4, lens_from="host")


def test_rejects_other_cache_types_and_shapes(gpu_pool):
    import ctypes as C

    import torch

    from glake_amd import _C

    lib = _C.lib()
    t = torch.zeros(1024, dtype=torch.uint8, device="cuda")
    p = C.c_void_p(t.data_ptr())
    ws = torch.empty(lib.vtkv_decode_attention_workspace_bytes(600, 8, 128, 16, 0), dtype=torch.uint8, device="cuda")
    rc = lib.vtkv_decode_append_attention(p, p, p, p, 128, 128, p, p, p, p, None, 1, 8, 1, 128, 1024, 1.0, 16, None,
                                          _C.BF16, _C.BF16, _C.F32, 1.0, 1.0, C.c_void_p(ws.data_ptr()), ws.numel(), 0, None)
    assert rc == _C.EINVAL and "q_dtype or FP8_E4M3" in _C.last_error()          # an fp32 cache
    rc = lib.vtkv_decode_append_attention(p, p, p, p, 64, 64, p, p, p, p, None, 1, 8, 1, 64, 512, 1.0, 16, None,
                                          _C.BF16, _C.BF16, _C.FP8_E4M3, 1.0, 1.0, C.c_void_p(ws.data_ptr()), ws.numel(),
                                          0, None)
    assert rc == _C.EINVAL and "16-bit rows" in _C.last_error()     # new rows are quantised at head size 128 only
    rc = lib.vtkv_decode_append_attention(p, p, p, p, 128, 128, p, p, p, p, None, 1, 8, 1, 128, 1024, 1.0, 16, None,
                                          _C.BF16, _C.BF16, _C.FP8_E4M3, 0.0, 1.0, C.c_void_p(ws.data_ptr()), ws.numel(),
                                          0, None)
    assert rc == _C.EINVAL and "scales" in _C.last_error()
