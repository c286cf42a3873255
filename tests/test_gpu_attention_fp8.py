"""GPU parity of decode attention over an fp8-e4m3fn KV cache (per-tensor scale = amax/448, K and V
scaled separately), through the C ABI.

The oracle follows the reference's own test protocol (tests/kernels/test_attention.py:233-252): the
cache is converted back to the model dtype (bf16) with the scale applied, and the unquantised
attention oracle runs on that.  Tolerance: 3e-2 absolute + 3e-2 relative on the values before the
final bf16 store (the absolute part scales with the spread of V when V is made wider than N(0,1)).  A second, tighter check (2e-3) is made against the oracle run on the exactly
dequantised values code*scale held in fp32, which is what the kernel computes with."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


def run_case(vmm, seed, seq_lens, hq, hkv, d=128, alibi=False, spread=1.0, partition_tokens=0, scales=None):
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(seq_lens)
    slots = rng.permutation(b + 2)[:b]
    k_f = [rng.standard_normal((t, hkv, d)).astype(np.float32) for t in seq_lens]
    v_f = [rng.standard_normal((t, hkv, d)).astype(np.float32) * spread for t in seq_lens]
    k_scale = float(max(np.abs(k).max() for k in k_f) / 448.0)
    v_scale = float(max(np.abs(v).max() for v in v_f) / 448.0)
    if scales is not None:  # given scales instead of amax / 448: values beyond 448 * scale saturate
        k_scale, v_scale = scales
    gpu = GpuSeqs(vmm, b + 2, hkv, d, 1, max(seq_lens))
    empty8 = np.zeros((1, hkv, d), np.uint8)
    k_codes, v_codes = [empty8] * (b + 2), [empty8] * (b + 2)
    for i in range(b):
        k_codes[slots[i]] = O.fp8_encode(k_f[i], k_scale)
        v_codes[slots[i]] = O.fp8_encode(v_f[i], v_scale)
        gpu.upload(int(slots[i]), k_codes[slots[i]], v_codes[slots[i]])
    q = bf16_randn(rng, (b, hq, d))
    scale = float(d) ** -0.5
    slopes = (rng.standard_normal(hq) * 0.1).astype(np.float32) if alibi else None

    # reference protocol: dequantise to bf16 (round to nearest), then the ordinary oracle
    k_bf = [O.fp8_decode(c, k_scale, to_bf16=True) for c in k_codes]
    v_bf = [O.fp8_decode(c, v_scale, to_bf16=True) for c in v_codes]
    want_ref = O.paged_attention_v1(O.bf16_to_f32(q), O.VTensorCache(k_bf, v_bf, slots, hkv, d), scale, seq_lens, slopes)
    # exact dequantisation in fp32
    k_32 = [O.fp8_decode(c, k_scale) for c in k_codes]
    v_32 = [O.fp8_decode(c, v_scale) for c in v_codes]
    want_exact = O.paged_attention_v1(O.bf16_to_f32(q), O.VTensorCache(k_32, v_32, slots, hkv, d), scale, seq_lens, slopes)

    kt, vt = gpu.table_tensors()
    out32 = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    out16 = torch.empty(b, hq, d, dtype=torch.bfloat16, device="cuda")
    args = (torch_bf16_from_bits(q), kt, vt, hkv, scale, torch.tensor(seq_lens, dtype=torch.int32, device="cuda"), 1,
            max(seq_lens), None if slopes is None else torch.from_numpy(slopes).cuda(), "fp8", k_scale,
            torch.tensor(slots, dtype=torch.int64, device="cuda"))
    ops.paged_attention_v1(out32, *args, v_scale=v_scale, partition_tokens=partition_tokens)
    ops.paged_attention_v1(out16, *args, v_scale=v_scale, partition_tokens=partition_tokens)
    torch.cuda.synchronize()
    gpu.close()
    got = out32.cpu().numpy()
    assert np.array_equal(bits_from_torch_bf16(out16), O.f32_to_bf16(got))
    err = np.abs(got - want_ref)
    assert np.all(err <= 3e-2 * spread + 3e-2 * np.abs(want_ref)), f"vs reference protocol: max err {err.max():.3e}"
    err = np.abs(got - want_exact)
    assert np.all(err <= 2e-3 * spread + 2e-3 * np.abs(want_exact)), f"vs exact dequantisation: max err {err.max():.3e}"
    return got


@pytest.mark.parametrize("hq,hkv", [(64, 8), (32, 8), (16, 16)])
def test_fp8_edge_lengths(gpu_pool, hq, hkv):
    run_case(gpu_pool, 1, [1, 7, 8, 9, 15, 16, 17, 63, 64, 65, 511, 512, 513, 1030], hq, hkv)


def test_fp8_config4_shape_llama70b_layer(gpu_pool):
    # BASELINE config 4 at reduced batch: Hq 64, Hkv 8 (GQA 8), ctx uniform in [1024, 8192]
    rng = np.random.default_rng(1003)
    run_case(gpu_pool, 1003, rng.integers(1024, 8193, 6).tolist(), 64, 8)


def test_fp8_with_the_reference_models_layer_scales(gpu_pool):
    """The per-layer scales of the reference's llama2-7b and llama2-70b fp8 checkpoints
    (tests/fp8_kv/*/kv_cache_scales.json) through the loader, one scale for K and V of a layer as the model passes
    it (llama.py:484-505; no doubling: this cache is OCP e4m3fn like the file, not FNUZ)."""
    import os

    from glake_amd.worker.kv_scales import layer_scales

    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_kv")
    s7 = layer_scales(os.path.join(golden, "llama2-7b_kv_cache_scales.json"), 32, model_type="llama")
    s70 = layer_scales(os.path.join(golden, "llama2-70b_kv_cache_scales.json"), 80, model_type="llama")
    for seed, (s, hq, hkv) in enumerate([(s7[0], 32, 32), (s7[31], 32, 8), (s70[0], 64, 8), (max(s70), 64, 8)]):
        run_case(gpu_pool, 40 + seed, [17, 300, 1111], hq, hkv, scales=(s, s))


def test_fp8_alibi_and_wide_values(gpu_pool):
    # V twenty times wider than K: exercises a V scale far from the K scale
    run_case(gpu_pool, 2, [33, 700], 64, 8, alibi=True, spread=20.0)


def test_fp8_every_code_decodes_exactly(gpu_pool):
    """T = 1: the output is the V row, so feeding all 254 finite codes as V checks the kernel's
    in-register widening of e4m3fn against the oracle's decode, subnormals included."""
    import torch

    from glake_amd import _custom_ops as ops

    hq, hkv, d = 32, 8, 128
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    v = np.resize(codes, (1, hkv, d)).astype(np.uint8)
    k = np.full((1, hkv, d), 0x38, np.uint8)  # 1.0
    gpu = GpuSeqs(gpu_pool, 1, hkv, d, 1, 16)
    gpu.upload(0, k, v)
    kt, vt = gpu.table_tensors()
    q = torch.ones(1, hq, d, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(1, hq, d, dtype=torch.float32, device="cuda")
    v_scale = 0.75
    ops.paged_attention_v1(out, q, kt, vt, hkv, 1.0, torch.tensor([1], dtype=torch.int32, device="cuda"), 1, 1, None,
                           "fp8", 1.0, torch.zeros(1, dtype=torch.int64, device="cuda"), v_scale=v_scale)
    torch.cuda.synchronize()
    gpu.close()
    got = out.cpu().numpy()[0]
    want = np.repeat(O.fp8_decode(v[0]) * np.float32(v_scale), hq // hkv, axis=0)
    assert np.array_equal(got, want)
