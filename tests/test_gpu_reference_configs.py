"""The HIP path on the reference-pinned inputs and on BASELINE's configurations at their full sizes.

* every golden case of tests/golden/reference_cpu.npz (outputs of the reference's own CPU kernels,
  GLakeServe/csrc/cpu/attention.cpp, on the integer-lattice inputs of tests/golden/gen_inputs.py) is fed to
  the HIP kernels directly: the paged caches are unrolled into contiguous ranges, the kernel runs through the
  C ABI, and the result is compared with the stored reference output, the oracle taking no part;
* config 1's seeded shape (B=8, ctx U[128,1024], seed 1000; fp32 in the reference, a CPU config) with its
  values rounded to bf16, against the fp32 oracle on the same values, plus the paged fp32 scatter at
  config 1's dimensions;
* config 3 with all four sequences and config 4 at full size (B=128, fp8 cache, fused append through
  DecodeStepPlan, the path bench.py times);
* the reference's split-K interface with its per-partition buffers.

Tolerances: 2e-3 abs + 2e-3 rel on fp32 results (tests/kernels/test_attention.py:271-274 uses 1e-3/1e-5 on
fp16/bf16 outputs of a kernel that rounds P to bf16; here the comparison is made before the final rounding,
see test_gpu_attention.py); fp8: 3e-2; bytes and codes: exact."""
import ctypes as C
import os

import numpy as np
import pytest

from golden import gen_inputs as G
from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_cpu.npz"))


def unroll_paged(c):
    """Paged K [nb,H,D/x,bs,x] / V [nb,H,D,bs] + block tables -> per-sequence [T,H,D] arrays."""
    k_cache, v_cache, bt, lens = c["k_cache"], c["v_cache"], c["block_tables"], c["seq_lens"]
    nb, h, dx, bs, x = k_cache.shape
    d = dx * x
    ks, vs = [], []
    for b, n in enumerate(lens):
        nblk = (int(n) + bs - 1) // bs
        blocks = bt[b, :nblk]
        k = k_cache[blocks].transpose(0, 3, 1, 2, 4).reshape(nblk * bs, h, d)   # [blk, bs, H, D/x, x]
        v = v_cache[blocks].transpose(0, 3, 1, 2).reshape(nblk * bs, h, d)      # [blk, bs, H, D]
        ks.append(np.ascontiguousarray(k[:n]))
        vs.append(np.ascontiguousarray(v[:n]))
    return ks, vs


@pytest.mark.parametrize("name", sorted(G.ATTENTION_CASES))
def test_hip_kernel_against_the_reference_cpu_outputs(gpu_pool, name):
    """GPU vs the stored outputs of the reference's CPU kernels.  The lattice inputs (multiples of 1/8) are
    exact in bf16, so the fp32 cases run on the bf16 kernel with the very same values.  The reference build
    stores bf16 by truncation: its fp32 result lies in [stored, stored + one bf16 step) in magnitude."""
    import torch

    from glake_amd import _custom_ops as ops

    c = G.attention_case(name)
    gold = GOLD["attn_" + name]
    ks, vs = unroll_paged(c)
    as_bits = (lambda a: a) if c["dtype"] == "bf16" else G.f32_to_bf16_bits
    q = as_bits(c["q"])
    b, hq, d = q.shape
    hkv = c["num_kv_heads"]
    lens = [int(n) for n in c["seq_lens"]]
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 2, max(lens), value_skew=256)
    for i in range(b):
        gpu.upload(i, as_bits(ks[i]), as_bits(vs[i]))
    kt, vt = gpu.table_tensors()
    out = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    slots = torch.arange(b, dtype=torch.int64, device="cuda")
    al = None if c["alibi_slopes"] is None else torch.from_numpy(c["alibi_slopes"]).cuda()
    q_t = torch_bf16_from_bits(q)
    if c["version"] == 1:
        ops.paged_attention_v1(out, q_t, kt, vt, hkv, c["scale"], sl, 1, max(lens), al, "auto", 1.0, slots)
    else:
        parts = (max(lens) + 511) // 512
        es = torch.zeros(b, hq, parts, dtype=torch.float32, device="cuda")
        ml = torch.zeros_like(es)
        tmp = torch.zeros(b, hq, parts, d, dtype=torch.bfloat16, device="cuda")
        ops.paged_attention_v2(out, es, ml, tmp, q_t, kt, vt, hkv, c["scale"], sl, 1, max(lens), al, "auto", 1.0, slots)
    torch.cuda.synchronize()
    gpu.close()
    got = out.cpu().numpy()
    if c["dtype"] == "f32":
        ok = bool(np.all(np.abs(got - gold) <= 2e-3 + 2e-3 * np.abs(gold)))
        assert ok, f"max err {np.abs(got - gold).max():.3e}"
    else:
        stored = O.bf16_to_f32(gold)
        step = np.maximum(np.abs(stored), 2.0 ** -126) * 2.0 ** -7      # at most one bf16 step at this magnitude
        excess = (got - stored) * np.where(stored < 0, -1.0, 1.0)      # how far beyond the stored magnitude
        tol = 2e-3 + 2e-3 * np.abs(stored)
        # the split-K twin also stores every partition's result in bf16, truncated, before it merges them
        # (csrc/cpu/attention.cpp:535-541): two truncations on the way to the stored value
        steps = 2 if c["version"] == 2 else 1
        low, high = float(excess.min() + tol[np.unravel_index(excess.argmin(), excess.shape)]), \
            float((excess - steps * step - tol).max())
        assert low >= 0 and high <= 0, f"outside [stored, stored + {steps} bf16 steps): {low:.3e} below, {high:.3e} above"


def test_config1_shape_on_the_bf16_kernels(gpu_pool):
    """BASELINE config 1 (B=8, Hq=32, Hkv=8, D=128, ctx U[128,1024], seed 1000) is fp32 and CPU-only in the
    reference; what one GPU can show of it: the same seeded shape with its N(0,1) values rounded to bf16,
    through the bf16 kernel, against the oracle's fp32 path on those values."""
    import torch

    from glake_amd import _custom_ops as ops

    gen = torch.Generator().manual_seed(1000)
    b, hq, hkv, d = 8, 32, 8, 128
    lens = torch.randint(128, 1025, (b,), generator=gen).tolist()
    q = O.f32_to_bf16(torch.randn(b, hq, d, generator=gen).numpy())
    ks = [O.f32_to_bf16(torch.randn(n, hkv, d, generator=gen).numpy()) for n in lens]
    vs = [O.f32_to_bf16(torch.randn(n, hkv, d, generator=gen).numpy()) for n in lens]
    scale = d ** -0.5
    # the oracle in fp32 on the bf16-representable values, contiguous layout (config 1's "vs contiguous" side)
    k32, v32 = [O.bf16_to_f32(k) for k in ks], [O.bf16_to_f32(v) for v in vs]
    want = O.paged_attention_v1(O.bf16_to_f32(q), O.VTensorCache(k32, v32, np.arange(b), hkv, d), scale, lens)
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 2, max(lens), value_skew=256)
    for i in range(b):
        gpu.upload(i, ks[i], vs[i])
    kt, vt = gpu.table_tensors()
    out = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    ops.paged_attention_v1(out, torch_bf16_from_bits(q), kt, vt, hkv, scale,
                           torch.tensor(lens, dtype=torch.int32, device="cuda"), 1, max(lens), None, "auto", 1.0,
                           torch.arange(b, dtype=torch.int64, device="cuda"))
    torch.cuda.synchronize()
    gpu.close()
    err = np.abs(out.cpu().numpy() - want)
    assert np.all(err <= 2e-3 + 2e-3 * np.abs(want)), f"max err {err.max():.3e}"


def test_config1_paged_scatter_in_fp32(gpu_pool):
    """reshape_and_cache at config 1's dimensions: fp32 (x = 4), block 16, B = 8 new rows of 8 x 128 into a
    paged cache sized for ctx U[128,1024]; equal to the oracle (pinned to the reference's cpu/cache.cpp) bit
    for bit."""
    import torch

    from glake_amd import _custom_ops as ops

    gen = torch.Generator().manual_seed(1000)
    b, hkv, d, bs, x = 8, 8, 128, 16, 4
    lens = torch.randint(128, 1025, (b,), generator=gen).tolist()
    nblk = sum((n + 1 + bs - 1) // bs for n in lens)
    perm = torch.randperm(nblk, generator=gen).tolist()
    k_cache = torch.randn(nblk, hkv, d // x, bs, x, generator=gen)
    v_cache = torch.randn(nblk, hkv, d, bs, generator=gen)
    key = torch.randn(b, hkv, d, generator=gen)
    value = torch.randn(b, hkv, d, generator=gen)
    slots, at = [], 0
    for n in lens:                                   # the new row is token n of its sequence
        blocks = perm[at:at + (n + 1 + bs - 1) // bs]
        slots.append(blocks[n // bs] * bs + n % bs)
        at += len(blocks)
    slot_t = torch.tensor(slots, dtype=torch.int64)
    kc, vc = k_cache.numpy().copy(), v_cache.numpy().copy()
    O.reshape_and_cache_paged(key.numpy(), value.numpy(), kc, vc, slot_t.numpy())
    kg, vg = k_cache.cuda(), v_cache.cuda()
    ops.reshape_and_cache_paged(key.cuda(), value.cuda(), kg, vg, slot_t.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(kg.cpu().numpy().view(np.uint32), kc.view(np.uint32))
    assert np.array_equal(vg.cpu().numpy().view(np.uint32), vc.view(np.uint32))
    # the closed form of the reference's own test (tests/kernels/test_cache.py:170-180)
    for i, s in enumerate(slots):
        blk, off = s // bs, s % bs
        assert torch.equal(kg[blk, :, :, off, :].reshape(hkv, d).cpu(), key[i])
        assert torch.equal(vg[blk, :, :, off].cpu(), value[i])


def test_config3_all_four_sequences(gpu_pool):
    """BASELINE config 3 at full size: B=4, contexts U[32768,131072] (seed 1002), hundreds of workgroups per
    (sequence, kv head)."""
    import test_gpu_attention as A

    gen = np.random.default_rng(1002)
    lens = [int(x) for x in gen.integers(32768, 131073, 4)]
    lens[-1] = 131072                                   # the longest the config allows
    A.run_case(gpu_pool, 1002, lens, 32, 8, shuffle_slots=False)


def test_config4_full_size_through_the_step_plan(gpu_pool):
    """BASELINE config 4 as bench.py runs it: B=128, Hq=64, Hkv=8, fp8-e4m3fn cache, ctx U[1024,8192]
    (seed 1003), two decode steps through DecodeStepPlan (range bookkeeping + one launch that quantises
    and appends the new rows and attends; merge mode and tile order as the library chooses for 512 (sequence,
    head pair) segments).  Appended codes bit-exact against the oracle's encoder, attention against the
    reference's fp8 protocol (dequantise to bf16, then the unquantised oracle) at 3e-2."""
    import torch

    from glake_amd import _C
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step import DecodeStepPlan

    b, hq, hkv, d = 128, 64, 8, 128
    rng = np.random.default_rng(1003)
    lens = [int(x) for x in rng.integers(1024, 8193, b)]
    row = hkv * d
    k_scale, v_scale = 6.0 / 448.0, 5.5 / 448.0
    eng = CacheEngine(1, hkv, d, torch.uint8, b, max(lens) + 8)
    segs = eng.vmm_kvcache_segment
    k_codes, v_codes = [], []
    for i, n in enumerate(lens):
        kc = O.fp8_encode(rng.standard_normal((n, hkv, d)).astype(np.float32), k_scale)
        vc = O.fp8_encode(rng.standard_normal((n, hkv, d)).astype(np.float32), v_scale)
        segs[i].ensure_mapped(n * row)
        _C.check(_C.lib().vtkv_memcpy_h2d(segs[i].getKeyDevicePtr(0), kc.ctypes.data_as(C.c_void_p), kc.nbytes))
        _C.check(_C.lib().vtkv_memcpy_h2d(segs[i].getValueDevicePtr(0), vc.ctypes.data_as(C.c_void_p), vc.nbytes))
        segs[i].set_used_size(n * row)
        k_codes.append(kc)
        v_codes.append(vc)
    plan = DecodeStepPlan(segs, list(range(b)), eng.k_cache_ptr[0], eng.v_cache_ptr[0], hq, hkv, d, d ** -0.5,
                          kv_cache_dtype="fp8", k_scale=k_scale, v_scale=v_scale)
    assert plan.fused
    out = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    for step in range(2):
        q = bf16_randn(rng, (b, hq, d))
        nk, nv = bf16_randn(rng, (b, hkv, d)), bf16_randn(rng, (b, hkv, d))
        plan.run(torch_bf16_from_bits(q), torch_bf16_from_bits(nk), torch_bf16_from_bits(nv), out)
        torch.cuda.synchronize()
        lens = [n + 1 for n in lens]
        assert plan.seq_lens.tolist() == lens
        new_kc, new_vc = O.fp8_encode(O.bf16_to_f32(nk), k_scale), O.fp8_encode(O.bf16_to_f32(nv), v_scale)
        for i in range(b):
            k_codes[i] = np.concatenate([k_codes[i], new_kc[i:i + 1]])
            v_codes[i] = np.concatenate([v_codes[i], new_vc[i:i + 1]])
            for codes, ptr in ((k_codes[i], segs[i].getKeyDevicePtr(0)), (v_codes[i], segs[i].getValueDevicePtr(0))):
                got = np.empty((1, hkv, d), np.uint8)          # the appended row, as the cache holds it
                _C.check(_C.lib().vtkv_memcpy_d2h(got.ctypes.data_as(C.c_void_p), ptr + (lens[i] - 1) * row, row))
                assert np.array_equal(got, codes[-1:]), f"appended codes of sequence {i} differ"
        k_bf = [O.fp8_decode(c, k_scale, to_bf16=True) for c in k_codes]
        v_bf = [O.fp8_decode(c, v_scale, to_bf16=True) for c in v_codes]
        want = O.paged_attention_v1(O.bf16_to_f32(q), O.VTensorCache(k_bf, v_bf, np.arange(b), hkv, d), d ** -0.5, lens)
        err = np.abs(out.cpu().numpy() - want)
        assert np.all(err <= 3e-2 + 3e-2 * np.abs(want)), f"step {step}: max err {err.max():.3e}"
    # a whole sequence's cache, first to last byte (the rows before the append are untouched)
    for i in (0, b // 2, b - 1):
        got = np.empty_like(k_codes[i])
        _C.check(_C.lib().vtkv_memcpy_d2h(got.ctypes.data_as(C.c_void_p), segs[i].getKeyDevicePtr(0), got.nbytes))
        assert np.array_equal(got, k_codes[i])
    eng.close()


@pytest.mark.parametrize("hq,hkv,fp8", [(32, 8, False), (64, 8, True), (8, 8, False), (71, 1, False), (48, 2, True)])
def test_split_k_interface_fills_the_callers_partition_buffers(gpu_pool, hq, hkv, fp8):
    """paged_attention_v2 with exp_sums / max_logits / tmp_out (csrc/attention/attention_kernels.cu:451-583):
    partition j of a sequence is rows [512 j, 512 j + 512).  Its entries are checked against values derived
    without the split: tmp_out[j] is plain attention over those rows alone (the v1 oracle on a slice of the
    cache), max_logits and exp_sums come from a float64 q.K^T; `out` is checked against the v1 oracle, and
    merging the buffers by the reference's rule (:515-582) gives `out` again."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(5)
    d = 128
    lens = [1, 511, 512, 513, 1024, 1500, 2049]
    b = len(lens)
    parts = (max(lens) + 511) // 512 + 1                # one spare partition column: must stay untouched
    k_scale, v_scale = (0.012, 0.02) if fp8 else (1.0, 1.0)
    if fp8:
        ks = [O.fp8_encode(rng.standard_normal((n, hkv, d)).astype(np.float32), k_scale) for n in lens]
        vs = [O.fp8_encode(rng.standard_normal((n, hkv, d)).astype(np.float32), v_scale) for n in lens]
        k32 = [O.fp8_decode(c, k_scale) for c in ks]
        v32 = [O.fp8_decode(c, v_scale) for c in vs]
    else:
        ks = [bf16_randn(rng, (n, hkv, d)) for n in lens]
        vs = [bf16_randn(rng, (n, hkv, d)) for n in lens]
        k32, v32 = [O.bf16_to_f32(k) for k in ks], [O.bf16_to_f32(v) for v in vs]
    q = bf16_randn(rng, (b, hq, d))
    q32 = O.bf16_to_f32(q)
    scale = d ** -0.5
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 1 if fp8 else 2, max(lens))
    for i in range(b):
        gpu.upload(i, ks[i], vs[i])
    kt, vt = gpu.table_tensors()
    out = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    es = torch.full((b, hq, parts), -7.0, dtype=torch.float32, device="cuda")
    ml = torch.full((b, hq, parts), -7.0, dtype=torch.float32, device="cuda")
    tmp = torch.full((b, hq, parts, d), -7.0, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention_v2(out, es, ml, tmp, torch_bf16_from_bits(q), kt, vt, hkv, scale,
                           torch.tensor(lens, dtype=torch.int32, device="cuda"), 1, max(lens), None,
                           "fp8" if fp8 else "auto", k_scale, torch.arange(b, dtype=torch.int64, device="cuda"),
                           v_scale=v_scale)
    torch.cuda.synchronize()
    gpu.close()
    got, es, ml = out.cpu().numpy(), es.cpu().numpy(), ml.cpu().numpy()
    tmp = O.bf16_to_f32(bits_from_torch_bf16(tmp))
    want = O.paged_attention_v1(q32, O.VTensorCache(k32, v32, np.arange(b), hkv, d), scale, lens)
    tol = 2e-3
    assert np.all(np.abs(got - want) <= tol + tol * np.abs(want))
    g = hq // hkv
    for i, n in enumerate(lens):
        np_i = (n + 511) // 512
        assert np.all(es[i, :, np_i:] == -7.0) and np.all(ml[i, :, np_i:] == -7.0) and np.all(tmp[i, :, np_i:] == -7.0)
        for j in range(np_i):
            lo, hi = 512 * j, min(n, 512 * j + 512)
            sl_k, sl_v = np.ascontiguousarray(k32[i][lo:hi]), np.ascontiguousarray(v32[i][lo:hi])
            part = O.paged_attention_v1(q32[i:i + 1], O.VTensorCache([sl_k], [sl_v], np.zeros(1, np.int64), hkv, d),
                                        scale, [hi - lo])[0]
            # tmp_out is stored in bf16: one more rounding (2^-9 relative)
            assert np.all(np.abs(tmp[i, :, j] - part) <= tol + (tol + 2.0 ** -8) * np.abs(part))
            for h in range(hq):
                s = scale * (sl_k[:, h // g].astype(np.float64) @ q32[i, h].astype(np.float64))
                assert abs(ml[i, h, j] - s.max()) <= 1e-4 + 1e-5 * abs(s.max())
                sm = np.exp(s - s.max()).sum()
                assert abs(es[i, h, j] - sm) <= 1e-4 * sm
        # the reference's merge of the buffers (attention_kernels.cu:515-582) reproduces `out`
        m = ml[i, :, :np_i].max(axis=1, keepdims=True)
        w = es[i, :, :np_i] * np.exp(ml[i, :, :np_i] - m)
        merged = (tmp[i, :, :np_i] * w[..., None]).sum(axis=1) / (w.sum(axis=1, keepdims=True) + 1e-6)
        assert np.all(np.abs(merged - got[i]) <= 4e-3 + 4e-3 * np.abs(got[i]))
