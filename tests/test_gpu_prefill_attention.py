"""GPU parity of prompt (prefill) attention over the contiguous ranges, through the C ABI, against
the prefill oracle on the same seeded inputs: plain prompts, prompt chunks behind a cached prefix,
GQA groups 1..8, ALiBi, an fp8 cache, and more units than one call takes.  Tolerance as for decode:
2e-3 abs + 2e-3 rel on the fp32 output (3e-2 for the fp8 cache against the reference's test protocol of
dequantising to bf16 first); the bf16 output must be the round-to-nearest of the fp32 one."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


def run_case(vmm, seed, query_lens, seq_lens, hq, hkv, d=128, alibi=False, fp8=False, tol=2e-3, shape_inputs=None,
             out_scale=1.0):
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(seq_lens)
    slots = rng.permutation(b + 2)[:b]
    gpu = GpuSeqs(vmm, b + 2, hkv, d, 1 if fp8 else 2, max(seq_lens))
    empty = np.zeros((1, hkv, d), np.uint8 if fp8 else np.uint16)
    k_host, v_host = [empty] * (b + 2), [empty] * (b + 2)
    k_scale = v_scale = 1.0
    if fp8:
        k_f = [rng.standard_normal((t, hkv, d)).astype(np.float32) for t in seq_lens]
        v_f = [rng.standard_normal((t, hkv, d)).astype(np.float32) for t in seq_lens]
        k_scale = float(max(np.abs(x).max() for x in k_f) / 448.0)
        v_scale = float(max(np.abs(x).max() for x in v_f) / 448.0)
    for i, t in enumerate(seq_lens):
        s = int(slots[i])
        if fp8:
            k_host[s], v_host[s] = O.fp8_encode(k_f[i], k_scale), O.fp8_encode(v_f[i], v_scale)
        else:
            k_host[s], v_host[s] = bf16_randn(rng, (t, hkv, d)), bf16_randn(rng, (t, hkv, d))
    n_tok = sum(query_lens)
    q = bf16_randn(rng, (n_tok, hq, d))
    if shape_inputs is not None:  # bf16 bit patterns, edited in place
        shape_inputs(q, [k_host[int(s)] for s in slots], [v_host[int(s)] for s in slots])
    for s in slots:
        gpu.upload(int(s), k_host[int(s)], v_host[int(s)])
    scale = float(d) ** -0.5
    slopes = (rng.standard_normal(hq) * 0.1).astype(np.float32) if alibi else None
    if fp8:  # exact dequantisation in fp32, which is what the kernel computes with
        kk = [O.fp8_decode(c, k_scale) for c in k_host]
        vv = [O.fp8_decode(c, v_scale) for c in v_host]
    else:
        kk, vv = k_host, v_host
    expect = O.prefill_attention(O.bf16_to_f32(q), O.VTensorCache(kk, vv, slots, hkv, d), scale, query_lens, seq_lens,
                                 slopes)
    kt, vt = gpu.table_tensors()
    out32 = torch.empty(n_tok, hq, d, dtype=torch.float32, device="cuda")
    out16 = torch.empty(n_tok, hq, d, dtype=torch.bfloat16, device="cuda")
    for o in (out32, out16):
        ops.prefill_attention(o, torch_bf16_from_bits(q), kt, vt, hkv, scale, query_lens, seq_lens,
                              torch.tensor(slots, dtype=torch.int64, device="cuda"),
                              None if slopes is None else torch.from_numpy(slopes).cuda(),
                              "fp8" if fp8 else "auto", k_scale, v_scale)
    torch.cuda.synchronize()
    gpu.close()
    got = out32.cpu().numpy()
    assert np.isfinite(got).all()
    assert np.array_equal(bits_from_torch_bf16(out16), O.f32_to_bf16(got)), "bf16 output is not RNE(fp32 output)"
    err = np.abs(got - expect)
    bound = tol * out_scale + tol * np.abs(expect)   # out_scale: the magnitude of the V values, 1 by default
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert np.all(err <= bound), (f"max err {err.max():.3e} at (token, head, d)={worst}: got {got[worst]!r} "
                                  f"want {expect[worst]!r}")
    return got


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (8, 8), (16, 1), (12, 4)])
def test_plain_prompts(gpu_pool, hq, hkv):
    lens = [1, 2, 3, 15, 16, 17, 33, 100, 257, 700]
    run_case(gpu_pool, 1, lens, lens, hq, hkv)


@pytest.mark.parametrize("hq,hkv", [(32, 8), (16, 1)])
def test_prompt_chunks_behind_a_cached_prefix(gpu_pool, hq, hkv):
    # (query tokens, rows): chunked prefill and prefix reuse; one decode-like entry with a single query token
    query_lens = [5, 64, 1, 130, 17, 300]
    seq_lens = [21, 64 + 1000, 400, 130 + 16, 17 + 2047, 300 + 300]
    run_case(gpu_pool, 2, query_lens, seq_lens, hq, hkv)


def test_alibi(gpu_pool):
    run_case(gpu_pool, 3, [40, 7, 260], [40, 100, 500], 32, 8, alibi=True)


def test_fp8_cache(gpu_pool):
    run_case(gpu_pool, 4, [33, 200, 64], [33, 200, 64 + 500], 32, 8, fp8=True)


def test_long_prompt_needs_several_calls(gpu_pool):
    # 5000 query tokens at 4 tokens per unit: 1250 units, more than the 1024 one call takes
    run_case(gpu_pool, 5, [4200, 800], [4200, 800 + 100], 32, 8)


def test_prefill_row_equals_decode_of_the_same_position(gpu_pool):
    """Cross-check without the oracle: every prompt token's output equals what decode attention gives for
    a context cut at that token, up to the rounding of the prompt kernel's softmax weights to fp16
    (2^-12 relative per weight; the decode kernel carries them as a bf16 head and tail, 2^-17)."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(6)
    hq, hkv, d, t = 32, 8, 128, 150
    gpu = GpuSeqs(gpu_pool, 1, hkv, d, 2, t)
    gpu.upload(0, bf16_randn(rng, (t, hkv, d)), bf16_randn(rng, (t, hkv, d)))
    q = torch_bf16_from_bits(bf16_randn(rng, (t, hq, d)))
    kt, vt = gpu.table_tensors()
    slot = torch.zeros(1, dtype=torch.int64, device="cuda")
    pre = torch.empty(t, hq, d, dtype=torch.float32, device="cuda")
    ops.prefill_attention(pre, q, kt, vt, hkv, d ** -0.5, [t], [t], slot)
    dec = torch.empty(t, hq, d, dtype=torch.float32, device="cuda")
    ops.paged_attention_v1(dec, q, kt, vt, hkv, d ** -0.5, torch.arange(1, t + 1, dtype=torch.int32, device="cuda"), 1,
                           t, None, "auto", 1.0, torch.zeros(t, dtype=torch.int64, device="cuda"))
    torch.cuda.synchronize()
    gpu.close()
    assert (pre - dec).abs().max().item() <= 2e-5 + 2.0 ** -12 * dec.abs().max().item()


def test_prompt_behind_a_shared_prefix(gpu_pool):
    """Prefix reuse end to end: a second sequence maps the first one's whole chunks instead of
    recomputing them, writes only its own rows (multi-token reshape_and_cache) and attends over prefix +
    own rows; the first sequence is untouched."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(8)
    hq, hkv, d = 32, 8, 128
    row = hkv * d * 2
    shared_rows, own_rows = 2050, 60                      # 2 whole chunks (2048 rows) + 2 rows copied
    gpu = GpuSeqs(gpu_pool, 2, hkv, d, 2, 4096)
    k_a, v_a = bf16_randn(rng, (2100, hkv, d)), bf16_randn(rng, (2100, hkv, d))
    gpu.upload(0, k_a, v_a)
    gpu.segs[1].share_prefix(gpu.segs[0], shared_rows * row, torch.cuda.current_stream().cuda_stream)
    assert gpu_pool.sharedBlocks() == 4                   # two chunks of K and of V
    nk, nv = bf16_randn(rng, (own_rows, hkv, d)), bf16_randn(rng, (own_rows, hkv, d))
    q = bf16_randn(rng, (own_rows, hq, d))
    kt, vt = gpu.table_tensors()
    slot_t = torch.tensor([1], dtype=torch.int64, device="cuda")
    # the step prologue reserves room for the new rows (maps a third chunk) and returns where they go
    slot_m = gpu_pool.extend_kv_cache_batch(None, None, [1], [own_rows * row], [gpu.segs[1]], [0], row, False)
    assert slot_m == [shared_rows * row]
    ops.reshape_and_cache(torch_bf16_from_bits(nk), torch_bf16_from_bits(nv), kt, vt,
                          torch.tensor(slot_m, dtype=torch.int64, device="cuda"), slot_t,
                          torch.tensor([own_rows], dtype=torch.int32, device="cuda"),
                          torch.zeros(1, dtype=torch.int32, device="cuda"), own_rows, hkv, d)
    out = torch.empty(own_rows, hq, d, dtype=torch.float32, device="cuda")
    ops.prefill_attention(out, torch_bf16_from_bits(q), kt, vt, hkv, d ** -0.5, [own_rows], [shared_rows + own_rows], slot_t)
    torch.cuda.synchronize()
    k_b = np.concatenate([k_a[:shared_rows], nk])
    v_b = np.concatenate([v_a[:shared_rows], nv])
    n = (shared_rows + own_rows) * row
    assert np.array_equal(gpu.download(1, n, which="k", dtype=np.uint16), k_b.reshape(-1))
    assert np.array_equal(gpu.download(1, n, which="v", dtype=np.uint16), v_b.reshape(-1))
    assert np.array_equal(gpu.download(0, 2100 * row, which="k", dtype=np.uint16), k_a.reshape(-1))
    expect = O.prefill_attention(O.bf16_to_f32(q), O.VTensorCache([k_a, k_b], [v_a, v_b], [1], hkv, d), d ** -0.5,
                                 [own_rows], [shared_rows + own_rows])
    got = out.cpu().numpy()
    gpu.close()
    assert np.all(np.abs(got - expect) <= 2e-3 + 2e-3 * np.abs(expect))
    assert gpu_pool.sharedBlocks() == 0


def test_logit_peaks_move_the_reference_point_mid_sequence(gpu_pool):
    """Rows whose logits tower over everything before them (by 15 to 60 in log2 units, far beyond the 8 the
    kernel tolerates before it moves a column's reference point), placed at the start, inside and at the end
    of stages and growing along the sequence: the accumulators are rescaled several times mid-sequence,
    for some columns of a wave and not for others (queries before a peak do not see it)."""
    d = 128
    u = np.where(np.arange(d) % 3 == 0, -1.0, 1.0).astype(np.float32)

    def peaks(q, ks, vs):
        qf = O.bf16_to_f32(q)
        qf += 3.0 * u                                     # every query leans towards u
        q[...] = O.f32_to_bf16(qf)
        for k in ks:
            for pos, c in ((0, 0.1), (31, 0.2), (32, 0.35), (200, 0.55), (333, 0.8), (511, 1.0)):
                if pos < k.shape[0]:
                    k[pos] = O.f32_to_bf16(np.broadcast_to(c * u, k[pos].shape))

    run_case(gpu_pool, 7, [512, 90, 300], [512, 90 + 260, 300], 32, 8, shape_inputs=peaks)
    run_case(gpu_pool, 8, [400], [400], 16, 8, alibi=True, shape_inputs=peaks)


def test_values_beyond_the_fp16_range(gpu_pool):
    """V travels as fp16 inside the prompt kernel; a bf16 cache can hold values fp16 cannot.  Values up to 6e4
    stay on the fast path; a unit that meets a larger one is computed a second time with V in bf16, so the
    prompt kernel agrees with the oracle (and with decode) for every bf16 input: huge values in a few rows, in
    all rows, next to ordinary ones whose weights they must not disturb, and behind masked positions."""
    import torch

    from glake_amd import _custom_ops as ops

    def clip(q, ks, vs):
        for v in vs:
            v[...] = O.f32_to_bf16(np.clip(O.bf16_to_f32(v) * 1.5e4, -6.0e4, 6.0e4))

    run_case(gpu_pool, 9, [70, 33], [70, 33 + 64], 32, 8, shape_inputs=clip, out_scale=1.5e4)

    def a_few_huge(q, ks, vs):
        # rows 5 and 300 of the first sequence and the last row of the second hold values around 1e8 and -3e20
        vs[0][5] = O.f32_to_bf16(np.full(vs[0][5].shape, 1.0e8, np.float32))
        vs[0][300, :, ::2] = O.f32_to_bf16(np.float32(-3.0e20))
        vs[1][-1] = O.f32_to_bf16(np.full(vs[1][-1].shape, 7.0e4, np.float32))

    # (the tolerance scales with the magnitude of V: 2e-3 relative to the largest value that enters an output)
    run_case(gpu_pool, 12, [400, 90, 64], [400, 90 + 40, 64], 32, 8, shape_inputs=a_few_huge, out_scale=3.0e20)

    def all_huge(q, ks, vs):
        for v in vs:
            v[...] = O.f32_to_bf16(O.bf16_to_f32(v) * np.float32(1.0e9))

    run_case(gpu_pool, 13, [130, 17], [130, 17 + 200], 16, 8, shape_inputs=all_huge, out_scale=1.0e9, fp8=False)

    # one key, value 1e5: the output is that value, bit for bit
    rng = np.random.default_rng(10)
    hq, hkv = 8, 8
    gpu = GpuSeqs(gpu_pool, 1, hkv, d := 128, 2, 1)
    v = O.f32_to_bf16(np.full((1, hkv, d), 1.0e5, np.float32))
    gpu.upload(0, bf16_randn(rng, (1, hkv, d)), v)
    kt, vt = gpu.table_tensors()
    out = torch.empty(1, hq, d, dtype=torch.float32, device="cuda")
    ops.prefill_attention(out, torch_bf16_from_bits(bf16_randn(rng, (1, hq, d))), kt, vt, hkv, d ** -0.5, [1], [1],
                          torch.zeros(1, dtype=torch.int64, device="cuda"))
    torch.cuda.synchronize()
    gpu.close()
    assert np.array_equal(out.cpu().numpy().reshape(hq, d), np.repeat(O.bf16_to_f32(v[0]), hq // hkv, axis=0))


def test_prompt_and_decode_agree_on_huge_values(gpu_pool):
    """The same rows through the prompt kernel (last position) and through the decode kernel: both keep V in
    bf16 where it matters, so they differ by fp32 summation order only."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(14)
    hq, hkv, d, n = 32, 8, 128, 777
    k = bf16_randn(rng, (n, hkv, d))
    v = O.f32_to_bf16(rng.standard_normal((n, hkv, d)).astype(np.float32) * np.float32(2.0e6))
    gpu = GpuSeqs(gpu_pool, 1, hkv, d, 2, n)
    gpu.upload(0, k, v)
    kt, vt = gpu.table_tensors()
    q = torch_bf16_from_bits(bf16_randn(rng, (n, hq, d)))
    slots = torch.zeros(1, dtype=torch.int64, device="cuda")
    out_p = torch.empty(n, hq, d, dtype=torch.float32, device="cuda")
    ops.prefill_attention(out_p, q, kt, vt, hkv, d ** -0.5, [n], [n], slots)
    out_d = torch.empty(1, hq, d, dtype=torch.float32, device="cuda")
    ops.paged_attention_v1(out_d, q[n - 1:], kt, vt, hkv, d ** -0.5, torch.tensor([n], dtype=torch.int32, device="cuda"), 1, n,
                           None, "auto", 1.0, slots)
    torch.cuda.synchronize()
    gpu.close()
    a, b = out_p[n - 1].cpu().numpy(), out_d[0].cpu().numpy()
    assert np.isfinite(a).all() and np.all(np.abs(a - b) <= 1e-4 * 2.0e6 + 1e-4 * np.abs(b))
