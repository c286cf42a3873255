"""Decode attention over the reference's whole surface of head sizes and 16-bit types
(vllm/attention/ops/paged_attn.py:33-34 [64, 80, 96, 112, 128, 256]; tests/kernels/test_attention.py:23-31
DTYPES half / bfloat16, NUM_HEADS (40, 40) and (64, 8), kv_cache_dtype auto / fp8, ALiBi), through the C ABI
against the oracle.

The oracle carries fp32 and bf16; an fp16 case is checked the way config 1 is: the oracle runs in fp32 on the
very values the GPU gets (they are exact in fp32), and the comparison is made on the kernel's fp32 output, i.e.
before the final rounding, at 2e-3 + 2e-3 |x| (fp8 caches: 3e-2 against the reference's protocol of dequantising
to the model's type first, 2e-3 against exact dequantisation).  The 16-bit output must be the round-to-nearest
of that fp32 output: numpy's float16 cast for fp16, the oracle's bf16 rounding for bf16."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bits_from_torch_bf16

pytestmark = pytest.mark.gpu

HEAD_SIZES = [64, 80, 96, 112, 128, 256]
LENS = [1, 15, 16, 17, 63, 64, 65, 257, 511, 512, 513, 1030, 2500]


def to_model(x32, dtype):
    """fp32 values -> (bits for upload, the same values in fp32)."""
    if dtype == "f16":
        h = x32.astype(np.float16)
        return h, h.astype(np.float32)
    b = O.f32_to_bf16(x32)
    return b, O.bf16_to_f32(b)


def check_partition_buffers(side, out, q32, k32, v32, lens, hq, hkv, d, scale, slopes):
    """The caller's buffers of paged_attention_v2 (csrc/attention/attention_kernels.cu:451-583): partition j of a
    sequence is rows [512 j, 512 j + 512).  tmp_out[j] is plain attention over those rows alone (a softmax does not
    see the constant that ALiBi's `- seq_len + 1` adds inside a partition, so the v1 oracle on a slice of the cache
    with the slice's own length gives it), max_logits and exp_sums come from a float64 q.K^T with the ALiBi bias of
    the row's place in the whole sequence (:404-419 qk_max carries it), and merging the buffers by the reference's
    rule (:515-582) gives `out` again."""
    import torch

    es, ml, tmp = (t.float().cpu().numpy() for t in side)
    g, tol = hq // hkv, 2e-3
    step = 2.0 ** -8 if side[2].dtype == torch.bfloat16 else 2.0 ** -11
    for i, n in enumerate(lens):
        np_i = (n + 511) // 512
        assert np.all(es[i, :, np_i:] == -7.0) and np.all(ml[i, :, np_i:] == -7.0) and np.all(tmp[i, :, np_i:] == -7.0)
        for j in range(np_i):
            lo, hi = 512 * j, min(n, 512 * j + 512)
            sl_k, sl_v = np.ascontiguousarray(k32[i][lo:hi]), np.ascontiguousarray(v32[i][lo:hi])
            part = O.paged_attention_v1(q32[i:i + 1], O.VTensorCache([sl_k], [sl_v], np.zeros(1, np.int64), hkv, d),
                                        scale, [hi - lo], slopes)[0]
            # tmp_out is stored in the model's type: one more rounding
            assert np.all(np.abs(tmp[i, :, j] - part) <= tol + (tol + step) * np.abs(part))
            for h in range(hq):
                s = scale * (sl_k[:, h // g].astype(np.float64) @ q32[i, h].astype(np.float64))
                if slopes is not None:
                    s = s + float(slopes[h]) * (np.arange(lo, hi) - n + 1)
                assert abs(ml[i, h, j] - s.max()) <= 1e-4 + 1e-5 * abs(s.max())
                sm = np.exp(s - s.max()).sum()
                assert abs(es[i, h, j] - sm) <= 1e-4 * sm
        m = ml[i, :, :np_i].max(axis=1, keepdims=True)
        w = es[i, :, :np_i] * np.exp(ml[i, :, :np_i] - m)
        merged = (tmp[i, :, :np_i] * w[..., None]).sum(axis=1) / (w.sum(axis=1, keepdims=True) + 1e-6)
        assert np.all(np.abs(merged - out[i]) <= 4e-3 + 4e-3 * np.abs(out[i]))


def run_case(vmm, seed, lens, hq, hkv, d, dtype, fp8=False, alibi=False, version="v1", partition_tokens=0):
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(lens)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    k_scale = v_scale = 1.0
    ks, vs, k32, v32, kref, vref = [], [], [], [], [], []
    for n in lens:
        kf = rng.standard_normal((n, hkv, d)).astype(np.float32)
        vf = rng.standard_normal((n, hkv, d)).astype(np.float32)
        ks.append(kf)
        vs.append(vf)
    if fp8:
        k_scale = float(max(np.abs(x).max() for x in ks) / 448.0)
        v_scale = float(max(np.abs(x).max() for x in vs) / 448.0)
        ks = [O.fp8_encode(x, k_scale) for x in ks]
        vs = [O.fp8_encode(x, v_scale) for x in vs]
        k32, v32 = [O.fp8_decode(c, k_scale) for c in ks], [O.fp8_decode(c, v_scale) for c in vs]
        # the reference's protocol: the cache converted back to the model's type (one more rounding)
        kref = [to_model(x, dtype)[1] for x in k32]
        vref = [to_model(x, dtype)[1] for x in v32]
    else:
        pairs_k, pairs_v = [to_model(x, dtype) for x in ks], [to_model(x, dtype) for x in vs]
        ks, vs = [p[0] for p in pairs_k], [p[0] for p in pairs_v]
        k32, v32 = [p[1] for p in pairs_k], [p[1] for p in pairs_v]
    q_bits, q32 = to_model(rng.standard_normal((b, hq, d)).astype(np.float32), dtype)
    scale = float(d) ** -0.5
    slopes = (rng.standard_normal(hq) * 0.1).astype(np.float32) if alibi else None
    gpu = GpuSeqs(vmm, b, hkv, d, 1 if fp8 else 2, max(lens), value_skew=256)
    for i in range(b):
        gpu.upload(i, ks[i], vs[i])
    kt, vt = gpu.table_tensors()
    q_t = torch.from_numpy(q_bits.view(np.int16).copy()).view(tdt).cuda()
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    slots = torch.arange(b, dtype=torch.int64, device="cuda")
    al = None if slopes is None else torch.from_numpy(slopes).cuda()
    out32 = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    out16 = torch.empty(b, hq, d, dtype=tdt, device="cuda")
    side = None
    for o in (out32, out16):
        if version == "v1":
            ops.paged_attention_v1(o, q_t, kt, vt, hkv, scale, sl, 1, max(lens), al, "fp8" if fp8 else "auto", k_scale,
                                   slots, v_scale=v_scale, partition_tokens=partition_tokens)
        else:
            parts = (max(lens) + 511) // 512 + 1           # one spare partition column: must stay untouched
            es = torch.full((b, hq, parts), -7.0, dtype=torch.float32, device="cuda")
            ml = torch.full((b, hq, parts), -7.0, dtype=torch.float32, device="cuda")
            tmp = torch.full((b, hq, parts, d), -7.0, dtype=tdt, device="cuda")
            ops.paged_attention_v2(o, es, ml, tmp, q_t, kt, vt, hkv, scale, sl, 1, max(lens), al,
                                   "fp8" if fp8 else "auto", k_scale, slots, v_scale=v_scale)
            side = (es, ml, tmp)
    torch.cuda.synchronize()
    gpu.close()
    got = out32.cpu().numpy()
    assert np.isfinite(got).all()
    want = O.paged_attention_v1(q32, O.VTensorCache(k32, v32, np.arange(b), hkv, d), scale, lens, slopes)
    if side is not None:
        check_partition_buffers(side, got, q32, k32, v32, lens, hq, hkv, d, scale, slopes)
    err = np.abs(got - want)
    ok = bool(np.all(err <= 2e-3 + 2e-3 * np.abs(want)))
    assert ok, f"max err {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}"
    if fp8:
        want_ref = O.paged_attention_v1(q32, O.VTensorCache(kref, vref, np.arange(b), hkv, d), scale, lens, slopes)
        assert bool(np.all(np.abs(got - want_ref) <= 3e-2 + 3e-2 * np.abs(want_ref)))
    if dtype == "f16":
        got16 = out16.cpu().numpy()
        assert np.array_equal(got16.view(np.uint16), got.astype(np.float16).view(np.uint16)), "fp16 out is not RNE(fp32 out)"
    else:
        assert np.array_equal(bits_from_torch_bf16(out16), O.f32_to_bf16(got)), "bf16 out is not RNE(fp32 out)"


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("d", HEAD_SIZES)
def test_every_head_size_gqa8(gpu_pool, d, dtype):
    run_case(gpu_pool, d, LENS, 64, 8, d, dtype)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("d", HEAD_SIZES)
def test_every_head_size_with_an_fp8_cache(gpu_pool, d, dtype):
    run_case(gpu_pool, 100 + d, LENS, 32, 8, d, dtype, fp8=True)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("d", [64, 80, 128, 256])
def test_forty_heads_without_grouping_and_alibi(gpu_pool, d, dtype):
    # NUM_HEADS = (40, 40) of the reference's matrix: every query head has its own kv head
    run_case(gpu_pool, 200 + d, [33, 700, 1, 2049, 130], 40, 40, d, dtype, alibi=True)


@pytest.mark.parametrize("d,dtype,fp8,alibi,heads", [
    (64, "f16", False, False, (32, 8)), (64, "bf16", False, True, (32, 8)), (80, "bf16", True, False, (32, 8)),
    (80, "f16", False, True, (32, 8)), (96, "f16", True, True, (32, 8)), (112, "bf16", False, False, (32, 8)),
    (112, "f16", True, True, (64, 8)), (128, "f16", False, True, (32, 8)), (128, "bf16", False, True, (32, 8)),
    (128, "f16", True, False, (32, 8)), (128, "bf16", True, True, (64, 8)), (256, "f16", False, False, (32, 8)),
    (256, "bf16", True, True, (16, 4)), (128, "bf16", False, True, (40, 2)), (96, "bf16", False, True, (40, 40))])
def test_split_k_interface_and_fixed_partitions_on_other_head_sizes(gpu_pool, d, dtype, fp8, alibi, heads):
    """The split-K interface with the caller's buffers over head sizes, fp16, fp8 rows and ALiBi, with head counts that
    take the variants of several kv heads per segment (32 over 8 at 64 to 112), the padded head sizes and kv heads
    served in parts (40 over 2): every partition's max, sum and partial result, not only the merged output."""
    hq, hkv = heads
    run_case(gpu_pool, 300 + d, [513, 2000, 100, 1025, 1], hq, hkv, d, dtype, fp8=fp8, alibi=alibi, version="v2")
    run_case(gpu_pool, 400 + d, [513, 2000, 100, 1025], hq, hkv, d, dtype, fp8=fp8, alibi=alibi, partition_tokens=256)


def test_long_context_on_a_small_head_and_a_large_one(gpu_pool):
    # many workgroups per (sequence, kv head): the merge of partial results of 64 and 256 columns
    run_case(gpu_pool, 7, [40000, 9000], 32, 8, 64, "f16")
    run_case(gpu_pool, 8, [30000, 100], 16, 4, 256, "bf16")


@pytest.mark.parametrize("d,dtype,fp8,alibi", [(64, "f16", False, False), (64, "bf16", True, True),
                                               (80, "bf16", False, False), (80, "f16", True, False),
                                               (96, "bf16", True, False), (96, "f16", False, True),
                                               (112, "f16", False, True), (112, "bf16", False, False),
                                               (128, "f16", False, False), (128, "f16", True, False),
                                               (128, "f16", False, True), (128, "f16", True, True),
                                               (256, "bf16", False, False), (256, "f16", True, True),
                                               (256, "bf16", True, False), (256, "f16", False, False)])
def test_prompt_attention_on_other_head_sizes(gpu_pool, d, dtype, fp8, alibi):
    """The prompt kernel on every head size of the reference's list, bf16 and fp16 models, 16-bit and fp8 caches,
    with and without ALiBi (shaped for bf16 at 128, which tests/test_gpu_prefill_attention.py covers).  Plain
    prompts and prompts behind cached rows, against the prompt oracle."""
    from glake_amd.attention.backends.vtensor import VTensorBackend

    VTensorBackend.get_impl_cls()(32, d, d ** -0.5, 8, None, None, "auto")     # the backend takes the head size
    run_prompt_case(gpu_pool, d + 7 * fp8 + 13 * alibi, [700, 20, 1, 400], [700, 33, 1, 1300], 32, 8, d, dtype, fp8, alibi)


def run_prompt_case(vmm, seed, query_lens, seq_lens, hq, hkv, d, dtype, fp8=False, alibi=False):
    """Prompts of query_lens tokens behind seq_lens - query_lens cached rows: fp32 output against the prompt oracle,
    and the output in the model's type equal to the fp32 one rounded once."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(seq_lens)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    k_scale, v_scale = (0.021, 0.033) if fp8 else (1.0, 1.0)

    def rows(n, sc):  # (what the cache holds, the same values in fp32)
        x = rng.standard_normal((n, hkv, d)).astype(np.float32)
        if fp8:
            codes = O.fp8_encode(x, sc)
            return codes, O.fp8_decode(codes, sc)
        return to_model(x, dtype)

    pairs_k = [rows(n, k_scale) for n in seq_lens]
    pairs_v = [rows(n, v_scale) for n in seq_lens]
    n_tok = sum(query_lens)
    q_bits, q32 = to_model(rng.standard_normal((n_tok, hq, d)).astype(np.float32), dtype)
    slopes = (rng.standard_normal(hq) * 0.3).astype(np.float32) if alibi else None
    gpu = GpuSeqs(vmm, b, hkv, d, 1 if fp8 else 2, max(seq_lens), value_skew=256)
    for i in range(b):
        gpu.upload(i, pairs_k[i][0], pairs_v[i][0])
    kt, vt = gpu.table_tensors()
    out = torch.empty(n_tok, hq, d, dtype=torch.float32, device="cuda")
    out16 = torch.empty(n_tok, hq, d, dtype=tdt, device="cuda")
    for o in (out, out16):
        ops.prefill_attention(o, torch.from_numpy(q_bits.view(np.int16).copy()).view(tdt).cuda(), kt, vt, hkv, d ** -0.5,
                              query_lens, seq_lens, torch.arange(b, dtype=torch.int64, device="cuda"),
                              None if slopes is None else torch.from_numpy(slopes).cuda(), "fp8" if fp8 else "auto",
                              k_scale, v_scale)
    torch.cuda.synchronize()
    gpu.close()
    want = O.prefill_attention(q32, O.VTensorCache([p[1] for p in pairs_k], [p[1] for p in pairs_v], np.arange(b), hkv, d),
                               d ** -0.5, query_lens, seq_lens, slopes)
    got = out.cpu().numpy()
    err = np.abs(got - want)
    assert bool(np.all(err <= 2e-3 + 2e-3 * np.abs(want))), f"max err {err.max():.3e}"
    # the output in the model's type is the fp32 result rounded once
    assert torch.equal(out16.cpu(), torch.from_numpy(got).to(tdt))


def run_append_case(vmm, seed, lens, hq, hkv, d, dtype, fp8=False, lens_from="host", alibi=True, partition_tokens=0):
    """vtkv_decode_append_attention: `lens` count the new token.  The new row must land in the cache as
    reshape_and_cache stores it (the 16-bit pattern, or the e4m3fn codes of value / scale) with nothing before it
    disturbed, and attention over all rows must agree with the oracle."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    eb = 1 if fp8 else 2
    row = hkv * d * eb
    b = len(lens)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    k_scale, v_scale = (0.021, 0.033) if fp8 else (1.0, 1.0)

    def stored(x32, sc):  # (bits in the cache, the values they stand for)
        if fp8:
            codes = O.fp8_encode(x32, sc)
            return codes, O.fp8_decode(codes, sc)
        return to_model(x32, dtype)

    gpu = GpuSeqs(vmm, b, hkv, d, eb, max(lens) + 1, value_skew=256)
    k_bits, v_bits, k32, v32 = [], [], [], []
    for i, t in enumerate(lens):
        kb, kf = stored(rng.standard_normal((t - 1, hkv, d)).astype(np.float32), k_scale)
        vb, vf = stored(rng.standard_normal((t - 1, hkv, d)).astype(np.float32), v_scale)
        gpu.upload(i, kb, vb)
        k_bits.append(kb), v_bits.append(vb), k32.append(kf), v32.append(vf)
    used = vmm.extend_kv_cache_batch(None, None, list(range(b)), [row] * b, gpu.segs, [0] * b, row, True)
    assert used == [(t - 1) * row for t in lens]
    q16, q32 = to_model(rng.standard_normal((b, hq, d)).astype(np.float32), dtype)
    nk16, nk32 = to_model(rng.standard_normal((b, hkv, d)).astype(np.float32), dtype)
    nv16, nv32 = to_model(rng.standard_normal((b, hkv, d)).astype(np.float32), dtype)
    slopes = (rng.standard_normal(hq) * 0.1).astype(np.float32) if alibi else None
    kt, vt = gpu.table_tensors()
    dev = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(tdt).cuda()
    out = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    lens_arg = list(lens) if lens_from == "host" else torch.tensor(lens, dtype=torch.int32, device="cuda")
    ops.decode_append_attention(out, dev(q16), dev(nk16).view(b, hkv * d), dev(nv16).view(b, hkv * d), kt, vt, hkv,
                                d ** -0.5, lens_arg, max(lens), None if slopes is None else torch.from_numpy(slopes).cuda(),
                                torch.arange(b, dtype=torch.int64, device="cuda"), partition_tokens=partition_tokens,
                                kv_cache_dtype="fp8" if fp8 else "auto", kv_scale=k_scale, v_scale=v_scale)
    torch.cuda.synchronize()
    # the appended rows, bit for bit, and nothing before them disturbed
    for i, t in enumerate(lens):
        nkb, nkf = stored(nk32[i:i + 1], k_scale)
        nvb, nvf = stored(nv32[i:i + 1], v_scale)
        want_k = np.concatenate([k_bits[i], nkb]).reshape(-1).view(np.uint8)
        want_v = np.concatenate([v_bits[i], nvb]).reshape(-1).view(np.uint8)
        assert np.array_equal(gpu.download(i, t * row, which="k"), want_k), ("k rows", i)
        assert np.array_equal(gpu.download(i, t * row, which="v"), want_v), ("v rows", i)
        k32[i], v32[i] = np.concatenate([k32[i], nkf]), np.concatenate([v32[i], nvf])
    gpu.close()
    want = O.paged_attention_v1(q32, O.VTensorCache(k32, v32, np.arange(b), hkv, d), d ** -0.5, lens, slopes)
    err = np.abs(out.cpu().numpy() - want)
    assert bool(np.all(err <= 2e-3 + 2e-3 * np.abs(want))), f"max err {err.max():.3e}"


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("lens_from", ["host", "device"])
def test_fused_append_for_fp16_models(gpu_pool, fp8, lens_from):
    """fp16 queries and new rows at head size 128, 16-bit and fp8 caches; lengths around tile and chunk boundaries,
    ALiBi, lengths from either side."""
    per = (2 << 20) // (8 * 128 * (1 if fp8 else 2))
    lens = [1, 2, 16, 17, 18, 33, 257, per - 1, per, per + 1, 2500]      # they count the new token
    run_append_case(gpu_pool, 90 + fp8, lens, 32, 8, 128, "f16", fp8=fp8, lens_from=lens_from)


@pytest.mark.parametrize("heads", [(32, 8), (40, 40), (15, 5), (64, 8), (71, 1), (40, 2)])
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("d", [64, 80, 96, 112, 256])
def test_fused_append_on_other_head_sizes(gpu_pool, d, dtype, heads):
    """The one-launch decode step for 16-bit caches of every other head size.  The head counts take each way the
    rows are streamed: several kv heads per wave tile (64, 80, 96 with 32 over 8 and 40 over 40; 64 and 96 with 64
    over 8), four kv heads per segment (112 with 32 over 8 and 40 over 40), one kv head per segment (256; 5 kv heads;
    80 and 112 with 64 over 8), kv heads of more than 16 query heads served in parts (71 over 1: parts of 15 heads,
    the shape of a multi-query model with head size 64; 40 over 2: parts of 10)."""
    hq, hkv = heads
    per = (2 << 20) // (hkv * d * 2)
    lens = [1, 2, 16, 17, 18, 33, 257, per, per + 1, 2 * per + 1, 1500]
    run_append_case(gpu_pool, 500 + d, lens, hq, hkv, d, dtype, lens_from="host", alibi=(hkv != 5))
    run_append_case(gpu_pool, 600 + d, [700, 65, 1, 1500, 2049, 17], hq, hkv, d, dtype, lens_from="device",
                    alibi=False, partition_tokens=256)


def test_fused_append_on_other_head_sizes_long_sequences(gpu_pool):
    # sequences spread over many workgroups: the new row's tile is then a segment of its own for some
    run_append_case(gpu_pool, 71, [30000, 1, 2, 5000], 32, 8, 80, "bf16", lens_from="device")
    run_append_case(gpu_pool, 72, [30000, 3, 4097], 32, 8, 112, "f16", lens_from="host")
    run_append_case(gpu_pool, 73, [20000, 1, 4097], 16, 4, 256, "bf16", lens_from="device")
    run_append_case(gpu_pool, 74, [30000, 1, 2, 5000], 16, 8, 64, "f16", lens_from="host")


def test_fused_append_refuses_fp8_rows_of_other_head_sizes(gpu_pool):
    with pytest.raises(Exception, match="16-bit rows"):
        run_append_case(gpu_pool, 75, [5, 40], 32, 8, 64, "bf16", fp8=True)


def test_workspace_is_sized_for_the_padded_head_size(gpu_pool):
    """A head size of 112 is held as 128 (fp8 rows pad to 64 elements): the workspace the library asks for must
    be sized for that, also through the split-K interface, where the grid and with it the scratch is exact."""
    run_case(gpu_pool, 964028853, [9, 4, 4, 10, 11, 6, 4, 10, 6, 5, 4261], 8, 8, 112, "f16", fp8=True, version="v2")
    run_case(gpu_pool, 5, [100, 3000, 17], 8, 8, 80, "bf16", fp8=True, version="v2")
    run_case(gpu_pool, 6, [100, 3000, 17], 16, 16, 80, "bf16", partition_tokens=64)
