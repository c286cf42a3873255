"""What the mathematics fixes about the oracle, independent of any implementation: a float64
textbook softmax(QK^T)V, closed forms and invariances (each chosen so that a dropped term, a
wrong index or a transposed operand fails it)."""
import numpy as np
import pytest

from oracle import oracle as O


def make_paged(rng, lens, hkv, d, dtype, bs=16, extra_blocks=5):
    x = 4 if dtype == "f32" else 8
    nblk = [(n + bs - 1) // bs for n in lens]
    nb = sum(nblk) + extra_blocks
    k = rng.standard_normal((nb, hkv, d // x, bs, x)).astype(np.float32)
    v = rng.standard_normal((nb, hkv, d, bs)).astype(np.float32)
    perm = rng.permutation(nb)
    bt = np.zeros((len(lens), max(nblk)), np.int32)
    at = 0
    for i, n in enumerate(nblk):
        bt[i, :n] = perm[at:at + n]
        at += n
    if dtype == "bf16":
        k, v = O.f32_to_bf16(k), O.f32_to_bf16(v)
    return k, v, bt


def rows_of(k, v, bt, seq, n, head, dtype):
    """Token-major [n, D] K and V rows of one kv head, gathered by the reference test's rule
    (tests/kernels/test_attention.py:82-94)."""
    bs = k.shape[3]
    kr, vr = [], []
    for t in range(n):
        blk, off = bt[seq, t // bs], t % bs
        kr.append(k[blk, head, :, off, :].reshape(-1))
        vr.append(v[blk, head, :, off])
    kr, vr = np.stack(kr), np.stack(vr)
    if dtype == "bf16":
        kr, vr = O.bf16_to_f32(kr), O.bf16_to_f32(vr)
    return kr, vr


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("version", [1, 2])
@pytest.mark.parametrize("alibi", [False, True])
def test_textbook_float64(dtype, version, alibi):
    rng = np.random.default_rng(3)
    lens, hq, hkv, d = [1, 17, 512, 700, 1030], 8, 2, 128
    k, v, bt = make_paged(rng, lens, hkv, d, dtype)
    q = rng.standard_normal((len(lens), hq, d)).astype(np.float32)
    slopes = (rng.standard_normal(hq) * 0.05).astype(np.float32) if alibi else None
    qq = O.f32_to_bf16(q) if dtype == "bf16" else q
    fn = O.paged_attention_v1 if version == 1 else O.paged_attention_v2
    got = fn(qq, O.PagedCache(k, v, bt), d ** -0.5, lens, slopes)
    got = O.bf16_to_f32(got) if dtype == "bf16" else got
    qf = O.bf16_to_f32(qq) if dtype == "bf16" else q
    for s, n in enumerate(lens):
        for h in range(hq):
            kr, vr = rows_of(k, v, bt, s, n, h // (hq // hkv), dtype)
            want = O.textbook_attention(qf[s, h], kr, vr, d ** -0.5, None if slopes is None else slopes[h])
            tol = 2e-5 if dtype == "f32" else 2.0 ** -8  # bf16 store + (v2) bf16 partials
            assert np.all(np.abs(got[s, h] - want) <= tol * (1 + np.abs(want))), (s, h, np.abs(got[s, h] - want).max())


def test_single_token_is_value_row():
    rng = np.random.default_rng(4)
    k, v, bt = make_paged(rng, [1, 1], 2, 128, "f32")
    q = rng.standard_normal((2, 8, 128)).astype(np.float32)
    out = O.paged_attention_v1(q, O.PagedCache(k, v, bt), 0.1, [1, 1])
    for s in range(2):
        for h in range(8):
            assert np.array_equal(out[s, h], v[bt[s, 0], h // 4, :, 0])


def test_probabilities_sum_to_one_and_constant_values_pass_through():
    rng = np.random.default_rng(5)
    lens = [33, 513]
    k, v, bt = make_paged(rng, lens, 2, 128, "f32")
    v[:] = 3.25  # sum_t p_t * c = c for any softmax
    q = rng.standard_normal((2, 8, 128)).astype(np.float32)
    for fn in (O.paged_attention_v1, O.paged_attention_v2):
        out = fn(q, O.PagedCache(k, v, bt), 128 ** -0.5, lens)
        assert np.allclose(out, 3.25, rtol=0, atol=5e-6)  # fp32 rounding of ~500 probabilities


def test_invariant_under_relabelling_physical_blocks():
    rng = np.random.default_rng(6)
    lens = [100, 600]
    k, v, bt = make_paged(rng, lens, 2, 128, "f32")
    q = rng.standard_normal((2, 8, 128)).astype(np.float32)
    base = O.paged_attention_v1(q, O.PagedCache(k, v, bt), 128 ** -0.5, lens)
    perm = rng.permutation(k.shape[0])          # new id of old block i is perm[i]
    k2, v2 = np.empty_like(k), np.empty_like(v)
    k2[perm], v2[perm] = k, v
    out = O.paged_attention_v1(q, O.PagedCache(k2, v2, perm[bt].astype(np.int32)), 128 ** -0.5, lens)
    assert np.array_equal(out, base)


def test_partition_count_does_not_change_the_result():
    rng = np.random.default_rng(7)
    lens = [511, 512, 513, 2048, 2500]
    k, v, bt = make_paged(rng, lens, 2, 128, "f32")
    q = rng.standard_normal((len(lens), 8, 128)).astype(np.float32)
    c = O.PagedCache(k, v, bt)
    v1 = O.paged_attention_v1(q, c, 128 ** -0.5, lens)
    v2 = O.paged_attention_v2(q, c, 128 ** -0.5, lens)
    assert np.all(np.abs(v1 - v2) <= 2e-6 * (1 + np.abs(v1)))
    assert np.array_equal(v1[0], v2[0])  # one partition: v2 bypasses the merge (csrc/cpu/attention.cpp:476,529)


def test_lse_merge_closed_form():
    """Two partitions by hand: out = (o1 l1 e^{m1-m} + o2 l2 e^{m2-m}) / (l1 e^{m1-m} + l2 e^{m2-m})."""
    rng = np.random.default_rng(8)
    n = 700
    k, v, bt = make_paged(rng, [n], 1, 128, "f32")
    q = rng.standard_normal((1, 1, 128)).astype(np.float32)
    out, es, ml, tmp = O.paged_attention_v2(q, O.PagedCache(k, v, bt), 128 ** -0.5, [n], return_partials=True)
    kr, vr = rows_of(k, v, bt, 0, n, 0, "f32")
    s = (kr.astype(np.float64) @ q[0, 0].astype(np.float64)) * 128 ** -0.5
    parts = [(0, 512), (512, n)]
    m = [s[a:b].max() for a, b in parts]
    l = [np.exp(s[a:b] - mi).sum() for (a, b), mi in zip(parts, m)]
    o = [np.exp(s[a:b] - mi) @ vr[a:b].astype(np.float64) / li for (a, b), mi, li in zip(parts, m, l)]
    mm = max(m)
    w = [li * np.exp(mi - mm) for li, mi in zip(l, m)]
    want = (o[0] * w[0] + o[1] * w[1]) / (w[0] + w[1])
    assert np.allclose(out[0, 0], want, rtol=2e-5, atol=2e-6)
    assert np.allclose(ml[0, 0], m, rtol=1e-6) and np.allclose(tmp[0, 0], np.stack(o), rtol=2e-5, atol=2e-6)
    # after the call exp_sums holds the rescale factors (csrc/cpu/attention.cpp:100-117)
    assert np.allclose(es[0, 0], np.array(w) / sum(w), rtol=1e-5)


def test_gqa_heads_of_one_group_with_equal_queries_agree_and_groups_differ():
    rng = np.random.default_rng(9)
    lens = [300]
    k, v, bt = make_paged(rng, lens, 2, 128, "f32")
    q = np.repeat(rng.standard_normal((1, 1, 128)).astype(np.float32), 8, axis=1)
    out = O.paged_attention_v1(q, O.PagedCache(k, v, bt), 128 ** -0.5, lens)
    assert np.array_equal(out[0, 0], out[0, 3]) and np.array_equal(out[0, 4], out[0, 7])
    assert not np.allclose(out[0, 0], out[0, 4])  # heads 0-3 read kv head 0, heads 4-7 kv head 1


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_contiguous_layout_equals_paged_layout(dtype):
    """BASELINE config 1 at reduced batch: the same tokens in the reference's paged block-16 layout
    and in per-sequence contiguous [T,Hkv,D] ranges give bit-identical results."""
    rng = np.random.default_rng(1000)
    lens = rng.integers(128, 1025, 4).tolist()
    hq, hkv, d = 32, 8, 128
    k, v, bt = make_paged(rng, lens, hkv, d, dtype)
    q = rng.standard_normal((len(lens), hq, d)).astype(np.float32)
    if dtype == "bf16":
        q = O.f32_to_bf16(q)
    paged = O.paged_attention_v1(q, O.PagedCache(k, v, bt), d ** -0.5, lens)
    kb, vb = [], []
    bs = 16
    for s, n in enumerate(lens):
        kk = np.stack([k[bt[s, t // bs], :, :, t % bs, :].reshape(hkv, d) for t in range(n)])
        vv = np.stack([v[bt[s, t // bs], :, :, t % bs] for t in range(n)])
        kb.append(np.ascontiguousarray(kk))
        vb.append(np.ascontiguousarray(vv))
    slots = np.array([2, 0, 3, 1])
    order = np.argsort(slots)
    cache = O.VTensorCache([kb[i] for i in order], [vb[i] for i in order], slots, hkv, d)
    assert np.array_equal(O.paged_attention_v1(q, cache, d ** -0.5, lens), paged)
    assert np.array_equal(O.paged_attention_v2(q, cache, d ** -0.5, lens),
                          O.paged_attention_v2(q, O.PagedCache(k, v, bt), d ** -0.5, lens))


def test_vtensor_scatter_brute_force():
    """csrc/cache_kernels.cu:176-199 by hand on tiny inputs: decode form, prefill form, skipped rows,
    strided sources."""
    rng = np.random.default_rng(10)
    hkv, d, eb = 2, 8, 2
    row = hkv * d
    bufs_k = [np.zeros(40 * row, np.uint16) for _ in range(3)]
    bufs_v = [np.zeros(40 * row, np.uint16) for _ in range(3)]
    kp = np.array([b.ctypes.data for b in bufs_k], np.int64)
    vp = np.array([b.ctypes.data for b in bufs_v], np.int64)
    # decode: 3 sequences, one row each, middle one skipped
    fused = rng.integers(0, 65535, (3, 3, hkv, d)).astype(np.uint16)
    key, value = fused[:, 1], fused[:, 2]
    slot_m = np.array([4 * row * eb, -1, 0], np.int64)
    slot_ids = np.array([2, 1, 0], np.int64)
    O.reshape_and_cache_vtensor(key, value, kp, vp, slot_m, slot_ids, [1, 1, 1], [0, 0, 0], 1, hkv, d)
    assert np.array_equal(bufs_k[2][4 * row:5 * row], key[0].reshape(-1))
    assert np.array_equal(bufs_v[0][:row], value[2].reshape(-1))
    assert not bufs_k[1].any() and bufs_k[2][:4 * row].sum() == 0
    # prefill: lengths 3 and 5 packed back to back, written from row offsets 1 and 2
    key = rng.integers(0, 65535, (8, hkv, d)).astype(np.uint16)
    value = rng.integers(0, 65535, (8, hkv, d)).astype(np.uint16)
    for b in bufs_k + bufs_v:
        b[:] = 0
    O.reshape_and_cache_vtensor(key, value, kp, vp, np.array([row * eb, 2 * row * eb], np.int64),
                                np.array([1, 0], np.int64), [3, 5], [0, 3], 5, hkv, d)
    assert np.array_equal(bufs_k[1][row:4 * row], key[0:3].reshape(-1)) and not bufs_k[1][4 * row:].any()
    assert np.array_equal(bufs_v[0][2 * row:7 * row], value[3:8].reshape(-1))


def test_prefill_oracle_equals_whole_matrix_causal_attention():
    """The prefill oracle (decode oracle applied per query position) against the float64 whole-matrix
    form with a lower-right aligned causal mask, with and without a cached prefix and ALiBi."""
    rng = np.random.default_rng(41)
    hq, hkv, d = 8, 2, 128
    g = hq // hkv
    query_lens, seq_lens = [5, 1, 19, 33], [5, 7, 40, 33]
    slots = [2, 0, 3, 1]
    k = [rng.standard_normal((40, hkv, d)).astype(np.float32) for _ in range(4)]
    v = [rng.standard_normal((40, hkv, d)).astype(np.float32) for _ in range(4)]
    q = rng.standard_normal((sum(query_lens), hq, d)).astype(np.float32)
    scale = d ** -0.5
    for slopes in (None, rng.standard_normal(hq).astype(np.float32)):
        cache = O.VTensorCache(k, v, slots, hkv, d)
        got = O.prefill_attention(q, cache, scale, query_lens, seq_lens, slopes)
        row = 0
        for b, (ql, sl) in enumerate(zip(query_lens, seq_lens)):
            for h in range(hq):
                want = O.textbook_causal_attention(q[row:row + ql, h], k[slots[b]][:sl, h // g], v[slots[b]][:sl, h // g],
                                                   scale, sl - ql, None if slopes is None else float(slopes[h]))
                np.testing.assert_allclose(got[row:row + ql, h], want, rtol=2e-5, atol=2e-6)
            row += ql
