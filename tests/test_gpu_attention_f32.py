"""Decode and prompt attention for float32 models (float32 queries over float32 rows), through the C ABI against
the oracle: the reference's third dtype (tests/kernels/test_attention.py:23 DTYPES = half, bfloat16, float) on its
head sizes, head counts, with ALiBi, through the plain entry point, the split-K interface with the caller's
buffers, the entry point that allocates nothing, the prompt path, the step plan and the backend.

Tolerance: |gpu - oracle| <= 1e-4 + 1e-4 |oracle| (both sides compute in fp32; the orders of summation differ)."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs

pytestmark = pytest.mark.gpu

TOL = 1e-4
EDGE = [1, 2, 7, 8, 9, 31, 32, 33, 63, 64, 65, 511, 512, 513, 1030, 2500]


def make_rows(rng, lens, hkv, d):
    k = [rng.standard_normal((t, hkv, d)).astype(np.float32) for t in lens]
    v = [rng.standard_normal((t, hkv, d)).astype(np.float32) for t in lens]
    return k, v


def run_case(vmm, seed, lens, hq, hkv, d=128, alibi=False, version="v1", entry="ops"):
    import torch

    from glake_amd import _C, _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(lens)
    slots = rng.permutation(b + 2)[:b]
    k, v = make_rows(rng, lens, hkv, d)
    gpu = GpuSeqs(vmm, b + 2, hkv, d, 4, max(lens), value_skew=256)
    k_all = [np.zeros((1, hkv, d), np.float32)] * (b + 2)
    v_all = [np.zeros((1, hkv, d), np.float32)] * (b + 2)
    for i in range(b):
        k_all[slots[i]], v_all[slots[i]] = k[i], v[i]
        gpu.upload(int(slots[i]), k[i], v[i])
    q = rng.standard_normal((b, hq, d)).astype(np.float32)
    scale = float(d) ** -0.5
    slopes = (rng.standard_normal(hq) * 0.1).astype(np.float32) if alibi else None
    kt, vt = gpu.table_tensors()
    q_t = torch.from_numpy(q).cuda()
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    slot_t = torch.tensor(slots, dtype=torch.int64, device="cuda")
    al = None if slopes is None else torch.from_numpy(slopes).cuda()
    out = torch.full((b, hq, d), -7.0, dtype=torch.float32, device="cuda")
    side = None
    if version == "v2":
        parts = (max(lens) + 511) // 512 + 1  # one spare partition column: must stay untouched
        es = torch.full((b, hq, parts), -7.0, dtype=torch.float32, device="cuda")
        ml = torch.full((b, hq, parts), -7.0, dtype=torch.float32, device="cuda")
        tmp = torch.full((b, hq, parts, d), -7.0, dtype=torch.float32, device="cuda")
        ops.paged_attention_v2(out, es, ml, tmp, q_t, kt, vt, hkv, scale, sl, 1, max(lens), al, "auto", 1.0, slot_t)
        side = (es, ml, tmp)
    elif entry == "noalloc":
        import ctypes as C

        lib = _C.lib()
        p = lambda t: C.c_void_p(t.data_ptr())
        _C.check(lib.vtkv_decode_attention_noalloc(
            p(out), p(q_t), ops._ptr(kt), ops._ptr(vt), p(slot_t), p(sl), b, hq, hkv, d, q_t.stride(0), scale, max(lens),
            None if al is None else p(al), _C.F32, _C.F32, _C.F32, 1.0, 1.0, ops._stream()))
    else:
        ops.paged_attention_v1(out, q_t, kt, vt, hkv, scale, sl, 1, max(lens), al, "auto", 1.0, slot_t)
    torch.cuda.synchronize()
    gpu.close()
    got = out.cpu().numpy()
    want = O.paged_attention_v1(q, O.VTensorCache(k_all, v_all, slots, hkv, d), scale, lens, slopes)
    err = np.abs(got - want)
    assert bool(np.all(err <= TOL + TOL * np.abs(want))), f"max err {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}"
    if side is not None:
        import test_gpu_head_sizes as H

        H.check_partition_buffers(side, got, q, k, v, lens, hq, hkv, d, scale, slopes)
    return got


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (8, 8), (16, 1), (40, 2), (7, 7), (6, 3)])
def test_edge_lengths_and_head_counts(gpu_pool, hq, hkv):
    # groups of 4, 8, 1, 16 (two passes of 8 heads), 20 (three passes, the last one half empty), 1, 2
    run_case(gpu_pool, 1, EDGE, hq, hkv)


@pytest.mark.parametrize("d", [64, 80, 96, 112, 128, 256])
@pytest.mark.parametrize("alibi", [False, True])
def test_every_head_size(gpu_pool, d, alibi):
    # NUM_HEADS of the reference's matrix: (40, 40) and (64, 8)
    run_case(gpu_pool, d, [33, 700, 1, 2049, 130], 40, 40, d=d, alibi=alibi)
    run_case(gpu_pool, d + 1, [513, 64, 1500], 64, 8, d=d, alibi=alibi)


def test_config1_shape(gpu_pool):
    """BASELINE config 1 as it is written: fp32, 8 sequences of 128..1024 rows, 32 query heads over 8 kv heads."""
    import torch

    lens = torch.randint(128, 1025, (8,), generator=torch.Generator().manual_seed(1000)).tolist()
    run_case(gpu_pool, 1000, lens, 32, 8)


def test_long_sequences_of_many_partitions(gpu_pool):
    run_case(gpu_pool, 3, [40000, 1, 9000], 32, 8)
    run_case(gpu_pool, 4, [30000], 8, 1, d=256)


@pytest.mark.parametrize("d,alibi,heads", [(128, False, (32, 8)), (128, True, (64, 8)), (80, True, (40, 40)),
                                           (256, False, (16, 4)), (64, True, (40, 2))])
def test_split_k_interface_fills_the_callers_buffers(gpu_pool, d, alibi, heads):
    run_case(gpu_pool, 5 + d, [513, 2000, 100, 1025, 1], heads[0], heads[1], d=d, alibi=alibi, version="v2")


def test_entry_point_that_allocates_nothing(gpu_pool):
    a = run_case(gpu_pool, 6, [700, 65, 1, 1500, 2049, 17], 32, 8, entry="noalloc")
    b = run_case(gpu_pool, 6, [700, 65, 1, 1500, 2049, 17], 32, 8)
    assert np.array_equal(a, b)


def test_many_sequences(gpu_pool):
    rng = np.random.default_rng(8)
    run_case(gpu_pool, 8, [int(x) for x in rng.integers(1, 60, 300)], 8, 2, d=64)


@pytest.mark.parametrize("d,alibi,heads", [(128, False, (32, 8)), (128, True, (8, 8)), (96, True, (12, 4)),
                                           (256, False, (16, 4))])
def test_prompt_attention(gpu_pool, d, alibi, heads):
    """Prompts, and prompts behind cached rows, of a float32 model against the prompt oracle."""
    import torch

    from glake_amd import _custom_ops as ops

    hq, hkv = heads
    rng = np.random.default_rng(20 + d)
    query_lens, seq_lens = [300, 20, 1, 77], [300, 33, 1, 500]
    b = len(seq_lens)
    k, v = make_rows(rng, seq_lens, hkv, d)
    n_tok = sum(query_lens)
    q = rng.standard_normal((n_tok, hq, d)).astype(np.float32)
    slopes = (rng.standard_normal(hq) * 0.3).astype(np.float32) if alibi else None
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 4, max(seq_lens), value_skew=256)
    for i in range(b):
        gpu.upload(i, k[i], v[i])
    kt, vt = gpu.table_tensors()
    out = torch.empty(n_tok, hq, d, dtype=torch.float32, device="cuda")
    ops.prefill_attention(out, torch.from_numpy(q).cuda(), kt, vt, hkv, d ** -0.5, query_lens, seq_lens,
                          torch.arange(b, dtype=torch.int64, device="cuda"),
                          None if slopes is None else torch.from_numpy(slopes).cuda())
    torch.cuda.synchronize()
    gpu.close()
    want = O.prefill_attention(q, O.VTensorCache(k, v, np.arange(b), hkv, d), d ** -0.5, query_lens, seq_lens, slopes)
    err = np.abs(out.cpu().numpy() - want)
    assert bool(np.all(err <= TOL + TOL * np.abs(want))), f"max err {err.max():.3e}"


def test_refuses_mixed_types(gpu_pool):
    import torch

    from glake_amd import _C, _custom_ops as ops

    gpu = GpuSeqs(gpu_pool, 1, 8, 128, 4, 64)
    gpu.upload(0, np.zeros((4, 8, 128), np.float32), np.zeros((4, 8, 128), np.float32))
    kt, vt = gpu.table_tensors()
    q = torch.zeros(1, 32, 128, dtype=torch.float32, device="cuda")
    sl = torch.tensor([4], dtype=torch.int32, device="cuda")
    slot = torch.zeros(1, dtype=torch.int64, device="cuda")
    with pytest.raises(_C.VtkvError, match="float32 cache"):
        ops.paged_attention_v1(torch.empty_like(q), q, kt, vt, 8, 1.0, sl, 1, 4, None, "fp8", 1.0, slot)
    with pytest.raises(_C.VtkvError, match="float32"):
        ops.paged_attention_v1(torch.empty(1, 32, 128, dtype=torch.bfloat16, device="cuda"), q, kt, vt, 8, 1.0, sl, 1, 4,
                               None, "auto", 1.0, slot)
    gpu.close()


def test_step_plan_runs_a_float32_model(gpu_pool):
    """DecodeStepPlan with a float32 model: reshape_and_cache + attention as two launches per step; rows bit for bit,
    results against the oracle over three steps."""
    import torch

    from glake_amd.worker.step import DecodeStepPlan

    rng = np.random.default_rng(31)
    hq, hkv, d = 32, 8, 128
    lens = [5, 300, 1023, 64]
    b = len(lens)
    row = hkv * d * 4
    k, v = make_rows(rng, lens, hkv, d)
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 4, max(lens) + 8, value_skew=256)
    for i in range(b):
        gpu.upload(i, k[i], v[i])
    kt, vt = gpu.table_tensors()
    plan = DecodeStepPlan(gpu.segs, list(range(b)), kt, vt, hq, hkv, d, d ** -0.5, model_dtype=torch.float32)
    assert not plan.fused
    for step in range(3):
        q = rng.standard_normal((b, hq, d)).astype(np.float32)
        nk = rng.standard_normal((b, hkv, d)).astype(np.float32)
        nv = rng.standard_normal((b, hkv, d)).astype(np.float32)
        out = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
        plan.run(torch.from_numpy(q).cuda(), torch.from_numpy(nk).cuda().view(b, -1), torch.from_numpy(nv).cuda().view(b, -1), out)
        torch.cuda.synchronize()
        k = [np.concatenate([k[i], nk[i:i + 1]]) for i in range(b)]
        v = [np.concatenate([v[i], nv[i:i + 1]]) for i in range(b)]
        now = [t + step + 1 for t in lens]
        want = O.paged_attention_v1(q, O.VTensorCache(k, v, np.arange(b), hkv, d), d ** -0.5, now, None)
        err = np.abs(out.cpu().numpy() - want)
        assert bool(np.all(err <= TOL + TOL * np.abs(want))), f"step {step}: max err {err.max():.3e}"
    for i in range(b):
        assert np.array_equal(gpu.download(i, (lens[i] + 3) * row, which="k"), k[i].reshape(-1).view(np.uint8))
        assert np.array_equal(gpu.download(i, (lens[i] + 3) * row, which="v"), v[i].reshape(-1).view(np.uint8))
    gpu.close()


def test_backend_prompt_run_then_decode_with_a_float32_model(gpu_pool):
    """VTensorImpl.forward as the model code drives it (llama.py:307-351 -> xformers.py:269-433) for a float32
    model over a float32 cache: a batch of prompts, then two decode steps."""
    import torch

    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step import prepare_step

    hq, hkv, d, max_seqs = 32, 8, 128, 4
    row = hkv * d * 4
    rng = np.random.default_rng(3)
    eng = CacheEngine(1, hkv, d, torch.float32, max_seqs, 4096)
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    slots = [2, 0, 3]
    lens = [37, 600, 5]
    dev = torch.device("cuda")
    n_tok = sum(lens)

    def metadata(prefill: bool, lens):
        starts = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        meta = VTensorBackend.make_metadata(
            num_prefills=len(slots) if prefill else 0, num_prefill_tokens=n_tok if prefill else 0,
            num_decode_tokens=0 if prefill else len(slots),
            slot_mapping=torch.tensor(slots, dtype=torch.int64, device=dev), seq_lens=list(lens) if prefill else None,
            seq_lens_tensor=torch.tensor(lens, dtype=torch.int32, device=dev), max_query_len=max(lens) if prefill else None,
            max_prefill_seq_len=max(lens) if prefill else 0, max_decode_seq_len=0 if prefill else max(lens),
            query_start_loc=torch.tensor(starts, device=dev) if prefill else None, seq_start_loc=None,
            context_lens_tensor=None, block_tables=None, is_extend=0, kv_batch_stride=eng.kv_batch_stride,
            kv_num_heads=hkv, kv_head_size=d, max_seq_len=max(lens), slot_mapping_list=slots,
            set_used_size=[0] * len(slots), extend_seq_list=[-1] * len(slots), use_cuda_graph=False)
        if prefill:
            meta.cache_seq_lens = torch.tensor(starts[:-1], dtype=torch.int32, device=dev)
        meta.k_cache_segment_ptr_list = eng.k_cache_ptr
        meta.v_cache_segment_ptr_list = eng.v_cache_ptr
        meta.kvcache_segment = [eng.vmm_kvcache_segment[s] for s in slots]
        prepare_step(meta, eng.gpu_cache, model_elem_bytes=4)
        return meta

    kc, vc = eng.gpu_cache[0]
    q = rng.standard_normal((n_tok, hq * d)).astype(np.float32)
    k = rng.standard_normal((n_tok, hkv * d)).astype(np.float32)
    v = rng.standard_normal((n_tok, hkv * d)).astype(np.float32)
    out = impl.forward(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), kc, vc,
                       metadata(True, lens))
    kb = [np.zeros((1, hkv, d), np.float32)] * max_seqs
    vb = list(kb)
    row0 = 0
    for s, n in zip(slots, lens):
        kb[s], vb[s] = k[row0:row0 + n].reshape(n, hkv, d), v[row0:row0 + n].reshape(n, hkv, d)
        row0 += n
    want = O.prefill_attention(q.reshape(n_tok, hq, d), O.VTensorCache(kb, vb, slots, hkv, d), d ** -0.5, lens, lens)
    err = np.abs(out.cpu().numpy().reshape(n_tok, hq, d) - want)
    assert bool(np.all(err <= TOL + TOL * np.abs(want))), f"prompts: max err {err.max():.3e}"
    for step in range(2):
        lens = [n + 1 for n in lens]
        meta = metadata(False, lens)
        assert meta.slot_m.tolist() == [(n - 1) * row for n in lens]
        q1 = rng.standard_normal((len(slots), hq * d)).astype(np.float32)
        k1 = rng.standard_normal((len(slots), hkv * d)).astype(np.float32)
        v1 = rng.standard_normal((len(slots), hkv * d)).astype(np.float32)
        out = impl.forward(torch.from_numpy(q1).cuda(), torch.from_numpy(k1).cuda(), torch.from_numpy(v1).cuda(), kc, vc, meta)
        for i, s in enumerate(slots):
            kb[s] = np.concatenate([kb[s], k1[i].reshape(1, hkv, d)])
            vb[s] = np.concatenate([vb[s], v1[i].reshape(1, hkv, d)])
        want = O.paged_attention_v1(q1.reshape(len(slots), hq, d), O.VTensorCache(kb, vb, slots, hkv, d), d ** -0.5, lens)
        err = np.abs(out.cpu().numpy().reshape(len(slots), hq, d) - want)
        assert bool(np.all(err <= TOL + TOL * np.abs(want))), f"decode step {step}: max err {err.max():.3e}"
    eng.close()


def test_float32_calls_leave_the_arrival_counters_of_the_16_bit_kernels_alone(gpu_pool):
    """The workspace of a stream is shared by all calls on it, and the 16-bit kernels keep their arrival counters at
    its start, at zero between calls: a float32 call that writes partial results must leave them alone.  A
    float32 call of many partitions, then 16-bit calls that merge inside the stream kernel (which is what reads
    the counters)."""
    import test_gpu_attention as A
    from glake_amd import _C

    run_case(gpu_pool, 3, [40000, 1, 9000], 32, 8)
    run_case(gpu_pool, 5, [513, 2000, 100, 1025, 1] * 8, 64, 8)
    lib = _C.lib()
    _C.check(lib.vtkv_set_fused_merge(1))
    try:
        A.run_case(gpu_pool, 61, [1, 15, 16, 17, 63, 64, 65, 511, 1030], 71, 1)
        A.run_case(gpu_pool, 62, [30000, 3, 9000, 700], 32, 8)
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
