"""GPU parity of decode attention: the HIP split-K kernel, called through the C ABI, against the
CPU oracle on the same seeded inputs.

Tolerance for bf16 KV: |gpu - oracle| <= 2e-3 + 2e-3 * |oracle|, checked on the values BEFORE the
final store to bf16 on both sides (fp32 `out` on the GPU; the oracle run with an fp32 query/output
holding the same bf16-representable values): a bf16 store alone moves a value by up to 2^-8 = 3.9e-3
relative, so two correctly computed bf16 tensors can differ by more than the tolerance.  For the
bf16 output the checks are: it is the round-to-nearest-even of the kernel's fp32 result bit for
bit, and it is never more than one bf16 step from the oracle's bf16 output."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu

ATOL = RTOL = 2e-3


def run_case(vmm, seed, seq_lens, hq, hkv, d=128, partition_tokens=0, alibi=False, shuffle_slots=True, version="v1",
             bf16_step_check=True):
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(seed)
    b = len(seq_lens)
    num_slots = b + 3
    slots = rng.permutation(num_slots)[:b] if shuffle_slots else np.arange(b)
    gpu = GpuSeqs(vmm, num_slots, hkv, d, 2, max(seq_lens))
    k_host = [np.zeros((1, hkv, d), np.uint16) for _ in range(num_slots)]
    v_host = [np.zeros((1, hkv, d), np.uint16) for _ in range(num_slots)]
    for i, t in enumerate(seq_lens):
        k_host[slots[i]] = bf16_randn(rng, (t, hkv, d))
        v_host[slots[i]] = bf16_randn(rng, (t, hkv, d))
        gpu.upload(int(slots[i]), k_host[slots[i]], v_host[slots[i]])
    q = bf16_randn(rng, (b, hq, d))
    scale = float(d) ** -0.5
    slopes = rng.standard_normal(hq).astype(np.float32) if alibi else None

    cache = O.VTensorCache(k_host, v_host, slots, hkv, d)
    expect = O.paged_attention_v1(q, cache, scale, seq_lens, slopes)               # bf16, round to nearest
    expect32 = O.paged_attention_v1(O.bf16_to_f32(q), cache, scale, seq_lens, slopes)  # before the final rounding

    kt, vt = gpu.table_tensors()
    out = torch.empty(b, hq, d, dtype=torch.bfloat16, device="cuda")
    out32 = torch.empty(b, hq, d, dtype=torch.float32, device="cuda")
    q_t = torch_bf16_from_bits(q)
    sl_t = torch.tensor(seq_lens, dtype=torch.int32, device="cuda")
    slot_t = torch.tensor(slots, dtype=torch.int64, device="cuda")
    al_t = None if slopes is None else torch.from_numpy(slopes).cuda()
    for o in (out, out32):
        if version == "v1":
            ops.paged_attention_v1(o, q_t, kt, vt, hkv, scale, sl_t, 1, max(seq_lens), al_t, "auto", 1.0, slot_t,
                                   partition_tokens=partition_tokens)
        else:
            ops.paged_attention_v2(o, None, None, None, q_t, kt, vt, hkv, scale, sl_t, 1, max(seq_lens), al_t,
                                   "auto", 1.0, slot_t)
    torch.cuda.synchronize()
    got_bits = bits_from_torch_bf16(out)
    got = out32.cpu().numpy()
    want = O.bf16_to_f32(expect)
    gpu.close()
    assert np.array_equal(got_bits, O.f32_to_bf16(got)), "bf16 output is not RNE(fp32 output)"
    err = np.abs(got - expect32)
    bound = ATOL + RTOL * np.abs(expect32)
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert np.all(err <= bound), (f"max err {err.max():.3e}, worst excess {(err - bound).max():.3e} at (seq, head, d)="
                                  f"{worst}: got {got[worst]!r} want {expect32[worst]!r}, len {seq_lens[worst[0]]}"
                                  + (f", slope {slopes[worst[1]]!r}" if slopes is not None else ""))
    # bf16 results: at most one representable step apart (sign-magnitude bit patterns are ordered)
    def key(bits):
        b = bits.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    if not bf16_step_check:
        return got, want
    steps = np.abs(key(got_bits) - key(expect))
    big = np.abs(expect32) >= 2.0 ** -6   # below that a bf16 step is < 3.1e-5 and the absolute bound rules
    assert steps[big].max(initial=0) <= 1, f"{(steps[big] > 1).sum()} elements differ by more than one bf16 step"
    return got, want


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (8, 8), (16, 1)])
def test_small_edge_lengths(gpu_pool, hq, hkv):
    # lengths straddling the 16-row tile, the 64-row wave stride and the 256-row partition
    run_case(gpu_pool, 1, [1, 15, 16, 17, 63, 64, 65, 255, 256, 257, 511, 512, 513, 1025], hq, hkv)


def test_config2_shape_llama8b(gpu_pool):
    # batch 64, Hq 32, Hkv 8, ctx uniform in [512, 4096]
    rng = np.random.default_rng(1001)
    lens = rng.integers(512, 4097, 64).tolist()
    run_case(gpu_pool, 1001, lens, 32, 8)


@pytest.mark.parametrize("pt", [64, 128, 512, 1024])
def test_partition_count_invariance(gpu_pool, pt):
    # the result must not depend on how the rows are split (v1 == v2 in the reference's tests)
    lens = [700, 64, 1500, 2049]
    got, _ = run_case(gpu_pool, 7, lens, 32, 8, partition_tokens=pt)
    base, _ = run_case(gpu_pool, 7, lens, 32, 8, partition_tokens=256)
    assert np.abs(got - base).max() <= 2e-3


def test_v2_entry_point(gpu_pool):
    run_case(gpu_pool, 3, [513, 2000, 100], 32, 8, version="v2")


def test_alibi(gpu_pool):
    run_case(gpu_pool, 5, [33, 400, 1000], 32, 8, alibi=True)


def test_single_token_returns_value_row(gpu_pool):
    # T = 1: softmax over one logit is 1, so out = V[0] bit for bit
    import torch

    got, want = run_case(gpu_pool, 11, [1, 1, 1], 32, 8)
    assert np.array_equal(got, want)  # fp32 result equals the (bf16-valued) V row exactly


def test_config3_long_context_split_k(gpu_pool):
    """BASELINE config 3 at reduced batch: contexts of 32k-131k rows, hundreds of partitions per
    sequence, so the cross-partition log-sum-exp merge carries the result."""
    rng = np.random.default_rng(1002)
    lens = [int(rng.integers(32768, 131073)), 131072, 40000]
    run_case(gpu_pool, 1002, lens, 32, 8)


@pytest.mark.parametrize("mode", [0, 1])
def test_merge_inside_and_outside_the_kernel(gpu_pool, mode):
    """The partial results of workgroups that share a (sequence, kv head) are merged either by the
    workgroup that finishes last or by a second kernel; the library picks per call.  Both forced here,
    on short sequences (many per workgroup), long ones (many workgroups per sequence) and fixed
    partitions."""
    from glake_amd import _C

    lib = _C.lib()
    _C.check(lib.vtkv_set_fused_merge(mode))
    try:
        run_case(gpu_pool, 21, [1, 15, 16, 17, 64, 65, 257, 1025], 32, 8)
        run_case(gpu_pool, 22, [30000, 3, 9000, 700], 32, 8)
        run_case(gpu_pool, 23, [700, 64, 1500, 2049], 64, 8, partition_tokens=128)
        rng = np.random.default_rng(1001)
        run_case(gpu_pool, 1001, rng.integers(512, 4097, 64).tolist(), 32, 8)
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))


@pytest.mark.parametrize("mode,merge", [(0, 0), (1, 0), (1, 1)])
def test_head_major_and_sequence_major_tile_orders(gpu_pool, mode, merge):
    """The workgroups walk over the batch in (sequence, kv head, rows) or in (kv head, sequence, rows) order;
    the library picks the second where it lines the kv heads up with the XCDs.  Both forced here, the head-major
    one with the separate merge kernel and with the merge inside the kernel: short sequences, several per workgroup; long ones over
    many workgroups; 8, 3, 1 and 16 kv heads; ALiBi; the fused append; fp8 rows (pairs of kv heads)."""
    from glake_amd import _C

    import test_gpu_append_attention as A

    lib = _C.lib()
    _C.check(lib.vtkv_set_head_major(mode))
    _C.check(lib.vtkv_set_fused_merge(merge))
    try:
        run_case(gpu_pool, 51, [1, 15, 16, 17, 64, 65, 257, 1025], 32, 8)
        run_case(gpu_pool, 52, [30000, 3, 9000, 700], 32, 8)
        run_case(gpu_pool, 53, [700, 64, 1500, 2049, 1, 33], 12, 3, alibi=True)
        run_case(gpu_pool, 54, [5000, 17, 900], 8, 1)
        run_case(gpu_pool, 55, [333, 4000, 16, 2], 32, 16)
        rng = np.random.default_rng(1001)
        run_case(gpu_pool, 1001, rng.integers(512, 4097, 64).tolist(), 32, 8)
        A.run_case(gpu_pool, 56, [1, 2, 17, 1025, 1026, 40000, 300], 32, 8, lens_from="device")
        A.run_case(gpu_pool, 57, rng.integers(1, 3000, 48).tolist(), 64, 8)
        # fp8 rows: a segment is a pair of kv heads
        A.run_case(gpu_pool, 58, [1, 2, 17, 2049, 2050, 30000, 300], 64, 8, fp8=True)
        A.run_case(gpu_pool, 59, rng.integers(1, 5000, 40).tolist(), 32, 4, lens_from="device", fp8=True, alibi=True)
    finally:
        _C.check(lib.vtkv_set_head_major(-1))
        _C.check(lib.vtkv_set_fused_merge(-1))


@pytest.mark.parametrize("mode", [-1, 0, 1])
def test_very_many_short_sequences_pair_their_kv_heads(gpu_pool, mode):
    """From 4096 (sequence, kv head) segments on the library runs the variants in which a workgroup streams a
    pair of adjacent kv heads (two waves per head); 540 sequences of 8 kv heads, most of a few rows, a few
    long enough to be shared by several workgroups, with and without ALiBi, every merge mode."""
    from glake_amd import _C

    rng = np.random.default_rng(77)
    lens = [int(x) for x in rng.integers(1, 40, 536)] + [700, 1, 1500, 16]
    lib = _C.lib()
    _C.check(lib.vtkv_set_fused_merge(mode))
    try:
        run_case(gpu_pool, 41, lens, 32, 8)
        run_case(gpu_pool, 42, lens[200:], 16, 16, alibi=True, bf16_step_check=False)
        run_case(gpu_pool, 43, lens, 24, 8, partition_tokens=64)
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))


def test_more_sequences_than_one_launch_takes(gpu_pool):
    """A launch takes 1024 sequences; 1300 in one call run as two launches on the same stream and scratch.
    Lengths differ on either side of the cut, a few sequences are long enough to be shared by workgroups."""
    rng = np.random.default_rng(78)
    lens = [int(x) for x in rng.integers(1, 40, 1296)] + [700, 1, 1500, 16]
    lens[1023], lens[1024] = 300, 2
    run_case(gpu_pool, 44, lens, 8, 2)
    run_case(gpu_pool, 45, lens, 8, 2, partition_tokens=256)


def test_calls_on_two_streams_do_not_share_scratch(gpu_pool):
    """Two batches attend at the same time on two streams, twenty times over; each result equals the one
    the same call gives when it runs alone (the wrapper keeps one scratch buffer per device and stream)."""
    import torch

    from glake_amd import _custom_ops as ops

    rng = np.random.default_rng(21)
    hq, hkv, d = 32, 8, 128
    scale = d ** -0.5
    batches = []
    for lens in ([900, 1500, 700, 64, 2100], [1300, 40, 1800, 1000]):
        gpu = GpuSeqs(gpu_pool, len(lens), hkv, d, 2, max(lens))
        for i, t in enumerate(lens):
            gpu.upload(i, bf16_randn(rng, (t, hkv, d)), bf16_randn(rng, (t, hkv, d)))
        kt, vt = gpu.table_tensors()
        q = torch_bf16_from_bits(bf16_randn(rng, (len(lens), hq, d)))
        sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
        slot = torch.arange(len(lens), dtype=torch.int64, device="cuda")
        batches.append(dict(gpu=gpu, kt=kt, vt=vt, q=q, sl=sl, slot=slot, max=max(lens),
                            out=torch.empty(len(lens), hq, d, dtype=torch.float32, device="cuda")))

    def attend(b, out):
        ops.paged_attention_v1(out, b["q"], b["kt"], b["vt"], hkv, scale, b["sl"], 1, b["max"], None, "auto", 1.0,
                               b["slot"])

    alone = []
    for b in batches:
        ref = torch.empty_like(b["out"])
        attend(b, ref)
        alone.append(ref)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(20):
        for b, st in zip(batches, streams):
            b["out"].fill_(float("nan"))
        torch.cuda.synchronize()
        for b, st in zip(batches, streams):
            with torch.cuda.stream(st):
                attend(b, b["out"])
        torch.cuda.synchronize()
        for b, ref in zip(batches, alone):
            assert torch.equal(b["out"], ref)
    for b in batches:
        b["gpu"].close()


def test_two_threads_attend_while_timing_is_on_and_the_knobs_flip(gpu_pool):
    """The kernel timer and the two tuning knobs are process-wide: two host threads attend on their own
    streams with timing switched on while the main thread keeps flipping the knobs.  Every result must equal
    one of the results the same call gives alone (the knobs only change fp32 summation order), the timer must
    have recorded whole calls, and nothing may crash."""
    import threading

    import torch

    from glake_amd import _C, _custom_ops as ops

    lib = _C.lib()
    rng = np.random.default_rng(61)
    hq, hkv, d = 32, 8, 128
    scale = d ** -0.5
    lens = [900, 1500, 700, 64, 2100, 33]
    gpu = GpuSeqs(gpu_pool, len(lens), hkv, d, 2, max(lens))
    ks, vs = [], []
    for i, t in enumerate(lens):
        ks.append(bf16_randn(rng, (t, hkv, d)))
        vs.append(bf16_randn(rng, (t, hkv, d)))
        gpu.upload(i, ks[-1], vs[-1])
    kt, vt = gpu.table_tensors()
    q = bf16_randn(rng, (len(lens), hq, d))
    q_t = torch_bf16_from_bits(q)
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    slot = torch.arange(len(lens), dtype=torch.int64, device="cuda")
    want = O.paged_attention_v1(O.bf16_to_f32(q), O.VTensorCache(ks, vs, np.arange(len(lens)), hkv, d), scale, lens)
    errors, results = [], [[], []]

    def worker(idx):
        try:
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for _ in range(60):
                    out = torch.empty(len(lens), hq, d, dtype=torch.float32, device="cuda")
                    ops.paged_attention_v1(out, q_t, kt, vt, hkv, scale, sl, 1, max(lens), None, "auto", 1.0, slot)
                    results[idx].append(out)
            st.synchronize()
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    _C.check(lib.vtkv_set_kernel_timing(1))
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    flips = 0
    while any(t.is_alive() for t in threads):
        _C.check(lib.vtkv_set_fused_merge(flips % 3 - 1))
        _C.check(lib.vtkv_set_head_major((flips // 3) % 3 - 1))
        flips += 1
    for t in threads:
        t.join()
    _C.check(lib.vtkv_set_fused_merge(-1))
    _C.check(lib.vtkv_set_head_major(-1))
    _C.check(lib.vtkv_set_kernel_timing(0))
    assert not errors, errors
    t_stream = (C.c_float * 200)()
    t_reduce = (C.c_float * 200)()
    n = _C.check(lib.vtkv_attention_kernel_times(t_stream, t_reduce, 200))
    assert n == 120 and all(0.0 < t_stream[i] < 100.0 and 0.0 <= t_reduce[i] < 100.0 for i in range(n))
    torch.cuda.synchronize()
    for outs in results:
        assert len(outs) == 60
        for o in outs:
            err = np.abs(o.cpu().numpy() - want)
            assert np.all(err <= ATOL + RTOL * np.abs(want))
    gpu.close()
