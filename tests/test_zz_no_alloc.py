"""The entry point that allocates nothing, vtkv_decode_attention_noalloc, through the C ABI: its output must
equal vtkv_decode_attention's bit for bit (same kernels, the library's static scratch instead of a workspace of
the caller's) and match the oracle within the decode tolerance (2e-3 + 2e-3 |x| on the fp32 result), on two calls
in a row of which the second is smaller (the shared scratch keeps the first call's contents), in both merge
modes (the arrival counters live in that scratch too), for a bf16 and an fp8 cache; sizes beyond the static
scratch are refused."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


def attend(entry, out, q_t, kt, vt, slot_t, sl_t, b, hq, hkv, d, scale, max_len, kv_dt, k_scale, v_scale, ws=None):
    import torch

    from glake_amd import _C

    lib = _C.lib()
    p = lambda t: C.c_void_p(t.data_ptr())
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (p(out), p(q_t), p(kt), p(vt), p(slot_t), p(sl_t), b, hq, hkv, d, q_t.stride(0), scale, max_len, None,
            _C.BF16, _C.F32, kv_dt, k_scale, v_scale)
    if entry == "noalloc":
        _C.check(lib.vtkv_decode_attention_noalloc(*head, stream))
    else:
        _C.check(lib.vtkv_decode_attention(*head, p(ws), ws.numel(), 0, stream))


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("merge", [-1, 0, 1])
def test_noalloc_entry_point_equals_the_workspace_one(gpu_pool, fp8, merge):
    import torch

    from glake_amd import _C

    lib = _C.lib()
    rng = np.random.default_rng(17 + merge)
    hq, hkv, d = 32, 8, 128
    scale = d ** -0.5
    k_scale, v_scale = (0.013, 0.011) if fp8 else (1.0, 1.0)
    kv_dt = _C.FP8_E4M3 if fp8 else _C.BF16
    lens_all = [int(x) for x in rng.integers(1, 3000, 40)] + [9000, 1, 17]
    b_all = len(lens_all)
    gpu = GpuSeqs(gpu_pool, b_all, hkv, d, 1 if fp8 else 2, max(lens_all), value_skew=256)
    ks, vs = [], []
    for i, n in enumerate(lens_all):
        if fp8:
            k = O.fp8_encode(rng.standard_normal((n, hkv, d)).astype(np.float32), k_scale)
            v = O.fp8_encode(rng.standard_normal((n, hkv, d)).astype(np.float32), v_scale)
        else:
            k, v = bf16_randn(rng, (n, hkv, d)), bf16_randn(rng, (n, hkv, d))
        ks.append(k)
        vs.append(v)
        gpu.upload(i, k, v)
    kt, vt = gpu.table_tensors()
    q = bf16_randn(rng, (b_all, hq, d))
    q_t = torch_bf16_from_bits(q)
    if fp8:
        k32, v32 = [O.fp8_decode(c, k_scale) for c in ks], [O.fp8_decode(c, v_scale) for c in vs]
    else:
        k32, v32 = ks, vs
    need = lib.vtkv_decode_attention_workspace_bytes(b_all, hq, d, max(lens_all), 0)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    _C.check(lib.vtkv_set_fused_merge(merge))
    try:
        # two calls in a row, the second on fewer and shorter sequences
        for first, count in ((0, b_all), (5, 9)):
            lens = lens_all[first:first + count]
            slot_t = torch.arange(first, first + count, dtype=torch.int64, device="cuda")
            sl_t = torch.tensor(lens, dtype=torch.int32, device="cuda")
            outs = {}
            for entry in ("noalloc", "workspace"):
                out = torch.full((count, hq, d), float("nan"), dtype=torch.float32, device="cuda")
                attend(entry, out, q_t[first:first + count], kt, vt, slot_t, sl_t, count, hq, hkv, d, scale, max(lens),
                       kv_dt, k_scale, v_scale, ws)
                torch.cuda.synchronize()
                outs[entry] = out.cpu().numpy()
            assert np.array_equal(outs["noalloc"], outs["workspace"]), "the two entry points differ"
            want = O.paged_attention_v1(O.bf16_to_f32(q[first:first + count]),
                                        O.VTensorCache(k32, v32, np.arange(first, first + count), hkv, d), scale, lens)
            err = np.abs(outs["noalloc"] - want)
            assert np.all(err <= 2e-3 + 2e-3 * np.abs(want)), f"max err {err.max():.3e}"
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
        gpu.close()


def test_noalloc_entry_point_refuses_what_its_scratch_cannot_hold(gpu_pool):
    import torch

    from glake_amd import _C

    lib = _C.lib()
    assert lib.vtkv_decode_attention_noalloc_max_bytes() == 32 << 20
    b, hq, hkv, d = 1024, 64, 8, 128                      # 65 536 (sequence, head) pairs: 34 MB of partial slots
    dummy = torch.zeros(b * hq * d, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(b, hq, d, dtype=torch.float32, device="cuda")
    tab = torch.zeros(b, dtype=torch.int64, device="cuda")
    lens = torch.ones(b, dtype=torch.int32, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    rc = lib.vtkv_decode_attention_noalloc(p(out), p(dummy), p(tab), p(tab), p(tab), p(lens), b, hq, hkv, d, hq * d,
                                           1.0, 1, None, _C.BF16, _C.F32, _C.BF16, 1.0, 1.0, None)
    assert rc == _C.EINVAL and "static scratch" in _C.last_error()


@pytest.mark.parametrize("merge", [0, 1])
def test_noalloc_entry_point_under_graph_capture_and_without_allocations(gpu_pool, merge):
    """What the entry point is for.  After one call outside capture (the first call on a device looks up the
    scratch's address and the kernels' occupancy), a call is recorded into a HIP graph and replayed three times
    with other lengths in the device-side seq_lens, eager calls and synchronisations in between; every replay is
    compared with the oracle and with the eager call.  Free device memory (hipMemGetInfo) and torch's own
    allocation counters are the same before and after the eager calls."""
    import torch

    from glake_amd import _C

    lib = _C.lib()
    rng = np.random.default_rng(23)
    hq, hkv, d = 32, 8, 128
    scale = d ** -0.5
    cap = [700, 64, 1500, 2100, 33, 900]
    b = len(cap)
    gpu = GpuSeqs(gpu_pool, b, hkv, d, 2, max(cap), value_skew=256)
    ks = [bf16_randn(rng, (n, hkv, d)) for n in cap]
    vs = [bf16_randn(rng, (n, hkv, d)) for n in cap]
    for i in range(b):
        gpu.upload(i, ks[i], vs[i])
    kt, vt = gpu.table_tensors()
    q = bf16_randn(rng, (b, hq, d))
    q_t = torch_bf16_from_bits(q)
    slot_t = torch.arange(b, dtype=torch.int64, device="cuda")
    sl_t = torch.tensor(cap, dtype=torch.int32, device="cuda")
    out_graph = torch.zeros(b, hq, d, dtype=torch.float32, device="cuda")
    out_eager = torch.zeros_like(out_graph)
    lens_sets = [cap, [n // 2 + 1 for n in cap], [1, 64, 17, 2100, 33, 5], [n - 1 for n in cap]]
    staged = [torch.tensor(l, dtype=torch.int32, device="cuda") for l in lens_sets]
    want = [O.paged_attention_v1(O.bf16_to_f32(q), O.VTensorCache(ks, vs, np.arange(b), hkv, d), scale, l)
            for l in lens_sets]
    _C.check(lib.vtkv_set_fused_merge(merge))
    try:
        call = lambda out: attend("noalloc", out, q_t, kt, vt, slot_t, sl_t, b, hq, hkv, d, scale, max(cap), _C.BF16,
                                  1.0, 1.0)
        call(out_eager)                      # the first call on this device, outside capture
        torch.cuda.synchronize()
        free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        for _ in range(3):
            call(out_eager)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0, "free device memory changed across noalloc calls"
        assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call(out_graph)
        for i, lens in enumerate(lens_sets):
            sl_t.copy_(staged[i])
            out_graph.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            got = out_graph.cpu().numpy()
            err = np.abs(got - want[i])
            assert np.all(err <= 2e-3 + 2e-3 * np.abs(want[i])), f"replay {i}: max err {err.max():.3e}"
            call(out_eager)                  # eager work between the replays, on the same scratch
            torch.cuda.synchronize()
            assert torch.equal(out_graph, out_eager), f"replay {i} differs from the eager call"
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
        gpu.close()
