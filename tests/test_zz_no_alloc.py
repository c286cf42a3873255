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
