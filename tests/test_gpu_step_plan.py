"""DecodeStepPlan (one call per decode step) against the separate ops and the oracle: the cache bytes
it appends are exact, its attention output equals the separate ops' bit for bit when it uses the same
kernels with the same arguments (unfused), and all outputs are within tolerance of the oracle.  The ring of staging rows is lapped several
times and one sequence crosses a 2 MiB chunk boundary during the run."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import GpuSeqs, bf16_randn, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kv,fused,skew", [("bf16", True, 0), ("bf16", False, 0), ("fp8", False, 0), ("fp8", True, 0),
                                           ("bf16", True, 256), ("bf16", False, 256), ("fp8", True, 256)])
def test_plan_matches_ops_and_oracle(gpu_pool, kv, fused, skew):
    """skew: bytes between the base of a V range and its first row (0 = the reference's placement, 256 = what
    the cache engine sets up)."""
    import torch

    from glake_amd import _custom_ops as ops, vmm_allocator as vmm
    from glake_amd.worker.step import DecodeStepPlan

    B, hq, hkv, d, steps = 6, 32, 8, 128, 11
    fp8 = kv == "fp8"
    eb = 1 if fp8 else 2
    row = hkv * d * eb
    rows_per_chunk = (2 << 20) // row
    rng = np.random.default_rng(77)
    ctx = [int(x) for x in rng.integers(40, 700, B)]
    ctx[1] = rows_per_chunk - 4  # crosses into its second chunk at step 5
    k_scale, v_scale = (0.02, 0.03) if fp8 else (1.0, 1.0)
    kv_dtype = "fp8" if fp8 else "auto"
    scale = d ** -0.5
    # two identical sets of sequences: one driven by the plan, one by the separate ops
    sets = [GpuSeqs(vmm, B, hkv, d, eb, rows_per_chunk + 64, value_skew=skew) for _ in range(2)]
    host_k, host_v = [], []
    for b in range(B):
        kb, vb = bf16_randn(rng, (ctx[b], hkv, d)), bf16_randn(rng, (ctx[b], hkv, d))
        if fp8:
            kc = O.fp8_encode(O.bf16_to_f32(kb), k_scale)
            vc = O.fp8_encode(O.bf16_to_f32(vb), v_scale)
        else:
            kc, vc = kb, vb
        for s in sets:
            s.upload(b, kc, vc)
        host_k.append(kc)
        host_v.append(vc)
    tables = [s.table_tensors() for s in sets]
    slot_ids = list(range(B))
    slot_t = torch.arange(B, dtype=torch.int64, device="cuda")
    plan = DecodeStepPlan(sets[0].segs, slot_ids, tables[0][0], tables[0][1], hq, hkv, d, scale,
                          kv_cache_dtype=kv_dtype, k_scale=k_scale, v_scale=v_scale, ring=4, fused=fused)
    assert plan.fused == fused
    lens = list(ctx)
    for step in range(steps):
        q_bits = bf16_randn(rng, (B, hq, d))
        nk_bits, nv_bits = bf16_randn(rng, (B, hkv, d)), bf16_randn(rng, (B, hkv, d))
        q, nk, nv = (torch_bf16_from_bits(x) for x in (q_bits, nk_bits, nv_bits))
        out_plan = torch.empty(B, hq, d, dtype=torch.float32, device="cuda")
        out_ops = torch.empty_like(out_plan)
        max_len = plan.run(q, nk.view(B, hkv * d), nv.view(B, hkv * d), out_plan)
        # the same step through the reference-style calls
        slot_m = vmm.extend_kv_cache_batch(None, None, slot_ids, [row] * B, sets[1].segs, [0] * B, row, True)
        assert slot_m == [n * row for n in lens]
        lens = [n + 1 for n in lens]
        assert max_len == max(lens) and plan.seq_lens.tolist() == lens
        ops.reshape_and_cache(nk, nv, tables[1][0], tables[1][1], torch.tensor(slot_m, dtype=torch.int64, device="cuda"),
                              slot_t, None, None, 1, hkv, d, kv_dtype, k_scale, v_scale)
        ops.paged_attention_v1(out_ops, q, tables[1][0], tables[1][1], hkv, scale,
                               torch.tensor(lens, dtype=torch.int32, device="cuda"), 1, max(lens), None, kv_dtype,
                               k_scale, slot_t, v_scale=v_scale)
        torch.cuda.synchronize()
        if fused:  # other tiling of the rows, so another fp32 summation order
            assert (out_plan - out_ops).abs().max().item() <= 2e-3
        else:
            assert torch.equal(out_plan, out_ops), f"step {step}: plan and ops outputs differ"
        for b in range(B):
            if fp8:
                nkc = O.fp8_encode(O.bf16_to_f32(nk_bits[b:b + 1]), k_scale)
                nvc = O.fp8_encode(O.bf16_to_f32(nv_bits[b:b + 1]), v_scale)
            else:
                nkc, nvc = nk_bits[b:b + 1], nv_bits[b:b + 1]
            host_k[b] = np.concatenate([host_k[b], nkc])
            host_v[b] = np.concatenate([host_v[b], nvc])
        if step in (0, 5, steps - 1):
            # oracle attention over the host copies (fp8: over the exactly dequantised codes, held in fp32)
            if fp8:
                kk = [O.fp8_decode(x, k_scale) for x in host_k]
                vv = [O.fp8_decode(x, v_scale) for x in host_v]
            else:
                kk, vv = host_k, host_v
            cache = O.VTensorCache(kk, vv, np.arange(B), hkv, d)
            expect = O.paged_attention_v1(O.bf16_to_f32(q_bits), cache, scale, lens)
            np.testing.assert_allclose(out_plan.cpu().numpy(), expect, rtol=2e-3, atol=2e-3)
    # every appended byte is in place, for both drivers
    for s in sets:
        for b in range(B):
            n = lens[b] * row
            assert np.array_equal(s.download(b, n, which="k"), host_k[b].reshape(-1).view(np.uint8))
            assert np.array_equal(s.download(b, n, which="v"), host_v[b].reshape(-1).view(np.uint8))
    assert sets[0].segs[1].actual_size == 2 * (2 << 20)
    for s in sets:
        s.close()
