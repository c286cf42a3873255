"""A decode step recorded into a HIP graph and replayed.  `reshape_and_cache` and `paged_attention_v1`
(through the C ABI) launch kernels on the caller's stream and nothing else: no allocation, no copy, no
wait, so a serving loop can capture them once and replay the graph every step.  Between replays the host
updates the step's device-side inputs in place (query, new rows, byte offsets, lengths) and grows the
ranges; every replay is checked bit for bit against the same step run eagerly on a twin set of sequences,
with eager work and synchronisations in between."""
import numpy as np
import pytest

from kvharness import GpuSeqs, bf16_randn, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kv", ["bf16", "fp8"])
def test_decode_step_replays_from_a_graph(gpu_pool, kv):
    import torch

    from glake_amd import _custom_ops as ops, vmm_allocator as vmm

    B, hq, hkv, d, steps = 5, 32, 8, 128, 6
    fp8 = kv == "fp8"
    eb = 1 if fp8 else 2
    row = hkv * d * eb
    kv_dtype = "fp8" if fp8 else "auto"
    k_scale, v_scale = (0.02, 0.03) if fp8 else (1.0, 1.0)
    scale = d ** -0.5
    rng = np.random.default_rng(31)
    rows_per_chunk = (2 << 20) // row
    ctx = [int(x) for x in rng.integers(30, 400, B)]
    ctx[2] = rows_per_chunk - 3          # grows into its second chunk while the graph is in use
    bound = max(ctx) + steps + 1         # max_seq_len recorded in the graph: an upper bound of every step
    sets = [GpuSeqs(vmm, B, hkv, d, eb, rows_per_chunk + 64) for _ in range(2)]   # [0] graph, [1] eager
    for b in range(B):
        if fp8:
            kc = rng.integers(0, 120, (ctx[b], hkv, d)).astype(np.uint8)   # positive finite e4m3fn codes
            vc = rng.integers(0, 120, (ctx[b], hkv, d)).astype(np.uint8)
        else:
            kc, vc = bf16_randn(rng, (ctx[b], hkv, d)), bf16_randn(rng, (ctx[b], hkv, d))
        for s in sets:
            s.upload(b, kc, vc)
    tables = [s.table_tensors() for s in sets]
    slot_ids = list(range(B))
    slot_t = torch.arange(B, dtype=torch.int64, device="cuda")

    # the graph's inputs and output live at fixed addresses
    q = torch.zeros(B, hq, d, dtype=torch.bfloat16, device="cuda")
    nk = torch.zeros(B, hkv, d, dtype=torch.bfloat16, device="cuda")
    nv = torch.zeros_like(nk)
    slot_m = torch.zeros(B, dtype=torch.int64, device="cuda")
    lens_t = torch.zeros(B, dtype=torch.int32, device="cuda")
    out_graph = torch.zeros(B, hq, d, dtype=torch.float32, device="cuda")
    out_eager = torch.zeros_like(out_graph)

    def step_kernels(which, out):
        ops.reshape_and_cache(nk, nv, tables[which][0], tables[which][1], slot_m, slot_t, None, None, 1, hkv, d,
                              kv_dtype, k_scale, v_scale)
        ops.paged_attention_v1(out, q, tables[which][0], tables[which][1], hkv, scale, lens_t, 1, bound, None,
                               kv_dtype, k_scale, slot_t, v_scale=v_scale)

    def host_side(which, lens):
        """What the engine does before the kernels of a step: grow the ranges, hand out byte offsets."""
        offs = vmm.extend_kv_cache_batch(None, None, slot_ids, [row] * B, sets[which].segs, [0] * B, row, True)
        assert offs == [n * row for n in lens]
        return offs

    def new_inputs(lens, offs):
        q.copy_(torch_bf16_from_bits(bf16_randn(rng, (B, hq, d))))
        nk.copy_(torch_bf16_from_bits(bf16_randn(rng, (B, hkv, d))))
        nv.copy_(torch_bf16_from_bits(bf16_randn(rng, (B, hkv, d))))
        slot_m.copy_(torch.tensor(offs, dtype=torch.int64))
        lens_t.copy_(torch.tensor([n + 1 for n in lens], dtype=torch.int32))

    lens = list(ctx)
    # step 0 runs eagerly on both sets (it also creates the attention workspace, outside the capture)
    offs = host_side(0, lens)
    assert host_side(1, lens) == offs
    new_inputs(lens, offs)
    step_kernels(0, out_graph)
    step_kernels(1, out_eager)
    torch.cuda.synchronize()
    assert torch.equal(out_graph, out_eager)
    lens = [n + 1 for n in lens]

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step_kernels(0, out_graph)

    for step in range(1, steps):
        offs = host_side(0, lens)
        assert host_side(1, lens) == offs
        new_inputs(lens, offs)
        out_graph.fill_(float("nan"))
        graph.replay()
        step_kernels(1, out_eager)
        torch.cuda.synchronize()
        assert torch.isfinite(out_graph).all(), f"step {step}: the replay left output rows unwritten"
        assert torch.equal(out_graph, out_eager), f"step {step}: replayed and eager outputs differ"
        lens = [n + 1 for n in lens]
    assert sets[0].segs[2].actual_size == 2 * (2 << 20)      # the range grew under the graph's feet
    for b in range(B):
        nbytes = lens[b] * row
        for which in ("k", "v"):
            assert np.array_equal(sets[0].download(b, nbytes, which=which), sets[1].download(b, nbytes, which=which))
    for s in sets:
        s.close()
