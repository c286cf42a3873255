"""A seeded random serving loop on a two-layer cache engine: prompt runs into free slots (some starting
on another sequence's prefix by aliasing its chunks), decode steps over random subsets of the running
sequences (separate ops with fixed or stream-K partitions, or the fused append+attention launch with
lengths on the device or in the kernel arguments), swaps out and in, releases, and unmapping of retired
chunks in between.  Every attention result is checked against the oracle on a host mirror of the cache
(2e-3 abs + 2e-3 rel on the fp32 output) and the cache bytes against the mirror bit for bit, after swaps,
before releases and at the end.  Long prompts make sequences span and cross 2 MiB chunks."""
import numpy as np
import pytest

from oracle import oracle as O

from kvharness import bf16_randn, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed,max_prompt,ops_count", [(1, 400, 500), (2, 2200, 250)])
def test_random_serving_loop(gpu_pool, seed, max_prompt, ops_count):
    import torch

    from glake_amd import _C, _custom_ops as ops
    from glake_amd.worker.cache_engine import CacheEngine

    vmm = gpu_pool
    rng = np.random.default_rng(seed)
    free0 = vmm.showFreeBlocks()
    S, LAYERS, HQ, HKV, D = 10, 2, 32, 8, 128
    ROW = HKV * D * 2
    MAXTOK = 2600
    eng = CacheEngine(LAYERS, HKV, D, torch.bfloat16, S, MAXTOK, swap_space_bytes=2 * LAYERS * S * MAXTOK * ROW)
    dev = torch.device("cuda")
    scale = D ** -0.5
    state = ["free"] * S
    mirror = [[None] * LAYERS for _ in range(S)]   # per slot, per layer: (k [T,HKV,D] bits, v bits)
    lens = [0] * S
    TOL = 2e-3
    nchk = [0]

    def cache_for(layer, slots):
        kb = [np.zeros((1, HKV, D), np.uint16)] * S; vb = list(kb)
        for s in slots:
            kb[s], vb[s] = mirror[s][layer]
        return O.VTensorCache(kb, vb, list(slots), HKV, D)

    def check(got32, want32, what):
        err = np.abs(got32 - want32); bound = TOL + TOL * np.abs(want32)
        assert np.all(err <= bound), (what, float(err.max()))
        nchk[0] += 1

    def admit(slot, share_from=None):
        L = int(rng.integers(1, max_prompt))
        seg = eng.vmm_kvcache_segment[slot]
        shared = 0
        if share_from is not None and lens[share_from] > 0:
            shared = int(rng.integers(1, min(lens[share_from], L) + 1))
            seg.share_prefix(eng.vmm_kvcache_segment[share_from], shared * ROW)
            seg.set_used_size(shared * ROW)
        offs = vmm.extend_kv_cache_batch(None, None, [slot], [(L - shared) * ROW], [seg], [0], ROW, False)
        assert offs == [shared * ROW], offs
        slot_t = torch.tensor([slot], dtype=torch.int64, device=dev)
        for l in range(LAYERS):
            k = bf16_randn(rng, (L, HKV, D)); v = bf16_randn(rng, (L, HKV, D))
            if shared:
                k[:shared] = mirror[share_from][l][0][:shared]; v[:shared] = mirror[share_from][l][1][:shared]
            mirror[slot][l] = (k, v)
            nq = L - shared
            if nq:
                ops.reshape_and_cache(torch_bf16_from_bits(k[shared:]), torch_bf16_from_bits(v[shared:]), eng.k_cache_ptr[l],
                                      eng.v_cache_ptr[l], torch.tensor([shared * ROW], dtype=torch.int64, device=dev), slot_t,
                                      torch.tensor([nq], dtype=torch.int32, device=dev),
                                      torch.tensor([0], dtype=torch.int32, device=dev), nq, HKV, D)
                q = bf16_randn(rng, (nq, HQ, D))
                out = torch.empty(nq, HQ, D, dtype=torch.float32, device=dev)
                ops.prefill_attention(out, torch_bf16_from_bits(q), eng.k_cache_ptr[l], eng.v_cache_ptr[l], HKV, scale, [nq], [L], slot_t)
                want = O.prefill_attention(O.bf16_to_f32(q), cache_for(l, [slot]), scale, [nq], [L])
                check(out.cpu().numpy(), want, ("prefill", slot, l, L, shared))
        seg.set_used_size(L * ROW)
        lens[slot] = L; state[slot] = "run"

    def decode(slots):
        segs = [eng.vmm_kvcache_segment[s] for s in slots]
        offs = vmm.extend_kv_cache_batch(None, None, list(slots), [ROW] * len(slots), segs, [0] * len(slots), ROW, True)
        assert offs == [lens[s] * ROW for s in slots], (offs, [lens[s] for s in slots])
        new_lens = [lens[s] + 1 for s in slots]
        slot_t = torch.tensor(list(slots), dtype=torch.int64, device=dev)
        lens_t = torch.tensor(new_lens, dtype=torch.int32, device=dev)
        for l in range(LAYERS):
            q = bf16_randn(rng, (len(slots), HQ, D)); nk = bf16_randn(rng, (len(slots), HKV, D)); nv = bf16_randn(rng, (len(slots), HKV, D))
            for i, s in enumerate(slots):
                k, v = mirror[s][l]
                mirror[s][l] = (np.concatenate([k, nk[i:i + 1]]), np.concatenate([v, nv[i:i + 1]]))
            out = torch.empty(len(slots), HQ, D, dtype=torch.float32, device=dev)
            mode = int(rng.integers(3))
            if mode == 0:
                ops.reshape_and_cache(torch_bf16_from_bits(nk), torch_bf16_from_bits(nv), eng.k_cache_ptr[l], eng.v_cache_ptr[l],
                                      torch.tensor(offs, dtype=torch.int64, device=dev), slot_t, None, None, 1, HKV, D)
                ops.paged_attention_v1(out, torch_bf16_from_bits(q), eng.k_cache_ptr[l], eng.v_cache_ptr[l], HKV, scale, lens_t, 1,
                                       max(new_lens), None, "auto", 1.0, slot_t, partition_tokens=int(rng.choice([0, 256, 512])))
            else:
                ops.decode_append_attention(out, torch_bf16_from_bits(q), torch_bf16_from_bits(nk), torch_bf16_from_bits(nv),
                                            eng.k_cache_ptr[l], eng.v_cache_ptr[l], HKV, scale, lens_t if mode == 1 else new_lens,
                                            max(new_lens), None, slot_t)
            want = O.paged_attention_v1(O.bf16_to_f32(q), cache_for(l, slots), scale, new_lens, None)
            check(out.cpu().numpy(), want, ("decode", list(slots), l, mode))
        for s in slots: lens[s] += 1

    def verify_bytes(slot):
        seg = eng.vmm_kvcache_segment[slot]
        n = lens[slot] * ROW
        assert seg.used_size == n, (seg.used_size, n)
        for l in range(LAYERS):
            for which, base in ((0, seg.getKeyDevicePtr(l)), (1, seg.getValueDevicePtr(l))):
                back = np.empty(n, np.uint8)
                _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data, base, n))
                assert np.array_equal(back.view(np.uint16).reshape(-1, HKV, D), mirror[slot][l][which]), ("bytes", slot, l, which)

    n = 0; hist = {}
    while n < ops_count:
        run = [s for s in range(S) if state[s] == "run"]; free = [s for s in range(S) if state[s] == "free"]
        swp = [s for s in range(S) if state[s] == "swapped"]
        op = rng.choice(["admit", "share", "decode", "decode", "decode", "swapout", "swapin", "finish", "verify", "trim"] + ["decode"] * (25 if max_prompt > 1000 else 0))
        if op == "admit" and free:
            admit(int(rng.choice(free)))
        elif op == "share" and free and run:
            admit(int(rng.choice(free)), share_from=int(rng.choice(run)))
        elif op == "decode" and run:
            pick = [s for s in run if lens[s] < MAXTOK - 1]
            if pick:
                k = int(rng.integers(1, len(pick) + 1))
                decode([int(x) for x in rng.permutation(pick)[:k]])
        elif op == "swapout" and run:
            k = int(rng.integers(1, len(run) + 1)); pick = [int(x) for x in rng.permutation(run)[:k]]
            eng.swap_out(pick)
            for s in pick: state[s] = "swapped"
        elif op == "swapin" and swp:
            k = int(rng.integers(1, len(swp) + 1)); pick = [int(x) for x in rng.permutation(swp)[:k]]
            eng.swap_in(pick)
            for s in pick: state[s] = "run"; verify_bytes(s)
        elif op == "finish" and run:
            s = int(rng.choice(run)); verify_bytes(s)
            eng.vmm_kvcache_segment[s].release_seq(s); state[s] = "free"; lens[s] = 0; mirror[s] = [None] * LAYERS
        elif op == "verify" and run:
            verify_bytes(int(rng.choice(run)))
        elif op == "trim":
            vmm.trim(int(rng.integers(-1, 6)))
        else:
            continue
        hist[op] = hist.get(op, 0) + 1; n += 1
    torch.cuda.synchronize()
    for s in range(S):
        if state[s] == "run": verify_bytes(s)
    assert nchk[0] > ops_count // 2
    eng.close()
    assert vmm.showFreeBlocks() == free0
