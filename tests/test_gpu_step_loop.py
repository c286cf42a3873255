"""The step loop of the product (glake_amd/worker/step_loop.py over glake_amd/core/scheduler.py) on the GPU: a
small chunk budget forces the scheduler to preempt (by recompute, or by swap to pinned host memory), sequences
cross 2 MiB chunk boundaries through the growth the scheduler announces, finished sequences release their
slots.  A toy "model" feeds every layer random q/k/v rows (the same rows again when a sequence is recomputed)
through VTensorImpl.forward; every output is checked against the oracle on a host record of each request's rows
(2e-3 + one bf16 step; prompts on their last 24 query positions), the cache bytes against that record at the
end of a request, and the allocator's state against the manager's counts after every step.

With a prefix store (glake_amd/worker/prefix_store.py) prompts are given by their tokens and their rows follow
from the tokens, position by position: a prompt that begins like a finished request's starts from that
request's rows (whole chunks mapped a second time) and runs the rest, which the same oracle checks see through
the outputs and the cache bytes; the store's chunks stay within what the pool has beyond the manager's
promises while sequences that share chunks are preempted, swapped and released."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import CHUNK, bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


# long-running sequences that outgrow their first chunk, short ones in between
# (a prompt of up to 923 rows fits one chunk with its slack of 100 rows; its 25th..124th new token opens the next)
PLAN = [(900, 150), (40, 30), (910, 200), (700, 420), (15, 10), (905, 90), (300, 60), (890, 130)]


@pytest.mark.parametrize("mode_name", ["RECOMPUTE", "SWAP"])
def test_step_loop_preempts_grows_and_releases(gpu_pool, mode_name):
    preempted, grown, released, checked = run_loop(gpu_pool, mode_name, 7 if mode_name == "SWAP" else 8, list(PLAN),
                                                   budget=10, max_seqs=4, every=7)
    assert preempted >= 1 and grown >= 3 and released == len(PLAN), (preempted, grown, released)
    assert checked["prompt"] >= len(PLAN) and checked["decode"] > 500


DOC = list(range(100, 2800))                              # 2700 tokens: two whole chunks of rows and 652 more


def test_step_loop_starts_prompts_from_cached_prefixes(gpu_pool):
    """One request after the other (every 70 steps), so every prompt finds what the ones before it left."""
    plan = [(DOC[:2600], 40),                             # nothing cached; kept when it finishes
            (DOC[:2500] + list(range(5000, 5300)), 30),   # 2500 rows: cut inside the third chunk
            (DOC[:1024] + list(range(6000, 6200)), 50),   # 1024 rows: exactly the first chunk
            (DOC[:2600], 20),                             # cached in full: its last token runs
            (700, 60),                                    # no tokens: not looked up, not kept
            (DOC[:2500] + list(range(5000, 5150)) + list(range(7000, 7100)), 25)]   # 2650 rows of the second request's
    preempted, grown, released, checked = run_loop(gpu_pool, "RECOMPUTE", 21, plan, budget=20, max_seqs=4, every=70,
                                                   prefix_slots=8, prefix_chunks=48)
    assert released == 6 and preempted == 0
    assert checked["hits"] == 4 and checked["hit_rows"] == 2500 + 1024 + 2599 + 2650
    assert checked["kept"] >= 5                           # four prompts and the cuts made for the lookups


@pytest.mark.parametrize("mode_name,seed", [("RECOMPUTE", 31), ("SWAP", 32), ("RECOMPUTE", 33)])
def test_step_loop_with_prefixes_under_pressure(gpu_pool, mode_name, seed):
    """Random prompts that begin like one another, more sequences than the manager's chunks can hold, and a
    prefix store with little room: sequences that share chunks with holders are preempted and come back."""
    rnd = np.random.default_rng(seed)
    docs = [DOC, DOC[:1500] + list(range(20000, 21000)), list(range(30000, 32000))]
    plan = []
    for i in range(14):
        doc = docs[int(rnd.integers(len(docs)))]
        head = doc[:int(rnd.integers(200, len(doc)))]
        tail = list(range(40000 + 1000 * i, 40000 + 1000 * i + int(rnd.integers(0, 300))))
        plan.append((head + tail, int(rnd.integers(5, 160))))
    preempted, grown, released, checked = run_loop(gpu_pool, mode_name, seed, plan, budget=14, max_seqs=4, every=9,
                                                   prefix_slots=5, prefix_chunks=30)
    assert released == 14 and checked["hits"] >= 3 and checked["evicted_rows"] > 0, (released, checked)
    assert preempted >= 1


def token_rows(tokens, layer, hkv, d):
    """K and V rows of a prompt as a causal model makes them: row i is a function of tokens[:i + 1] (and the
    layer) only, so two prompts with a common prefix have the same rows there."""
    k = np.empty((len(tokens), hkv, d), np.uint16)
    v = np.empty_like(k)
    h = 17 + layer
    for i, t in enumerate(tokens):
        h = (h * 1000003 + int(t) + 1) % ((1 << 61) - 1)
        kv = O.f32_to_bf16(np.random.default_rng(h).standard_normal((2, hkv, d)).astype(np.float32))
        k[i], v[i] = kv[0], kv[1]
    return k, v


def run_loop(gpu_pool, mode_name, seed, plan, budget, max_seqs, every, prefix_slots=0, prefix_chunks=0):
    """Feed the requests of `plan` ((prompt rows or prompt tokens, tokens to generate), a new one every `every`
    steps) through the step loop with `budget` chunks of one layer and `max_seqs` slots; every check of the
    module docstring.  With `prefix_slots` the loop has a prefix store of that many holders, and the engine and
    the store together may hold `prefix_chunks` physical chunks more than the manager's budget in every layer."""
    import torch

    from glake_amd import _C
    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.core import ChunkSpaceManager, PreemptionMode, SeqStatus, StepScheduler
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.prefix_store import PrefixStore
    from glake_amd.worker.step_loop import StepLoop

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    layers, hq, hkv, d = 2, 32, 8, 128
    row = hkv * d * 2
    rng = np.random.default_rng(seed)                     # (budget 10: five K+V pairs for four slots)
    eng = CacheEngine(layers, hkv, d, torch.bfloat16, max_seqs + prefix_slots, 4096, swap_space_bytes=256 << 20)
    mgr = ChunkSpaceManager(max_seqs, budget, watermark=0.0)
    sched = StepScheduler(mgr, row, max_seqs, 4096, value_skew=eng.value_skew, preemption=PreemptionMode[mode_name])
    store = PrefixStore(eng, list(range(max_seqs, max_seqs + prefix_slots))) if prefix_slots else None
    pool_chunks = layers * budget + prefix_chunks
    loop = StepLoop(eng, sched, prefix_store=store, pool_chunks=pool_chunks if store else None)
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    hist = {}                                             # request id -> per layer [k rows, v rows] by position
    checked = {"prompt": 0, "decode": 0, "hits": 0, "hit_rows": 0, "kept": 0}

    def rows_for(req, layer, lo, hi):
        """K and V rows of positions [lo, hi) of a request: what was fed before, else new random rows."""
        k, v = hist.setdefault(req.request_id, [[np.zeros((0, hkv, d), np.uint16)] * 2 for _ in range(layers)])[layer]
        if k.shape[0] < hi:
            n = hi - k.shape[0]
            k = np.concatenate([k, O.f32_to_bf16(rng.standard_normal((n, hkv, d)).astype(np.float32))])
            v = np.concatenate([v, O.f32_to_bf16(rng.standard_normal((n, hkv, d)).astype(np.float32))])
            hist[req.request_id][layer] = [k, v]
        return k[lo:hi], v[lo:hi]

    def run_model(meta, out):
        seqs = out.prompts + out.decodes
        new_rows = [r.total_len - r.prefix_rows for r in out.prompts] + [1] * len(out.decodes)
        n_tok = sum(new_rows)
        for l in range(layers):
            q = O.f32_to_bf16(rng.standard_normal((n_tok, hq * d)).astype(np.float32))
            ks, vs = [], []
            for r, n in zip(seqs, new_rows):
                k, v = rows_for(r, l, r.total_len - n, r.total_len)
                ks.append(k)
                vs.append(v)
            key = np.concatenate(ks).reshape(n_tok, hkv * d)
            value = np.concatenate(vs).reshape(n_tok, hkv * d)
            kc, vc = eng.gpu_cache[l]
            got = impl.forward(torch_bf16_from_bits(q), torch_bf16_from_bits(key), torch_bf16_from_bits(value), kc, vc, meta)
            got = O.bf16_to_f32(bits_from_torch_bf16(got).reshape(n_tok, hq, d))
            q = q.reshape(n_tok, hq, d)
            kb = [np.zeros((1, hkv, d), np.uint16)] * (max_seqs + prefix_slots)
            vb = list(kb)
            for r in seqs:
                kb[r.slot], vb[r.slot] = (x[:r.total_len] for x in hist[r.request_id][l])
            at = 0
            for r, n in zip(seqs, new_rows):
                cache = O.VTensorCache(kb, vb, [r.slot], hkv, d)
                if n > 1 or r in out.prompts:
                    tail = min(n, 24)                     # the last query positions of the prompt
                    want = O.prefill_attention(q[at + n - tail:at + n], cache, d ** -0.5, [tail], [r.total_len])
                    have = got[at + n - tail:at + n]
                    checked["prompt"] += 1
                else:
                    want = O.paged_attention_v1(q[at:at + 1], cache, d ** -0.5, [r.total_len])
                    have = got[at:at + 1]
                    checked["decode"] += 1
                want = O.bf16_to_f32(want)
                diff = np.abs(have - want)
                assert np.all(diff <= 2e-3 + (2e-3 + 2.0 ** -7) * np.abs(want)), (r.request_id, l, float(diff.max()))
                at += n

    def check_bytes(req):
        seg = eng.vmm_kvcache_segment[req.slot if req.status is SeqStatus.RUNNING else req.final_slot]
        n = req.num_cached
        for l in range(layers):
            for rows, ptr in zip(hist[req.request_id][l], (seg.getKeyDevicePtr(l), seg.getValueDevicePtr(l))):
                back = np.empty((n, hkv, d), np.uint16)
                _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), ptr, n * row))
                assert np.array_equal(back, rows[:n]), ("cache bytes", req.request_id, l)

    reqs = []
    preempted = grown = released = 0
    for step in range(20000):
        if plan and (step % every == 0):
            p, g = plan.pop(0)
            if isinstance(p, int):
                reqs.append(sched.add_request(p, g))
            else:                                         # a prompt given by its tokens: rows follow from them
                reqs.append(sched.add_request(len(p), g, token_ids=list(p)))
                hist[reqs[-1].request_id] = [list(token_rows(p, l, hkv, d)) for l in range(layers)]
        # finished requests are checked before their slot is released inside the step: hook on_step_done
        res = loop.step(run_model)
        preempted += len(res.outputs.recompute) + len(res.outputs.swapped_out)
        grown += len(res.outputs.extend_list)
        released += len(res.finished)
        checked["hits"] += len(res.outputs.prefix_hits)
        checked["hit_rows"] += sum(n for _, _, n in res.outputs.prefix_hits)
        vmm.wait_map_ahead()
        torch.cuda.synchronize()
        for r, _, _ in res.outputs.prefix_hits:           # the shared rows and the rows run behind them
            if r.status is SeqStatus.RUNNING:
                check_bytes(r)
        held = 0
        for r in sched.running:
            seg = eng.vmm_kvcache_segment[r.slot]
            assert seg.used_size == r.num_cached * row, (step, r.request_id, seg.used_size, r.num_cached)
            mapped = 2 * (seg.actual_size // CHUNK)
            assert mapped <= mgr.block_tables[r.slot], (step, r.slot, mapped, mgr.block_tables[r.slot])
            assert seg.used_size + eng.value_skew <= seg.actual_size
            held += mapped
        assert held <= budget - mgr.get_num_free_gpu_blocks()
        assert mgr.sum_all_blocks() == budget
        if store is not None:
            # the pool can serve everything the manager has promised, and the loop stays within its chunks
            assert loop.prefix_room() >= 0, (step, loop.prefix_room())
            assert free0 - vmm.showFreeBlocks() <= pool_chunks, (step, free0 - vmm.showFreeBlocks())
            assert len(store.rows) + len(store.free_slots) == prefix_slots and not store._pinned
        if step % 50 == 0:
            for r in sched.running:
                check_bytes(r)
        if not plan and not sched.has_unfinished():
            break
    assert not sched.has_unfinished() and all(r.status in (SeqStatus.FINISHED, SeqStatus.IGNORED) for r in reqs)
    assert all(r.generated == r.max_new_tokens for r in reqs if r.status is SeqStatus.FINISHED)
    if store is not None:
        checked["kept"], checked["evicted_rows"] = len(store.rows), store.evicted_rows
        store.evict(10 ** 9)
        assert not store.rows and vmm.sharedBlocks() == 0
    eng.close()
    assert vmm.showFreeBlocks() == free0
    return preempted, grown, released, checked
