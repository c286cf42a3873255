"""The step loop of the product (glake_amd/worker/step_loop.py over glake_amd/core/scheduler.py) on the GPU: a
small chunk budget forces the scheduler to preempt (by recompute, or by swap to pinned host memory), sequences
cross 2 MiB chunk boundaries through the growth the scheduler announces, finished sequences release their
slots.  A toy "model" feeds every layer random q/k/v rows (the same rows again when a sequence is recomputed)
through VTensorImpl.forward; every output is checked against the oracle on a host record of each request's rows
(2e-3 + one bf16 step; prompts on their last 24 query positions), the cache bytes against that record at the
end of a request, and the allocator's state against the manager's counts after every step."""
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


def run_loop(gpu_pool, mode_name, seed, plan, budget, max_seqs, every):
    """Feed the requests of `plan` ((prompt rows, tokens to generate), a new one every `every` steps) through the
    step loop with `budget` chunks of one layer and `max_seqs` slots; every check of the module docstring."""
    import torch

    from glake_amd import _C
    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.core import ChunkSpaceManager, PreemptionMode, SeqStatus, StepScheduler
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step_loop import StepLoop

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    layers, hq, hkv, d = 2, 32, 8, 128
    row = hkv * d * 2
    rng = np.random.default_rng(seed)                     # (budget 10: five K+V pairs for four slots)
    eng = CacheEngine(layers, hkv, d, torch.bfloat16, max_seqs, 4096, swap_space_bytes=256 << 20)
    mgr = ChunkSpaceManager(max_seqs, budget, watermark=0.0)
    sched = StepScheduler(mgr, row, max_seqs, 4096, value_skew=eng.value_skew, preemption=PreemptionMode[mode_name])
    loop = StepLoop(eng, sched)
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    hist = {}                                             # request id -> per layer [k rows, v rows] by position
    checked = {"prompt": 0, "decode": 0}

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
        new_rows = [r.total_len for r in out.prompts] + [1] * len(out.decodes)
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
            kb = [np.zeros((1, hkv, d), np.uint16)] * max_seqs
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
            reqs.append(sched.add_request(p, g))
        # finished requests are checked before their slot is released inside the step: hook on_step_done
        res = loop.step(run_model)
        preempted += len(res.outputs.recompute) + len(res.outputs.swapped_out)
        grown += len(res.outputs.extend_list)
        released += len(res.finished)
        vmm.wait_map_ahead()
        torch.cuda.synchronize()
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
        if step % 50 == 0:
            for r in sched.running:
                check_bytes(r)
        if not plan and not sched.has_unfinished():
            break
    assert not sched.has_unfinished() and all(r.status in (SeqStatus.FINISHED, SeqStatus.IGNORED) for r in reqs)
    assert all(r.generated == r.max_new_tokens for r in reqs if r.status is SeqStatus.FINISHED)
    eng.close()
    assert vmm.showFreeBlocks() == free0
    return preempted, grown, released, checked
