"""The engine-side accounting (glake_amd/core) against what the chunk pool really maps when the scheduler's
decisions are carried out on the allocator the way the reference's step does (llm_engine.py:686-701 preempt,
llama.py:307-341 prologue with eagerExtend for every slot of the step's extend_list, llm_engine.py:607-618
release): the manager's count for a slot equals the chunks mapped into its ranges at every step (it runs 100
rows ahead of the rows written, vllm/sequence.py:343, which is the head start the map-ahead worker gets), and
admission by its rules never exhausts the real pool."""
import random

import pytest

from kvharness import CHUNK

pytestmark = pytest.mark.gpu


def test_manager_counts_equal_the_real_mapping(gpu_pool):
    from glake_amd.core import ChunkSpaceManager, StepScheduler

    vmm = gpu_pool
    vmm.trim()
    layers, hkv, d, max_seqs = 2, 8, 128, 6
    row = hkv * d * 2
    budget = 24                                   # chunks of one layer the engine may use: too few for six long sequences
    free0 = vmm.showFreeBlocks()
    mgr = ChunkSpaceManager(max_seqs, budget, watermark=0.0)
    sched = StepScheduler(mgr, row, max_seqs, 8192)
    segs = [vmm.KVcacheSegment(layers, 16 * CHUNK, 0, False) for _ in range(max_seqs)]
    rng = random.Random(11)
    preempted = 0
    for step in range(2600):
        if rng.random() < 0.05 or not sched.has_unfinished():
            sched.add_request(rng.randint(2, 3000), rng.randint(1, 1500))
        out = sched.schedule()
        for slot in out.preempted_slot:
            segs[slot].preempt_seq(slot)
        preempted += len(out.recompute)
        if out.prompts:   # extend_kv_cache_batch(gen=False) reserves the rows plus the slack
            vmm.extend_kv_cache_batch(None, None, [r.slot for r in out.prompts], [r.total_len * row for r in out.prompts],
                                      [segs[r.slot] for r in out.prompts], [0] * len(out.prompts), row, False)
        if out.decodes:
            for slot in out.extend_list:
                segs[slot].eagerExtend(row, slot)
            vmm.extend_kv_cache_batch(None, None, [r.slot for r in out.decodes], [row] * len(out.decodes),
                                      [segs[r.slot] for r in out.decodes], [0] * len(out.decodes), row, True)
        for r in sched.on_step_done(out):
            segs[r.final_slot].release_seq(r.final_slot)
        vmm.wait_map_ahead()                          # eagerExtend is asynchronous
        for r in sched.running:
            mapped = 2 * (segs[r.slot].actual_size // CHUNK)
            assert mapped == mgr.block_tables[r.slot], (step, r.slot, mapped, mgr.block_tables[r.slot])
            assert segs[r.slot].used_size == r.num_cached * row <= segs[r.slot].actual_size
        held = sum(2 * layers * (g.actual_size // CHUNK) for g in segs)
        assert vmm.showFreeBlocks() == free0 - held
        assert held <= layers * (budget - mgr.get_num_free_gpu_blocks())
    assert preempted > 0
    for g in segs:
        g.destroy()
    assert vmm.showFreeBlocks() == free0
