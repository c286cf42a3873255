"""The engine-side accounting (glake_amd/core) against what the chunk pool really maps when the same
traffic is driven through the allocator the way the reference's step prologue does
(vllm/model_executor/models/llama.py:307-341): with every growth the manager announces carried out by eagerExtend, the manager's count for a slot
equals the chunks mapped into its ranges at every step (it runs 100 rows ahead of the rows written,
vllm/sequence.py:343, which is the head start the map-ahead worker gets), and admission by its rules
never exhausts the real pool."""
import random

import pytest

from kvharness import CHUNK

pytestmark = pytest.mark.gpu


def test_manager_counts_bound_the_real_mapping(gpu_pool):
    from glake_amd.core import AllocStatus, ChunkSpaceManager, SequenceChunks

    vmm = gpu_pool
    vmm.trim()
    layers, hkv, d, max_seqs = 2, 8, 128, 6
    row = hkv * d * 2
    budget = 60                                   # chunks of one layer the engine may use
    free0 = vmm.showFreeBlocks()
    mgr = ChunkSpaceManager(max_seqs, budget, watermark=0.0)
    segs = [vmm.KVcacheSegment(layers, 16 * CHUNK, 0, False) for _ in range(max_seqs)]
    rng = random.Random(11)
    running = []
    for step in range(2600):
        if rng.random() < 0.02 or not running:
            s = SequenceChunks(row)
            prompt = rng.randint(2, 3000)
            s.append_tokens(prompt)
            if mgr.can_allocate(s) is AllocStatus.OK and mgr.allocate(s):
                # prefill: extend_kv_cache_batch(gen=False) reserves the rows plus the slack
                vmm.extend_kv_cache_batch(None, None, [s.slot], [prompt * row], [segs[s.slot]], [0], row, False)
                running.append(s)
        if running and mgr.can_append_slots(len(running)):
            ext = []
            for s in running:
                s.append_tokens(1)
                mgr.append_slots(s, ext)
            for slot in ext:
                segs[slot].eagerExtend(row, slot)
            vmm.extend_kv_cache_batch(None, None, [s.slot for s in running], [row] * len(running),
                                      [segs[s.slot] for s in running], [0] * len(running), row, True)
        elif running:
            s = running.pop()
            s.preempted = True
            segs[mgr.free(s)].preempt_seq(s.slot)
        if running and rng.random() < 0.004:
            s = running.pop(rng.randrange(len(running)))
            segs[mgr.free(s)].release_seq(s.slot)
        vmm.wait_map_ahead()                          # eagerExtend is asynchronous
        for s in running:
            mapped = 2 * (segs[s.slot].actual_size // CHUNK)
            assert mapped == mgr.block_tables[s.slot], (step, s.slot, mapped, mgr.block_tables[s.slot])
            assert segs[s.slot].used_size <= segs[s.slot].actual_size
        held = sum(2 * layers * (g.actual_size // CHUNK) for g in segs)
        assert vmm.showFreeBlocks() == free0 - held
        assert held <= layers * (budget - mgr.get_num_free_gpu_blocks())
    for g in segs:
        g.destroy()
    assert vmm.showFreeBlocks() == free0
