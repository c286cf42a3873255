"""StepLoop.prefix_room (glake_amd/worker/step_loop.py) on the CPU, with a stand-in for the cache engine and the
pool: the chunks a prefix store may take are what the pool has free beyond everything the manager has promised.
Checked on hand-made states whose answer follows from counting chunks, not from the formula."""
import types

import pytest

from glake_amd.core import ChunkSpaceManager, StepScheduler
from glake_amd.core.chunk_manager import PHY_GRAN

ROW = 8 * 128 * 2
LAYERS = 2


class FakeStore:
    def __init__(self, slots):
        self.free_slots = list(slots)
        self.room = None

    def lookup(self, tokens):
        return None, 0


def make(monkeypatch, pool_free, max_seqs=3, budget=10, pool_chunks=None, cache_token=0, store_slots=(3, 4)):
    from glake_amd.worker import step_loop

    free = {"n": pool_free}
    monkeypatch.setattr(step_loop.vmm, "showFreeBlocks", lambda: free["n"])
    segs = [types.SimpleNamespace(actual_size=0) for _ in range(max_seqs + 2)]
    eng = types.SimpleNamespace(num_layers=LAYERS, chunk_bytes=PHY_GRAN, vmm_kvcache_segment=segs, device=0)
    mgr = ChunkSpaceManager(max_seqs, budget, watermark=0.0, cache_token=cache_token, cache_seq=1 if cache_token else 0)
    sched = StepScheduler(mgr, ROW, max_seqs, 8192)
    store = FakeStore(store_slots)
    loop = step_loop.StepLoop(eng, sched, prefix_store=store, pool_chunks=pool_chunks)
    return loop, sched, mgr, segs, free, store


def test_room_is_what_the_pool_has_beyond_the_managers_promises(monkeypatch):
    # a pool of 100 free chunks of which this loop may use 30: 2 layers x 10 for the manager, 10 for prefixes
    loop, sched, mgr, segs, free, store = make(monkeypatch, pool_free=100, pool_chunks=30)
    assert store.room == loop.prefix_room and sched.prefix_lookup == store.lookup
    assert loop.prefix_room() == 10
    # a prompt of 900 rows is admitted: one K and one V chunk of every layer promised, none mapped yet
    a = sched.add_request(900, 5)
    out = sched.schedule()
    assert out.prompts == [a] and mgr.block_tables[a.slot] == 2
    assert loop.prefix_room() == 10                       # the promise moved from the pool to the slot
    segs[a.slot].actual_size = PHY_GRAN                   # the step maps it: 4 physical chunks leave the pool
    free["n"] -= 4
    assert loop.prefix_room() == 10
    free["n"] -= 6                                        # a holder takes 6 chunks of its own
    assert loop.prefix_room() == 4
    # the request finishes: the manager has its chunks back at once, the slot unmaps a moment later
    sched.on_step_done(out)
    for _ in range(4):
        done = sched.on_step_done(sched.schedule())
    assert done == [a] and mgr.get_num_free_gpu_blocks() == 10
    assert loop.prefix_room() == 4                        # mapped chunks of a slot nobody owns count as free
    # ... but two of the four were shared with a holder and stay in use: the store is 2 over after the release
    segs[a.final_slot].actual_size = 0
    free["n"] += 2
    assert loop.prefix_room() == 2
    free["n"] -= 5
    assert loop.prefix_room() == -3                       # what make_room has to evict


def test_the_loop_checks_its_pool_and_the_stores_slots(monkeypatch):
    with pytest.raises(ValueError):                       # fewer chunks than the manager hands out in both layers
        make(monkeypatch, pool_free=100, pool_chunks=19)
    with pytest.raises(ValueError):                       # more than the pool has
        make(monkeypatch, pool_free=25, pool_chunks=30)
    with pytest.raises(ValueError):                       # a holder in a slot the manager hands out
        make(monkeypatch, pool_free=100, store_slots=(2, 3))
    with pytest.raises(ValueError):                       # pre-mapped slots are never empty
        make(monkeypatch, pool_free=100, cache_token=1)
    loop, *_ = make(monkeypatch, pool_free=100)           # by default everything that is free
    assert loop.prefix_room() == 100 - LAYERS * 10
