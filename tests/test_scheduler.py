"""The step scheduler (glake_amd/core/scheduler.py) against the rules of the reference's vTensor scheduler
(vllm/core/scheduler.py:425-522 running queue, :653-779 prompts, :781-873 one step, :1160-1225 preemption;
vllm/engine/llm_engine.py:607-618 release): checked through what the rules imply (order of admission, who is
preempted, closed forms for when a slot grows, conservation of chunks, every request finishing), not by
re-running the scheduler's own arithmetic."""
import random

import pytest

from glake_amd.core import (AllocStatus, ChunkSpaceManager, PreemptionMode, SeqStatus, SequenceChunks, StepScheduler)
from glake_amd.core.chunk_manager import PHY_GRAN, PREFILL_SLACK_TOKENS

ROW = 8 * 128 * 2            # 1024 rows per 2 MiB chunk
ROWS_PER_CHUNK = PHY_GRAN // ROW


def make(max_seqs=4, chunks=16, tokens=8192, mode=PreemptionMode.RECOMPUTE, **kw):
    mgr = ChunkSpaceManager(max_seqs, chunks, watermark=0.0, **kw)
    return mgr, StepScheduler(mgr, ROW, max_seqs, tokens, preemption=mode)


def test_prompts_run_first_and_apart_from_decodes_in_arrival_order():
    mgr, s = make(max_seqs=3, chunks=40)
    reqs = [s.add_request(p, 5) for p in (100, 200, 300, 400)]
    out = s.schedule()
    assert [r.request_id for r in out.prompts] == [0, 1, 2] and not out.decodes      # three slots, FCFS
    assert sorted(r.slot for r in out.prompts) == [0, 1, 2]
    s.on_step_done(out)
    out = s.schedule()                                    # request 3 still waits for a slot: decodes run
    assert not out.prompts and [r.request_id for r in out.decodes] == [0, 1, 2]
    s.on_step_done(out)
    for _ in range(3):
        s.on_step_done(s.schedule())
    assert all(r.status is SeqStatus.FINISHED and r.generated == 5 for r in reqs[:3])
    out = s.schedule()                                    # the freed slots admit the fourth prompt
    assert [r.request_id for r in out.prompts] == [3] and not out.decodes
    assert mgr.sum_all_blocks() == 40


def test_token_budget_and_prompt_limit():
    mgr, s = make(max_seqs=8, chunks=64, tokens=1000)
    a, b, c, d = (s.add_request(p, 2) for p in (600, 300, 200, 1001))
    out = s.schedule()
    assert [r.request_id for r in out.prompts] == [0, 1] and out.num_batched_tokens == 900   # 200 more would pass 1000
    s.on_step_done(out)
    out = s.schedule()
    assert [r.request_id for r in out.prompts] == [2] and [r.request_id for r in out.ignored] == [3]
    assert d.status is SeqStatus.IGNORED


def test_a_prompt_that_can_never_fit_is_ignored_and_one_that_fits_later_waits():
    mgr, s = make(max_seqs=4, chunks=6, tokens=100000)
    big = s.add_request(4 * ROWS_PER_CHUNK, 3)            # 5 chunks per range with slack: 10 > 6, never
    ok = s.add_request(ROWS_PER_CHUNK, 3)                 # 2 chunks per range: 4
    late = s.add_request(ROWS_PER_CHUNK, 3)               # 4 more: only once `ok` is done
    out = s.schedule()
    assert big.status is SeqStatus.IGNORED and [r.request_id for r in out.prompts] == [1]
    assert late.status is SeqStatus.WAITING
    for _ in range(3):
        s.on_step_done(out)
        out = s.schedule()
    assert ok.status is SeqStatus.FINISHED and [r.request_id for r in out.prompts] == [2]


def test_extend_list_names_a_slot_exactly_when_its_claim_crosses_a_chunk():
    """A prompt of p rows claims ceil((p + 100) / 1024) chunks per range; the sampled tokens use up the slack, so
    the k-th decode step claims a new pair exactly when p + 100 + k + 1 passes a multiple of 1024."""
    mgr, s = make(max_seqs=2, chunks=64)
    p = 900
    req = s.add_request(p, 1500)
    s.on_step_done(s.schedule())
    grown_at = []
    for k in range(1, 1400):
        out = s.schedule()
        assert [r.request_id for r in out.decodes] == [0]
        if out.extend_list:
            assert out.extend_list == [req.slot]
            grown_at.append(k)
        s.on_step_done(out)
    first = ROWS_PER_CHUNK - (p + PREFILL_SLACK_TOKENS)   # rows left in the first chunk after the prompt
    # on_step_done claims the token sampled in that step, schedule() sees the claim in the next step
    assert grown_at == [first + 1, first + 1 + ROWS_PER_CHUNK]
    assert mgr.block_tables[req.slot] == 2 * 3


@pytest.mark.parametrize("mode", [PreemptionMode.RECOMPUTE, PreemptionMode.SWAP])
def test_the_last_sequence_in_is_preempted_when_the_pool_runs_dry(mode):
    mgr, s = make(max_seqs=3, chunks=8, mode=mode)
    reqs = [s.add_request(p, 400) for p in (900, 900, 900)]       # 2 chunks each at admission: 6 of 8
    s.on_step_done(s.schedule())
    victim = None
    for step in range(200):
        out = s.schedule()
        if out.recompute or out.swapped_out:
            victim = (out.recompute or out.swapped_out)[0]
            break
        s.on_step_done(out)
    # 24 rows of the first chunk remain after the prompt and its slack; when they are used up all three want a
    # chunk pair and one pair is left (8 - 6): the first sequence takes it, the pool is empty, can_append_slots
    # fails for the second, and the LAST sequence of the queue pays.
    assert victim is reqs[2]
    assert [r.request_id for r in out.decodes] == [0, 1]
    if mode is PreemptionMode.RECOMPUTE:
        assert victim.status is SeqStatus.WAITING and s.waiting[0] is victim and victim.slot == -1
        assert out.preempted_slot and victim.num_cached == 0
    else:
        assert victim.status is SeqStatus.SWAPPED and s.swapped[0] is victim and victim.swap_slot >= 0
        assert not out.preempted_slot
    assert mgr.sum_all_blocks() == 8
    s.on_step_done(out)
    gen_before = victim.generated
    # it comes back only when chunks are free again, ahead of newer requests, and keeps what it generated
    newer = s.add_request(50, 5)
    back = None
    for step in range(2000):
        out = s.schedule()
        if victim in out.prompts or victim in out.swapped_in:
            back = out
            break
        assert newer not in out.prompts
        s.on_step_done(out)
    assert back is not None and victim.generated == gen_before
    if mode is PreemptionMode.RECOMPUTE:
        assert victim in back.prompts and victim.total_len == 900 + gen_before
    else:
        assert victim in back.swapped_in and victim in back.decodes


@pytest.mark.parametrize("mode", [PreemptionMode.RECOMPUTE, PreemptionMode.SWAP])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_traffic_conserves_chunks_and_finishes_everything(mode, seed):
    rng = random.Random(seed)
    mgr, s = make(max_seqs=6, chunks=20, tokens=6000, mode=mode)
    reqs = []
    for step in range(12000):
        if rng.random() < 0.01 and len(reqs) < 40:
            reqs.append(s.add_request(rng.randint(1, 2500), rng.randint(1, 1200)))
        out = s.schedule()
        assert not (out.prompts and [r for r in out.decodes if r not in out.swapped_in])
        slots = [r.slot for r in out.prompts + out.decodes]
        assert len(set(slots)) == len(slots) and all(0 <= x < 6 for x in slots)
        assert set(out.extend_list) <= set(slots)
        assert len(s.running) <= 6
        s.on_step_done(out)
        assert mgr.sum_all_blocks() == 20 and mgr.get_num_free_gpu_blocks() >= 0
        for r in s.running:
            # the manager's count for a slot bounds the rows the sequence has and is about to write
            assert mgr.block_tables[r.slot] * PHY_GRAN // 2 >= (r.total_len) * ROW
        if len(reqs) == 40 and not s.has_unfinished():
            break
    assert len(reqs) == 40 and not s.has_unfinished()
    for r in reqs:
        assert r.status in (SeqStatus.FINISHED, SeqStatus.IGNORED)
        if r.status is SeqStatus.FINISHED:
            assert r.generated == r.max_new_tokens
    assert mgr.get_num_free_gpu_blocks() == 20


def test_a_prompt_behind_a_cached_prefix_is_charged_for_the_rest_only():
    """scheduler.py:726-766: the token budget counts the rows that still have to run, at least one token runs,
    the chunks of the whole prompt are claimed, and the lookup is not asked when no slot is free."""
    cached = {tuple(range(600)): ("holder-a", 600)}
    asked = []

    def lookup(tokens):
        asked.append(len(tokens))
        for key, (holder, rows) in cached.items():
            if tuple(tokens[:len(key)]) == key:
                return holder, min(rows, len(tokens) - 1)
        return None, 0

    mgr = ChunkSpaceManager(3, 40, watermark=0.0)
    s = StepScheduler(mgr, ROW, 3, 1000, prefix_lookup=lookup)
    a = s.add_request(900, 3, token_ids=list(range(900)))            # 600 cached: 300 rows to run
    b = s.add_request(600, 3, token_ids=list(range(600)))            # cached in full: its last token runs
    c = s.add_request(650, 3, token_ids=list(range(5000, 5650)))     # nothing cached
    d = s.add_request(500, 3)                                         # no tokens given: never looked up
    out = s.schedule()
    # 300 + 1 + 650 = 951 of 1000 tokens; the fourth prompt finds no slot and is not looked up
    assert [r.request_id for r in out.prompts] == [0, 1, 2] and out.num_batched_tokens == 951
    assert [(r.request_id, h, n) for r, h, n in out.prefix_hits] == [(0, "holder-a", 600), (1, "holder-a", 599)]
    assert (a.prefix_rows, b.prefix_rows, c.prefix_rows) == (600, 599, 0) and asked == [900, 600, 650]
    # the claim is for the whole prompt: 900 + 100 rows of slack -> one chunk pair, as without a prefix
    assert a.chunks.get_logical_block_num() == 2 and mgr.block_tables[a.slot] == 2
    s.on_step_done(out)
    assert (a.num_cached, b.num_cached) == (900, 600)
    for _ in range(2):
        s.on_step_done(s.schedule())
    out = s.schedule()
    assert [r.request_id for r in out.prompts] == [3] and not out.prefix_hits and asked == [900, 600, 650]
    # without the prefix the first two prompts alone pass the budget of 1000 tokens
    s2 = StepScheduler(ChunkSpaceManager(3, 40, watermark=0.0), ROW, 3, 1000)
    s2.add_request(900, 3, token_ids=list(range(900)))
    s2.add_request(600, 3, token_ids=list(range(600)))
    assert [r.request_id for r in s2.schedule().prompts] == [0]


def test_a_recomputed_sequence_is_looked_up_again_with_its_prompt():
    rows = {"n": 0}

    def lookup(tokens):
        return ("h", min(rows["n"], len(tokens) - 1)) if rows["n"] else (None, 0)

    mgr = ChunkSpaceManager(2, 4, watermark=0.0)
    s = StepScheduler(mgr, ROW, 2, 4096, prefix_lookup=lookup)
    a = s.add_request(900, 400, token_ids=list(range(900)))
    b = s.add_request(900, 400, token_ids=list(range(1000, 1900)))
    s.on_step_done(s.schedule())
    rows["n"] = 900                                        # from now on every prompt is cached in full
    for _ in range(400):
        out = s.schedule()
        s.on_step_done(out)
        if out.recompute:
            break
    assert out.recompute == [b] and b.generated > 0        # both outgrew their chunk; the pool has no third pair
    while b.status is not SeqStatus.RUNNING:
        out = s.schedule()
        s.on_step_done(out)
    # its prompt's 900 tokens are cached, the tokens it had generated are run again behind them
    assert out.prompts == [b] and b.prefix_rows == 899 and out.prefix_hits == [(b, "h", 899)]
    assert out.num_batched_tokens == b.num_cached - 899
