"""Engine-side slot/chunk accounting (glake_amd/core/chunk_manager.py) against the arithmetic of the
reference (vllm/sequence.py:342-360, vllm/core/block_manager_v1.py:195-318,436-455,581-600): closed
forms for the per-sequence byte counting, conservation of chunks, the watermark rule, pre-mapped slots."""
import random

import pytest

from glake_amd.core import AllocStatus, ChunkSpaceManager, SequenceChunks
from glake_amd.core.chunk_manager import PHY_GRAN, PREFILL_SLACK_TOKENS

ROW = 8 * 128 * 2  # one bf16 token row of one range at Hkv=8, D=128


def chunks_for(tokens_with_slack: int) -> int:
    return -(-tokens_with_slack * ROW // PHY_GRAN)


@pytest.mark.parametrize("prompt", [1, 2, 923, 924, 925, 1024, 5000])
def test_prompt_reserves_rows_plus_slack_rounded_to_chunks(prompt):
    s = SequenceChunks(ROW)
    s.append_tokens(prompt)
    slack = 0 if prompt == 1 else PREFILL_SLACK_TOKENS
    n = chunks_for(prompt + slack)
    assert s.logical_block_num == 2 * n and s.reserve_size == n * PHY_GRAN
    assert s.free_size == n * PHY_GRAN - (prompt + slack) * ROW


def test_decode_claims_a_chunk_pair_exactly_when_the_rows_run_out():
    s = SequenceChunks(ROW)
    s.append_tokens(900)                      # 1000 rows with slack: one chunk of 1024 rows
    assert s.logical_block_num == 2
    grown_at = []
    for t in range(1, 1200):
        before = s.logical_block_num
        s.append_tokens(1)
        if s.logical_block_num != before:
            grown_at.append(t)
            assert s.logical_block_num == before + 2
    # 24 rows were left in the first chunk; the 25th new token opens the second, then every 1024
    assert grown_at == [25, 25 + 1024]


@pytest.mark.parametrize("prompt", [2, 923, 924, 925, 5000])
def test_value_skew_is_claimed_once_with_the_first_rows(prompt):
    """With the engine's 256-byte V offset a range needs rows * ROW + 256 bytes: the claim grows one row
    early at every chunk boundary and always bounds that need."""
    s = SequenceChunks(ROW, value_skew=256)
    s.append_tokens(prompt)
    rows = prompt + PREFILL_SLACK_TOKENS
    for t in range(2200):
        need = rows * ROW + 256
        assert s.reserve_size == -(-need // PHY_GRAN) * PHY_GRAN and s.logical_block_num == 2 * (s.reserve_size // PHY_GRAN)
        assert s.free_size == s.reserve_size - need
        s.append_tokens(1)
        rows += 1
    with pytest.raises(ValueError):
        SequenceChunks(ROW, value_skew=PHY_GRAN)


def test_conservation_and_watermark_under_random_traffic():
    rng = random.Random(5)
    total = 400
    m = ChunkSpaceManager(max_seqs=16, num_gpu_handles=total, watermark=0.05)
    running = []
    for step in range(3000):
        assert m.sum_all_blocks() == total and m.get_num_free_gpu_blocks() >= 0
        r = rng.random()
        if r < 0.15:
            s = SequenceChunks(ROW)
            s.append_tokens(rng.randint(2, 30000))
            st = m.can_allocate(s)
            if s.logical_block_num > total - m.watermark_blocks:
                assert st is AllocStatus.NEVER
            elif m.get_num_free_gpu_blocks() - s.logical_block_num >= m.watermark_blocks:
                assert st is AllocStatus.OK
            else:
                assert st is AllocStatus.LATER
            if st is AllocStatus.OK and m.allocate(s):
                assert m.block_tables[s.slot] == s.logical_block_num
                running.append(s)
        elif r < 0.9 and running:
            if m.can_append_slots(len(running)):
                ext = []
                for s in running:
                    s.append_tokens(1)
                    m.append_slots(s, ext)
                    assert m.block_tables[s.slot] == s.logical_block_num
                assert len(ext) == len(set(ext))
            else:  # preempt the newest sequence, as the scheduler does
                s = running.pop()
                s.preempted = True
                assert m.free(s) == s.slot and m.block_tables[s.slot] == 0
        elif running:
            s = running.pop(rng.randrange(len(running)))
            slot = m.free(s)
            assert m.kv_cache_slot[slot] == 0 and m.block_tables[slot] == 0
    for s in running:
        m.free(s)
    assert m.get_num_free_gpu_blocks() == total


def test_slots_run_out_before_memory():
    m = ChunkSpaceManager(max_seqs=2, num_gpu_handles=100)
    seqs = [SequenceChunks(ROW) for _ in range(3)]
    for s in seqs:
        s.append_tokens(10)
    assert m.allocate(seqs[0]) and m.allocate(seqs[1]) and not m.allocate(seqs[2])
    assert {seqs[0].slot, seqs[1].slot} == {0, 1}
    assert m.free(seqs[0]) == 0 and m.allocate(seqs[2]) and seqs[2].slot == 0


def test_premapped_slots_give_credit_and_keep_their_chunks():
    # 2 of 4 slots come with 3 chunks per range already mapped
    m = ChunkSpaceManager(max_seqs=4, num_gpu_handles=40, watermark=0.0, cache_token=3, cache_seq=2)
    assert m.get_num_free_gpu_blocks() == 40 - 12 and m.free_block_tables_block == 12 and m.sum_all_blocks() == 40
    s = SequenceChunks(ROW)
    s.append_tokens(2 * 1024)                 # 2148 rows with slack: 3 chunks per range = 6
    assert s.logical_block_num == 6
    assert m.can_allocate(s) is AllocStatus.OK and m.allocate(s)
    assert s.slot == 0 and m.get_num_free_gpu_blocks() == 28      # nothing taken: the slot already held 6
    big = SequenceChunks(ROW)
    big.append_tokens(5 * 1024)               # 6 chunks per range = 12, lands in pre-mapped slot 1, needs 6 more
    assert m.allocate(big) and big.slot == 1 and m.get_num_free_gpu_blocks() == 22
    assert m.free(big) == 1 and m.block_tables[1] == 6 and m.get_num_free_gpu_blocks() == 28  # keeps 3+3
    # when decode runs short, idle pre-mapped slots are given up
    m._take(27)
    assert not m.can_append_slots(2)
    assert m.cached_token_gc(2) == [1] and m.can_append_slots(2) and m.block_tables[1] == 0
    m._give(27)
    s.preempted = True
    m.free(s)
    assert m.sum_all_blocks() == 40 and m.get_num_free_gpu_blocks() == 40
