"""Engine-side slot and chunk accounting for per-sequence contiguous KV ranges.

The reference's scheduler does not track blocks of 16 tokens but, per sequence slot, how many 2 MiB
chunks the slot's K and V ranges hold, and asks this bookkeeping whether a prompt can be admitted, whether
the running sequences can take one more token, and which slots have to grow in the coming step
(``vllm/core/block_manager_v1.py:195-318,436-455,581-600`` for the manager, ``vllm/sequence.py:342-360``
for the per-sequence byte arithmetic).  Counts are in chunks of ONE layer: a growth step of a sequence
is 2 chunks (one for K, one for V); the allocator maps the same step for every layer.

This module restates that accounting as plain integer logic with the same method names and return
values.  Two defects of the reference are not reproduced: ``cached_token_gc`` returns its list (the
reference builds it and returns nothing, :369-379), and ``allocate`` gives an admitted sequence credit
only for chunks the slot really holds (the reference's ``minus = 0`` for a fresh slot is overwritten by
the next statement, :311-313, which happens to be right because a fresh slot holds zero chunks).
"""
from __future__ import annotations

import enum
from typing import Dict, List, Optional

PHY_GRAN = 2 * 1024 * 1024  # bytes of one chunk (sequence.py:345); pools with larger chunks pass their size
PREFILL_SLACK_TOKENS = 100  # a prompt reserves room for 100 more tokens (sequence.py:343)


class AllocStatus(enum.Enum):
    """block_manager_v1 ``AllocStatus``: admit now, admit when memory frees up, or never fits."""
    OK = enum.auto()
    LATER = enum.auto()
    NEVER = enum.auto()


class SequenceChunks:
    """Bytes and chunks one sequence needs in each of its ranges (sequence.py:342-360).

    ``token_size`` is the bytes of one token row of one range (num_kv_heads * head_size * element
    bytes).  ``logical_block_num`` counts K and V chunks together, i.e. two per chunk of rows."""

    def __init__(self, token_size: int, chunk_bytes: int = PHY_GRAN, value_skew: int = 0):
        if token_size <= 0:
            raise ValueError("token_size must be positive")
        if value_skew < 0 or value_skew >= chunk_bytes:
            raise ValueError("value_skew must lie in [0, chunk_bytes)")
        if chunk_bytes <= 0 or chunk_bytes % PHY_GRAN:
            raise ValueError("chunk_bytes must be a positive multiple of 2 MiB")
        self.token_size = int(token_size)
        self.chunk_bytes = int(chunk_bytes)
        # bytes by which the engine sets the V rows off from the base of their range (CacheEngine's
        # value_skew): claimed once, with the first rows, so that the claim bounds what the ranges map
        self.value_skew = int(value_skew)
        self.reserve_size = 0       # bytes the sequence has claimed per range, a multiple of the chunk
        self.free_size = 0          # claimed bytes not yet written
        self.logical_block_num = 0  # chunks claimed (K + V)
        self.slot = -1
        self.preempted = False

    def append_tokens(self, num_tokens: int) -> None:
        """One call per scheduling step: the prompt (any number of tokens, plus slack) or one new token."""
        plus = 0 if num_tokens == 1 else PREFILL_SLACK_TOKENS
        gran = self.chunk_bytes
        need = self.token_size * (num_tokens + plus)
        if self.reserve_size == 0:
            need += self.value_skew
            rounded = gran * ((need + gran - 1) // gran)
            self.reserve_size = rounded
            self.free_size = rounded - need
            self.logical_block_num = 2 * (rounded // gran)
        elif self.free_size >= need:
            self.free_size -= need
        else:
            gap = need - self.free_size
            rounded = gran * ((gap + gran - 1) // gran)
            self.reserve_size += rounded
            self.free_size = rounded - gap
            self.logical_block_num += 2 * (rounded // gran)

    # the reference's accessor names (sequence.py:331-340)
    def get_slot(self) -> int:
        return self.slot

    def set_slot(self, slot: int) -> None:
        self.slot = slot

    def get_logical_block_num(self) -> int:
        return self.logical_block_num


class ChunkSpaceManager:
    """Slots and chunk counts (block_manager_v1.py:195-258).

    ``num_gpu_handles`` is the size of the chunk pool in chunks of one layer.  The first ``cache_seq``
    slots start out holding ``cache_token`` chunks per range (pre-mapped ranges that release keeps
    mapped), so a new prompt that lands in one of them needs that much less from the pool."""

    def __init__(self, max_seqs: int, num_gpu_handles: int, watermark: float = 0.01, cache_token: int = 0,
                 cache_seq: int = 0):
        if watermark < 0.0:
            raise ValueError("watermark must be >= 0")
        if cache_seq > max_seqs or cache_seq * cache_token * 2 > num_gpu_handles:
            raise ValueError("the pre-mapped slots do not fit")
        self.max_seqs = max_seqs
        self.num_total_gpu_blocks = num_gpu_handles
        self.watermark = watermark
        self.watermark_blocks = int(watermark * num_gpu_handles)
        self.cache_token = cache_token
        self.cache_seq = cache_seq
        self._free = num_gpu_handles                      # UncachedBlockAllocator.free_blocks (:169)
        self.block_tables: Dict[int, int] = {i: (cache_token * 2 if i < cache_seq else 0) for i in range(max_seqs)}
        self.kv_cache_slot: List[int] = [0] * max_seqs    # 1 = a running sequence owns the slot
        self._take(cache_seq * cache_token * 2)
        self.free_block_tables_block = cache_seq * cache_token * 2  # chunks parked in idle pre-mapped slots

    # ------------------------------------------------------------------ pool counter (:171-181)
    def _take(self, num: int) -> None:
        if self._free < num:
            raise ValueError("Out of memory! No free blocks are available.")
        self._free -= num

    def _give(self, num: int) -> None:
        self._free += num

    def get_num_free_gpu_blocks(self) -> int:
        return self._free

    free_blocks = get_num_free_gpu_blocks

    def sum_all_blocks(self) -> int:
        """Chunks held by slots plus chunks in the pool: constant (:434-435)."""
        return sum(self.block_tables.values()) + self._free

    # ------------------------------------------------------------------ slots (:260-276)
    def get_free_slot(self) -> int:
        for i in range(self.max_seqs):
            if self.kv_cache_slot[i] == 0:
                self.kv_cache_slot[i] = 1
                return i
        return -1

    def get_cached_slot(self) -> int:
        if self.cache_token == 0:
            return -1
        for i in range(self.max_seqs):
            if self.kv_cache_slot[i] == 0 and self.block_tables[i] == self.cache_token * 2:
                self.kv_cache_slot[i] = 1
                self.free_block_tables_block -= self.cache_token * 2
                return i
        return -1

    # ------------------------------------------------------------------ admission (:281-320)
    def can_allocate(self, seq: SequenceChunks, preempted_flag: bool = False) -> AllocStatus:
        required = seq.get_logical_block_num() + (2 if preempted_flag else 0)
        credit = self.cache_token * 2 if self.free_block_tables_block > 0 else 0
        free = self._free + credit
        if self.num_total_gpu_blocks - required < self.watermark_blocks:
            return AllocStatus.NEVER
        if free - required >= self.watermark_blocks:
            return AllocStatus.OK
        return AllocStatus.LATER

    def allocate(self, seq: SequenceChunks) -> bool:
        slot = self.get_cached_slot()
        if slot == -1:
            slot = self.get_free_slot()
            if slot == -1:
                return False
        seq.set_slot(slot)
        missing = seq.get_logical_block_num() - self.block_tables[slot]
        if missing > 0:
            self._take(missing)
            self.block_tables[slot] += missing
        return True

    # ------------------------------------------------------------------ decode growth (:355-366,439-455)
    def can_append_slots(self, num_running_seqs: int, beta: int = 0) -> bool:
        """One K and one V chunk per running sequence must be available."""
        return 2 * num_running_seqs <= self._free + beta

    def append_slots(self, seq: SequenceChunks, extend_seq_list: Optional[List[int]] = None) -> bool:
        """Called after ``seq.append_tokens(1)``: claims the next K+V chunk pair when the sequence has
        outgrown what its slot holds, and records the slot for the step's eager extension."""
        slot = seq.get_slot()
        assert slot != -1
        if self.block_tables[slot] < seq.get_logical_block_num():
            if extend_seq_list is not None:
                extend_seq_list.append(slot)
            self._take(2)
            self.block_tables[slot] += 2
            return True
        return False

    def cached_token_gc(self, num_seqs: int) -> List[int]:
        """Give the chunks of idle pre-mapped slots back to the pool until ``num_seqs`` sequences can grow;
        returns the slots whose ranges must be unmapped (:367-379)."""
        gc_list: List[int] = []
        wanted = 2 * num_seqs - self._free
        for i in range(self.max_seqs):
            if self.cache_token and len(gc_list) < wanted and self.kv_cache_slot[i] == 0 \
                    and self.block_tables[i] == self.cache_token * 2:
                self.free_block_tables_block -= self.cache_token * 2
                self._give(self.cache_token * 2)
                self.block_tables[i] -= self.cache_token * 2
                gc_list.append(i)
        return gc_list

    # ------------------------------------------------------------------ release (:581-600)
    def free(self, seq: SequenceChunks) -> int:
        """Finished sequence: its slot keeps ``cache_token`` chunks per range if it holds that many
        (release_seq keeps them mapped); preempted sequence: everything goes back.  Returns the slot."""
        slot = seq.get_slot()
        if slot not in self.block_tables or slot == -1:
            return -1
        self.kv_cache_slot[slot] = 0
        held = self.block_tables[slot]
        if not seq.preempted:
            keep = 2 * self.cache_token if (self.cache_token and held >= 2 * self.cache_token) else 0
            self._give(held - keep)
            if keep:
                self.free_block_tables_block += keep
            self.block_tables[slot] = keep
        else:
            self._give(held)
            self.block_tables[slot] = 0
        return slot
