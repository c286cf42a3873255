"""Cached prefixes on the GPU side: the holders behind a :class:`glake_amd.core.radix_cache.RadixCache`.

The reference plans this (``vllm/core/scheduler.py:726-766`` looks a prompt up in ``prefix_cache``,
``vmm_allocator/radix_cache.py:177-188`` splits a node with ``vmmAllocator.split_and_copy``) but its allocator has
no ``split_and_copy`` and the scheduler always looks up the empty prompt.  Here a holder is a sequence slot of the
``CacheEngine`` set aside for cached prefixes, and every "copy" is ``KVcacheSegment.share_prefix``: the whole
chunks of a prefix are mapped a second time (one physical chunk, several addresses), only the partly filled chunk
at its end is copied.  A chunk returns to the pool when the last slot that maps it lets go.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from ..core.radix_cache import RadixCache
from .cache_engine import CacheEngine


class PrefixStore:
    """``cache_slots``: the slots of ``engine`` that hold cached prefixes (the scheduler must not hand them to
    running sequences)."""

    def __init__(self, engine: CacheEngine, cache_slots: Sequence[int]):
        self.engine = engine
        self.token_size = engine.token_size
        self.free_slots: List[int] = list(cache_slots)
        self.rows = {}                                   # cache slot -> rows it holds
        self.tree = RadixCache(self.token_size, self._split)

    def _stream(self) -> int:
        return torch.cuda.current_stream().cuda_stream

    def _take_slot(self) -> int:
        if not self.free_slots:
            self.evict(1)                                # the least recently used prefix nobody refers to
        if not self.free_slots:
            raise RuntimeError("no slot left for a cached prefix: every cached prefix is in use")
        return self.free_slots.pop()

    def _split(self, slot: int, nbytes: int) -> int:
        """The holder of the first ``nbytes`` bytes of what ``slot`` holds (radix_cache.py:184)."""
        new = self._take_slot()
        segs = self.engine.vmm_kvcache_segment
        segs[new].share_prefix(segs[slot], nbytes, self._stream())
        self.rows[new] = nbytes // self.token_size
        return new

    # ------------------------------------------------------------------ the engine's calls
    def lookup(self, tokens: Sequence[int]) -> Tuple[Optional[int], int]:
        """(cache slot, rows) of the longest cached prefix of ``tokens`` that leaves at least one token to
        run (scheduler.py:757-766 runs ``prefix_len - 1`` cached tokens when the whole prompt is cached)."""
        slot, n = self.tree.match_prefix(tokens)
        if slot is None:
            return None, 0
        return slot, min(n, len(tokens) - 1)

    def start_from(self, run_slot: int, cache_slot: int, rows: int) -> None:
        """Begin the (empty) running slot with ``rows`` cached rows of ``cache_slot``."""
        segs = self.engine.vmm_kvcache_segment
        segs[run_slot].share_prefix(segs[cache_slot], rows * self.token_size, self._stream())

    def keep(self, tokens: Sequence[int], run_slot: int) -> int:
        """Remember the rows of ``tokens`` that ``run_slot`` holds (call before the slot is released).  Returns
        how many leading tokens the tree had already."""
        if len(tokens) == 0:
            return 0
        new = self._take_slot()
        segs = self.engine.vmm_kvcache_segment
        segs[new].share_prefix(segs[run_slot], len(tokens) * self.token_size, self._stream())
        self.rows[new] = len(tokens)
        try:
            known = self.tree.insert(tokens, new)
        except Exception:                                # no slot for a split: the tree is as it was
            self._drop(new)
            raise
        if known == len(tokens):                         # nothing new: the tree did not take the holder
            self._drop(new)
        return known

    def _drop(self, slot: int) -> int:
        rows = self.rows.pop(slot, 0)
        torch.cuda.current_stream().synchronize()        # the tail copy into or out of this slot has run
        self.engine.vmm_kvcache_segment[slot].preempt_seq(slot)
        self.free_slots.append(slot)
        return rows

    def evict(self, num_tokens: int) -> int:
        """Free cached prefixes, least recently used first, until ``num_tokens`` rows' worth is gone."""
        return self.tree.evict(num_tokens, lambda value: self._drop(value[0]))
