"""Cached prefixes on the GPU side: the holders behind a :class:`glake_amd.core.radix_cache.RadixCache`.

The reference plans this (``vllm/core/scheduler.py:726-766`` looks a prompt up in ``prefix_cache``,
``vmm_allocator/radix_cache.py:177-188`` splits a node with ``vmmAllocator.split_and_copy``) but its allocator has
no ``split_and_copy`` and the scheduler always looks up the empty prompt.  Here a holder is a sequence slot of the
``CacheEngine`` set aside for cached prefixes, and every "copy" is ``KVcacheSegment.share_prefix``: the whole
chunks of a prefix are mapped a second time (one physical chunk, several addresses), only the partly filled chunk
at its end is copied.  A chunk returns to the pool when the last slot that maps it lets go.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence, Tuple

import torch

from ..core.radix_cache import RadixCache
from .cache_engine import CacheEngine


class PrefixStore:
    """``cache_slots``: the slots of ``engine`` that hold cached prefixes (the scheduler must not hand them to
    running sequences).  ``room() -> int``: physical chunks the store may still take from the pool (below zero:
    it holds chunks that running sequences have been promised); None: whatever the pool has.  A new holder takes
    chunks only for the partly filled end of its prefix; the store evicts least recently used prefixes to stay
    within ``room``, and a prefix that cannot be had that way is not cached (``keep``) or not found (``lookup``)."""

    def __init__(self, engine: CacheEngine, cache_slots: Sequence[int], room: Optional[Callable[[], int]] = None):
        self.engine = engine
        self.room = room
        self.token_size = engine.token_size
        self.free_slots: List[int] = list(cache_slots)
        self.rows = {}                                   # cache slot -> rows it holds
        self.tree = RadixCache(self.token_size, self._split)
        self.evicted_rows = 0                            # rows of all holders evicted so far
        self._pinned = []                                # nodes looked up in this step: not evicted before end_step

    def _stream(self) -> int:
        return torch.cuda.current_stream().cuda_stream

    def _own_chunks(self, nbytes: int) -> int:
        """Chunks a holder of ``nbytes`` bytes per range takes from the pool: what lies behind the prefix's whole
        chunks, up to the end of its V rows, in every K and V range."""
        gran = self.engine.chunk_bytes
        tail = nbytes + self.engine.value_skew - (nbytes // gran) * gran if nbytes else 0
        return 2 * self.engine.num_layers * ((tail + gran - 1) // gran)

    def _take_slot(self, nbytes: int) -> int:
        if not self.free_slots:
            self.evict(1)                                # the least recently used prefix nobody refers to
        if not self.free_slots:
            raise RuntimeError("no slot left for a cached prefix: every cached prefix is in use")
        need = self._own_chunks(nbytes)
        while self.room is not None and self.room() < need:
            if self.evict(1) == 0:
                raise RuntimeError("no chunks left for a cached prefix")
        return self.free_slots.pop()

    def make_room(self) -> int:
        """Evict until ``room()`` is not negative (or nothing is left to evict).  Returns the rows evicted."""
        gone = 0
        while self.room is not None and self.room() < 0:
            rows = self.evict(1)
            if rows == 0:
                break
            gone += rows
        return gone

    def _split(self, slot: int, nbytes: int) -> int:
        """The holder of the first ``nbytes`` bytes of what ``slot`` holds (radix_cache.py:184)."""
        new = self._take_slot(nbytes)
        self._share(new, slot, nbytes)
        self.rows[new] = nbytes // self.token_size
        return new

    def _share(self, new: int, src: int, nbytes: int) -> None:
        """Start the free holder ``new`` from the first ``nbytes`` bytes of slot ``src``; the holder goes back to
        the free ones if that fails (the pool can still run dry under a map-ahead request)."""
        segs = self.engine.vmm_kvcache_segment
        try:
            segs[new].share_prefix(segs[src], nbytes, self._stream())
        except Exception:
            self.free_slots.append(new)
            raise

    # ------------------------------------------------------------------ the engine's calls
    def lookup(self, tokens: Sequence[int]) -> Tuple[Optional[int], int]:
        """(cache slot, rows) of the longest cached prefix of ``tokens`` that leaves at least one token to
        run (scheduler.py:757-766 runs ``prefix_len - 1`` cached tokens when the whole prompt is cached)."""
        try:
            node = self.tree.match_node(tokens)          # (cuts a holder when the match ends inside an edge)
        except RuntimeError:                             # no slot or no chunks for the cut: the tree is as it was
            return None, 0
        if node is self.tree.root_node:
            return None, 0
        # a later lookup of the same step may have to evict for room: not what this one has just handed out
        self.tree.inc_ref_counter(node)
        self._pinned.append(node)
        return node.value[0], min(node.prefix_len, len(tokens) - 1)

    def end_step(self) -> None:
        """The step has started its sequences from what the lookups handed out: those holders may go again."""
        for node in self._pinned:
            self.tree.dec_ref_counter(node)
        self._pinned = []

    def start_from(self, run_slot: int, cache_slot: int, rows: int) -> None:
        """Begin the (empty) running slot with ``rows`` cached rows of ``cache_slot``."""
        segs = self.engine.vmm_kvcache_segment
        segs[run_slot].share_prefix(segs[cache_slot], rows * self.token_size, self._stream())

    def keep(self, tokens: Sequence[int], run_slot: int) -> int:
        """Remember the rows of ``tokens`` that ``run_slot`` holds (call before the slot is released).  Returns
        how many leading tokens the tree had already."""
        if len(tokens) == 0:
            return 0
        new = self._take_slot(len(tokens) * self.token_size)
        self._share(new, run_slot, len(tokens) * self.token_size)
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
        rows = self.tree.evict(num_tokens, lambda value: self._drop(value[0]))
        self.evicted_rows += rows
        return rows
