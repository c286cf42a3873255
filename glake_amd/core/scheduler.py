"""The scheduling decisions a serving step needs around the per-sequence KV ranges: which prompts are
admitted into which slots, which running sequences take one more token, who is preempted when the chunk pool
runs short, which slots have to grow in the coming step, and what is released when a sequence finishes.

Restates the vTensor part of the reference's scheduler over :class:`ChunkSpaceManager`:
``vllm/core/scheduler.py:425-522`` (``_schedule_running``: ``can_append_slots`` -> else preempt the
last sequence of the queue -> ``append_slots`` fills ``extend_list``), ``:726-766`` (``_schedule_prefills``:
``can_allocate`` / ``allocate`` give a prompt its slot), ``:781-873`` (``_schedule_default``: prompts first, and
no decodes in a step that runs prompts), ``:1160-1225`` (preemption by recompute or by swap), and the engine's
bookkeeping around a step, ``vllm/engine/llm_engine.py:607-618`` (release the slots of finished sequences) and
``:686-701`` (unmap the preempted slots before the model runs).  Sequence groups, LoRA, beam search and chunked
prefill are left out: one sequence per request, prompts and decodes in separate steps, as the fork runs.

The prefix-cache branch of ``_schedule_prefills`` (``scheduler.py:726-766``) is there in the form the reference
sketches and switches off (it looks up the empty prompt, ``:728``, and never inserts, ``:1097``): with a
``prefix_lookup`` a prompt that begins with a cached prefix is admitted with ``prefix_rows`` of its rows already
in place -- at least one token is left to run (``:757-766``) -- and the step computes only the rest.  Here the
prompt still gets a slot of its own, which the step loop starts from the cached prefix by mapping the prefix's
chunks a second time; the reference would hand the cached slot itself to the new sequence (``set_slot``).

The objects here only count; the GPU side (``CacheEngine``, ``prepare_step``, the attention backend) is driven
from their output by :class:`glake_amd.worker.step_loop.StepLoop`.
"""
from __future__ import annotations

import enum
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, List, Optional, Sequence, Tuple

from .chunk_manager import AllocStatus, ChunkSpaceManager, SequenceChunks


class SeqStatus(enum.Enum):
    WAITING = enum.auto()
    RUNNING = enum.auto()
    SWAPPED = enum.auto()
    FINISHED = enum.auto()
    IGNORED = enum.auto()   # the prompt can never fit (scheduler.py:741-748)


class PreemptionMode(enum.Enum):
    RECOMPUTE = enum.auto()  # drop the rows, run the prompt (and what was generated) again later
    SWAP = enum.auto()       # move the rows to pinned host memory and back


@dataclass
class Request:
    """One sequence: a prompt of ``prompt_len`` tokens that generates up to ``max_new_tokens``."""
    request_id: int
    prompt_len: int
    max_new_tokens: int
    status: SeqStatus = SeqStatus.WAITING
    generated: int = 0      # tokens sampled so far (the last one's row is not in the cache yet)
    num_cached: int = 0     # rows of this sequence in its slot's ranges
    chunks: Optional[SequenceChunks] = None
    preemptions: int = 0
    swap_slot: int = -1     # swapped out in this step: the slot its rows are still in
    final_slot: int = -1    # finished: the slot to release
    token_ids: Optional[Sequence[int]] = None  # the prompt's tokens, for the prefix lookup (None: never looked up)
    prefix_rows: int = 0    # rows of the coming prompt run that a cached prefix provides (set at admission)

    @property
    def total_len(self) -> int:
        return self.prompt_len + self.generated

    @property
    def slot(self) -> int:
        return -1 if self.chunks is None else self.chunks.get_slot()

    def is_finished(self) -> bool:
        return self.status in (SeqStatus.FINISHED, SeqStatus.IGNORED)


@dataclass
class SchedulerOutputs:
    """What one step runs (scheduler.py ``SchedulerOutputs``, the fields the vTensor path uses)."""
    prompts: List[Request] = field(default_factory=list)       # run their whole total_len as a prompt
    decodes: List[Request] = field(default_factory=list)       # one new token each
    preempted_slot: List[int] = field(default_factory=list)    # slots whose ranges are unmapped before the step
    extend_list: List[int] = field(default_factory=list)       # slots that grow by a K and a V chunk in this step
    swapped_out: List[Request] = field(default_factory=list)   # moved to host memory before the step
    swapped_in: List[Request] = field(default_factory=list)    # brought back before the step (they also decode)
    ignored: List[Request] = field(default_factory=list)
    recompute: List[Request] = field(default_factory=list)     # preempted by recompute: back at the head of waiting
    # prompts of this step that start from a cached prefix: (request, holder of the prefix, rows)
    prefix_hits: List[Tuple[Request, object, int]] = field(default_factory=list)
    num_batched_tokens: int = 0

    def is_empty(self) -> bool:
        return not (self.prompts or self.decodes or self.swapped_out or self.swapped_in or self.preempted_slot)


class StepScheduler:
    """FCFS scheduler over slots and chunk counts.

    ``token_size``: bytes of one token row of one range; ``value_skew``: what the engine sets the V rows off
    by (claimed with the first rows, as ``SequenceChunks`` does); ``preemption``: what happens to a sequence
    that loses its chunks; ``prefix_lookup(tokens) -> (holder, rows)``: the longest cached prefix of a prompt
    (``(None, 0)`` if none), e.g. ``PrefixStore.lookup``."""

    def __init__(self, manager: ChunkSpaceManager, token_size: int, max_num_seqs: int, max_num_batched_tokens: int,
                 chunk_bytes: int = 2 << 20, value_skew: int = 0,
                 preemption: PreemptionMode = PreemptionMode.RECOMPUTE, max_model_len: Optional[int] = None,
                 prefix_lookup: Optional[Callable[[Sequence[int]], Tuple[object, int]]] = None):
        self.block_manager = manager
        self.token_size = int(token_size)
        self.max_num_seqs = int(max_num_seqs)
        self.max_num_batched_tokens = int(max_num_batched_tokens)
        self.chunk_bytes = int(chunk_bytes)
        self.value_skew = int(value_skew)
        self.preemption = preemption
        self.prefix_lookup = prefix_lookup
        # scheduler.py:297-303: a prompt longer than this is ignored
        self.prompt_limit = min(max_model_len or max_num_batched_tokens, max_num_batched_tokens)
        self.waiting: Deque[Request] = deque()
        self.running: Deque[Request] = deque()
        self.swapped: Deque[Request] = deque()
        self.preempted_flag = False          # scheduler.py:450: set once anything was preempted
        self.num_cumulative_preemption = 0
        self._next_id = 0

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt_len: int, max_new_tokens: int, token_ids: Optional[Sequence[int]] = None) -> Request:
        if prompt_len <= 0 or max_new_tokens <= 0:
            raise ValueError("a request needs at least one prompt token and one token to generate")
        if token_ids is not None and len(token_ids) != prompt_len:
            raise ValueError("token_ids must hold the prompt's tokens")
        req = Request(self._next_id, int(prompt_len), int(max_new_tokens), token_ids=token_ids)
        self._next_id += 1
        self.waiting.append(req)
        return req

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running or self.swapped)

    def _new_chunks(self, num_tokens: int) -> SequenceChunks:
        """Sequence.__init__ -> _append_tokens_to_blocks(prompt) (sequence.py:342-360)."""
        c = SequenceChunks(self.token_size, self.chunk_bytes, self.value_skew)
        c.append_tokens(num_tokens)
        return c

    # ------------------------------------------------------------------ prompts (scheduler.py:653-779)
    def _schedule_prefills(self, out: SchedulerOutputs, num_curr_seqs: int) -> None:
        while self.waiting:
            req = self.waiting[0]
            num_new_tokens = req.total_len            # after a recompute the generated tokens are prompt too
            if num_new_tokens > self.prompt_limit:
                req.status = SeqStatus.IGNORED
                out.ignored.append(req)
                self.waiting.popleft()
                continue
            if num_curr_seqs + 1 > self.max_num_seqs:
                break
            # scheduler.py:726-766: rows a cached prefix provides need not be run; one token always is
            # (the lookup may cut a holder for the matched length: only asked once a slot could be had)
            holder, rows = None, 0
            if self.prefix_lookup is not None and req.token_ids is not None:
                holder, rows = self.prefix_lookup(req.token_ids)
                rows = min(int(rows), req.total_len - 1) if holder is not None else 0
            num_new_tokens -= rows
            if (out.num_batched_tokens + num_new_tokens > self.max_num_batched_tokens
                    or num_curr_seqs + 1 > self.max_num_seqs):
                break
            chunks = self._new_chunks(req.total_len)  # (a shared prefix is claimed in full: an upper bound)
            can = self.block_manager.can_allocate(chunks, self.preempted_flag)
            if can is AllocStatus.LATER:
                break
            if can is AllocStatus.NEVER:
                req.status = SeqStatus.IGNORED
                out.ignored.append(req)
                self.waiting.popleft()
                continue
            if not self.block_manager.allocate(chunks):
                break                                  # no slot is free
            req.chunks = chunks
            req.status = SeqStatus.RUNNING
            req.num_cached = 0
            req.prefix_rows = rows
            if rows:
                out.prefix_hits.append((req, holder, rows))
            self.waiting.popleft()
            out.prompts.append(req)
            out.num_batched_tokens += num_new_tokens
            num_curr_seqs += 1

    # ------------------------------------------------------------------ decodes (scheduler.py:395-522)
    def _preempt(self, req: Request, out: SchedulerOutputs) -> None:
        """scheduler.py:1160-1225: the sequence gives all its chunks back; by recompute it returns to the
        head of the waiting queue, by swap its rows are kept in host memory."""
        self.num_cumulative_preemption += 1
        req.preemptions += 1
        req.chunks.preempted = True
        slot = self.block_manager.free(req.chunks)
        if self.preemption is PreemptionMode.RECOMPUTE:
            out.preempted_slot.append(slot)           # llm_engine.py:700-701 -> preempt_seq
            req.status = SeqStatus.WAITING
            req.num_cached = 0
            req.chunks = None
            out.recompute.append(req)
        else:
            req.status = SeqStatus.SWAPPED
            req.swap_slot = slot                      # where the rows are until the step has moved them out
            out.swapped_out.append(req)

    def _schedule_running(self, out: SchedulerOutputs) -> None:
        mgr = self.block_manager
        queue = self.running
        self.running = deque()
        while queue:
            req = queue.popleft()
            scheduled = True
            while not mgr.can_append_slots(1):
                self.preempted_flag = True
                if queue:
                    self._preempt(queue.pop(), out)    # the lowest-priority sequence: the last one in
                elif mgr.can_append_slots(1, beta=mgr.free_block_tables_block) and (gc := mgr.cached_token_gc(1)):
                    out.preempted_slot.extend(gc)      # idle pre-mapped slots give their chunks up
                else:
                    self._preempt(req, out)            # nobody else left: the sequence itself
                    scheduled = False
                    break
            if scheduled:
                mgr.append_slots(req.chunks, out.extend_list)
                out.decodes.append(req)
                out.num_batched_tokens += 1
                self.running.append(req)

    # ------------------------------------------------------------------ swapped (scheduler.py:524-600)
    def _schedule_swapped(self, out: SchedulerOutputs) -> None:
        mgr = self.block_manager
        while self.swapped:
            req = self.swapped[0]
            if len(self.running) + 1 > self.max_num_seqs:
                break
            chunks = req.chunks                        # the sequence keeps its claim while it is swapped out
            if mgr.can_allocate(chunks, False) is not AllocStatus.OK:
                break
            chunks.preempted = False
            if not mgr.allocate(chunks):
                chunks.preempted = True
                break                                  # no slot is free
            req.status = SeqStatus.RUNNING
            self.swapped.popleft()
            out.swapped_in.append(req)
            out.decodes.append(req)
            out.num_batched_tokens += 1
            self.running.append(req)

    # ------------------------------------------------------------------ one step (scheduler.py:781-873)
    def schedule(self) -> SchedulerOutputs:
        out = SchedulerOutputs()
        if not self.swapped:                           # swapped sequences come before new prompts
            self._schedule_prefills(out, len(self.running))
        if not out.prompts:                            # no decodes in a step that runs prompts
            self._schedule_running(out)
            if not out.recompute and not out.swapped_out:
                self._schedule_swapped(out)
        self.waiting.extendleft(out.recompute)         # scheduler.py:842
        self.running.extend(out.prompts)
        self.swapped.extend(out.swapped_out)
        return out

    # ------------------------------------------------------------------ after the model ran
    def on_step_done(self, out: SchedulerOutputs) -> List[Request]:
        """Every scheduled sequence has its rows in the cache and samples one token
        (Sequence.append_token_id -> _append_tokens_to_blocks(1), sequence.py:320-329,342-360).  Returns the
        sequences that finished; their chunks are back in the manager's pool (scheduler.py:1095-1105) and
        their slots are what the engine releases (llm_engine.py:607-618)."""
        finished: List[Request] = []
        for req in out.prompts + out.decodes:
            req.num_cached = req.total_len
            req.generated += 1
            req.chunks.append_tokens(1)
            if req.generated >= req.max_new_tokens:
                req.status = SeqStatus.FINISHED
                finished.append(req)
        for req in finished:
            req.final_slot = self.block_manager.free(req.chunks)
        self.running = deque(r for r in self.running if r.status is SeqStatus.RUNNING)
        return finished
