"""One serving step around the vTensor KV cache, as the reference's engine runs it
(``vllm/engine/llm_engine.py:686-715`` ``LLMEngine.step`` and ``:565-625`` ``_process_model_outputs``,
``vllm/worker/worker.py:213-225,284-304`` ``cache_swap`` / ``execute_model``, ``vllm/worker/model_runner.py:
595-622,749-755`` metadata, ``vllm/model_executor/models/llama.py:307-351`` prologue and layers):

1. ``StepScheduler.schedule()`` decides what runs;
2. the slots of preempted sequences are unmapped (``preempt_seq``), swapped sequences move out or in;
3. the attention metadata of the batch is built, ``prepare_step`` advances every scheduled sequence's range
   (announcing the growth the scheduler foresaw to the map-ahead worker) and the caller's ``run_model`` runs the
   layers through the attention backend;
4. every scheduled sequence gets its sampled token accounted, and finished sequences release their slots
   (``release_seq``).

With a ``PrefixStore`` the loop also runs the prefix-cache branch that the reference sketches
(``vllm/core/scheduler.py:726-766``, ``vmm_allocator/radix_cache.py``): the scheduler looks every new prompt up,
a prompt that begins with a cached prefix has its slot started from the prefix's holder before the model runs
(whole chunks mapped a second time) and computes only the remaining rows, and a finished request's prompt rows
are kept as a new holder.  Holders take physical chunks that the manager does not count, so the loop tells the
store how many it may take (what the pool has beyond everything the manager has handed out or may still hand
out) and has it evict when a release leaves it above that.

The model itself (projections, sampling) is not part of this package: ``run_model(metadata, outputs)`` is the
caller's, and it calls ``VTensorImpl.forward`` once per layer with ``engine.gpu_cache[layer]``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional

import torch

from .. import vmm_allocator as vmm
from ..attention.backends.vtensor import VTensorBackend, VTensorMetadata
from ..core.scheduler import Request, SchedulerOutputs, StepScheduler
from .cache_engine import CacheEngine
from .prefix_store import PrefixStore
from .step import prepare_step


@dataclass
class StepResult:
    outputs: SchedulerOutputs
    metadata: Optional[VTensorMetadata]   # None when nothing ran
    finished: List[Request]


class StepLoop:
    """``prefix_store``: cached prefixes in slots of ``engine`` beyond the manager's ``max_seqs`` (requests need
    ``token_ids`` to take part).  ``pool_chunks``: physical chunks (all layers, K and V) that the engine and the
    store may take from the pool from now on; by default all that is free now."""

    def __init__(self, engine: CacheEngine, scheduler: StepScheduler, device: Optional[torch.device] = None,
                 prefix_store: Optional[PrefixStore] = None, pool_chunks: Optional[int] = None):
        self.engine = engine
        self.scheduler = scheduler
        self.device = torch.device("cuda", engine.device) if device is None else device
        self.prefix_store = prefix_store
        if prefix_store is not None:
            mgr = scheduler.block_manager
            if mgr.cache_token:
                raise ValueError("a prompt that starts from a cached prefix needs an empty slot: no pre-mapped slots")
            if any(s < mgr.max_seqs for s in prefix_store.free_slots):
                raise ValueError("the prefix store's slots must lie beyond the slots the manager hands out")
            free = vmm.showFreeBlocks()
            pool_chunks = free if pool_chunks is None else int(pool_chunks)
            if pool_chunks > free or pool_chunks < engine.num_layers * mgr.get_num_free_gpu_blocks():
                raise ValueError("pool_chunks must cover the manager's chunks in every layer and be free in the pool")
            self._pool_floor = free - pool_chunks       # free chunks of the pool that are not this loop's
            prefix_store.room = self.prefix_room
            if scheduler.prefix_lookup is None:
                scheduler.prefix_lookup = prefix_store.lookup

    def prefix_room(self) -> int:
        """Physical chunks the prefix store may still take: what the pool has free (counting what slots that no
        sequence owns any more are about to give back), less what the manager may still hand out and what it has
        handed out to slots that have not mapped it yet."""
        eng, mgr = self.engine, self.scheduler.block_manager
        owed = mgr.get_num_free_gpu_blocks()
        for slot in range(mgr.max_seqs):
            mapped = 2 * (eng.vmm_kvcache_segment[slot].actual_size // eng.chunk_bytes)
            if mgr.kv_cache_slot[slot]:
                owed += max(0, mgr.block_tables[slot] - mapped)
            else:
                owed -= mapped
        return vmm.showFreeBlocks() - self._pool_floor - eng.num_layers * owed

    def build_metadata(self, out: SchedulerOutputs) -> VTensorMetadata:
        """model_runner.py:595-622: prompts first, then decodes; per-sequence slot ids; ``extend_seq_list``
        names, at its place in the batch, every sequence whose ranges grow in this step."""
        eng, dev = self.engine, self.device
        seqs = out.prompts + out.decodes
        slots = [r.slot for r in seqs]
        seq_lens = [r.total_len for r in seqs]
        n_pre = len(out.prompts)
        grow = set(out.extend_list)
        # a prompt behind a cached prefix runs the rows after it (scheduler.py:757-766)
        cached = [r.prefix_rows for r in out.prompts] + [0] * len(out.decodes)
        query_lens = [n - c for n, c in zip(seq_lens[:n_pre], cached)]
        meta = VTensorBackend.make_metadata(
            num_prefills=n_pre, num_prefill_tokens=sum(query_lens), num_decode_tokens=len(out.decodes),
            slot_mapping=torch.tensor(slots, dtype=torch.int64, device=dev), seq_lens=seq_lens,
            seq_lens_tensor=torch.tensor(seq_lens, dtype=torch.int32, device=dev),
            max_query_len=max(query_lens) if n_pre else None,
            max_prefill_seq_len=max(seq_lens[:n_pre]) if n_pre else 0,
            max_decode_seq_len=max(seq_lens[n_pre:]) if out.decodes else 0, query_start_loc=None, seq_start_loc=None,
            context_lens_tensor=None, block_tables=None, is_extend=int(bool(grow)), kv_batch_stride=eng.kv_batch_stride,
            kv_num_heads=eng.num_kv_heads, kv_head_size=eng.head_size, max_seq_len=max(seq_lens),
            slot_mapping_list=slots, set_used_size=cached if any(cached) else [0] * len(slots),
            extend_seq_list=[s if s in grow else -1 for s in slots], use_cuda_graph=False)
        if any(cached):
            meta.query_lens = query_lens
        meta.k_cache_segment_ptr_list = eng.k_cache_ptr          # model_runner.py:749-755
        meta.v_cache_segment_ptr_list = eng.v_cache_ptr
        meta.kvcache_segment = [eng.vmm_kvcache_segment[s] for s in slots]
        return meta

    def step(self, run_model: Callable[[VTensorMetadata, SchedulerOutputs], None]) -> StepResult:
        eng = self.engine
        out = self.scheduler.schedule()
        stream = torch.cuda.current_stream(self.device)
        if out.preempted_slot:                                            # llm_engine.py:700-701
            # (the engine has read the last step's sampled tokens by now; a caller that queues steps without
            # reading anything back must not lose chunks under kernels that are still running)
            stream.synchronize()
            for slot in out.preempted_slot:
                eng.vmm_kvcache_segment[slot].preempt_seq(slot)
        if out.swapped_out:                                               # worker.py:213-225
            eng.swap_out([r.swap_slot for r in out.swapped_out], keys=[("req", r.request_id) for r in out.swapped_out])
        store = self.prefix_store
        if store is not None:
            for req, holder, rows in out.prefix_hits:                     # the slot begins as the prefix
                try:
                    store.start_from(req.slot, holder, rows)
                except RuntimeError:       # the pool ran dry under a map-ahead request: the prompt runs in full
                    req.prefix_rows = 0    # (its chunks were claimed for all of its rows)
            store.end_step()
            if out.recompute or out.swapped_out:
                store.make_room()      # a slot that shared a holder's chunks gave the pool less than its claim
        if out.swapped_in:
            eng.swap_in([r.slot for r in out.swapped_in], keys=[("req", r.request_id) for r in out.swapped_in])
        meta = None
        if out.prompts or out.decodes:
            meta = self.build_metadata(out)
            prepare_step(meta, eng.gpu_cache)                             # llama.py:307-341
            run_model(meta, out)                                          # llama.py:343-351
        finished = self.scheduler.on_step_done(out)
        if finished:                                                      # llm_engine.py:607-618
            stream.synchronize()                                          # the step's kernels have read the ranges
            for req in finished:
                if store is not None and req.token_ids is not None:
                    try:                                                  # the prompt's rows stay as a cached prefix
                        store.keep(req.token_ids, req.final_slot)
                    except RuntimeError:                                  # no slot or no chunks for it: not cached
                        pass
                eng.vmm_kvcache_segment[req.final_slot].release_seq(req.final_slot)
            if store is not None:
                store.make_room()
        return StepResult(out, meta, finished)
