"""The attention backend of this package: same interface and metadata fields as the reference's
one working backend (``vllm/attention/backends/xformers.py``: ``XFormersBackend`` :25-62,
``XFormersMetadata`` :65-211, ``XFormersImpl`` :214-433), with the cache write and the decode
attention served by the HIP kernels of ``libvtkv.so``.

Decode steps, prompt runs and batches that mix the two are served (prompt tokens first, then one token
per decode sequence, as upstream lays a batch out; the fork schedules the two kinds apart).  A prompt run
writes its rows into the cache and then attends over the ranges causally; without a cache (the engine's
profiling run) it attends over the key/value tensors themselves.  The sequence-wise metadata of the fork
(``slot_mapping`` = one slot id per sequence, ``slot_m``, ``seq_lens_tensor``) is ordered like the batch.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple, Type

import torch

from ..ops.paged_attn import PagedAttention, PagedAttentionMetadata
from .abstract import AttentionBackend, AttentionImpl, AttentionMetadata


class VTensorBackend(AttentionBackend):
    @staticmethod
    def get_name() -> str:
        return "vtensor-hip"

    @staticmethod
    def get_impl_cls() -> Type["VTensorImpl"]:
        return VTensorImpl

    @staticmethod
    def make_metadata(*args, **kwargs) -> "VTensorMetadata":
        return VTensorMetadata(*args, **kwargs)

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, ...]:
        return PagedAttention.get_kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size)

    @staticmethod
    def swap_blocks(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, src_to_dst: torch.Tensor) -> None:
        PagedAttention.swap_blocks(src_kv_cache, dst_kv_cache, src_to_dst)

    @staticmethod
    def copy_blocks(kv_caches: List[torch.Tensor], src_to_dists: torch.Tensor) -> None:
        PagedAttention.copy_blocks(kv_caches, src_to_dists)


@dataclass
class VTensorMetadata(AttentionMetadata, PagedAttentionMetadata):
    """Field for field the reference's XFormersMetadata (xformers.py:65-125)."""
    seq_lens: Optional[List[int]]
    seq_lens_tensor: Optional[torch.Tensor]
    max_query_len: Optional[int]
    max_prefill_seq_len: int
    max_decode_seq_len: int
    query_start_loc: Optional[torch.Tensor]
    seq_start_loc: Optional[torch.Tensor]
    context_lens_tensor: Optional[torch.Tensor]
    is_extend: int
    kv_batch_stride: int
    kv_num_heads: int
    kv_head_size: int
    max_seq_len: int
    slot_mapping_list: List[int]
    set_used_size: List[int]
    extend_seq_list: List[int]
    use_cuda_graph: bool
    cache_seq_lens: Optional[torch.Tensor] = None
    slot_m: Optional[torch.Tensor] = None
    k_cache_segment_ptr_list: Optional[List[torch.Tensor]] = None
    v_cache_segment_ptr_list: Optional[List[torch.Tensor]] = None
    kvcache_segment: Optional[list] = None
    decode_seq_len: Optional[torch.Tensor] = None
    # query tokens per prompt when a prompt continues behind rows that are already cached (a reused
    # prefix, a later chunk of a long prompt); None: every prompt is attended in full (query = all rows)
    query_lens: Optional[List[int]] = None
    query_lens_tensor: Optional[torch.Tensor] = None  # the same on the GPU (int32), made by prepare_step
    # the decode sequences' lengths of THIS step as a C array: made by prepare_step from seq_lens every step (never
    # by forward, so a metadata object that is reused or changed between steps cannot carry stale lengths)
    _host_decode_lens: Optional[object] = None
    _cached_prefill_metadata: Optional["VTensorMetadata"] = None
    _cached_decode_metadata: Optional["VTensorMetadata"] = None

    def _carry(self) -> Dict:
        return dict(is_extend=self.is_extend, kv_batch_stride=self.kv_batch_stride, kv_num_heads=self.kv_num_heads,
                    kv_head_size=self.kv_head_size, max_seq_len=self.max_seq_len,
                    slot_mapping_list=self.slot_mapping_list, set_used_size=self.set_used_size,
                    cache_seq_lens=self.cache_seq_lens, slot_m=self.slot_m,
                    k_cache_segment_ptr_list=self.k_cache_segment_ptr_list,
                    v_cache_segment_ptr_list=self.v_cache_segment_ptr_list, kvcache_segment=self.kvcache_segment)

    @property
    def prefill_metadata(self) -> Optional["VTensorMetadata"]:
        # xformers.py:138-174
        if self.num_prefills == 0:
            return None
        if self._cached_prefill_metadata is None:
            self._cached_prefill_metadata = VTensorMetadata(
                num_prefills=self.num_prefills, num_prefill_tokens=self.num_prefill_tokens, num_decode_tokens=0,
                slot_mapping=self.slot_mapping[:self.num_prefills], seq_lens=self.seq_lens[:self.num_prefills],
                seq_lens_tensor=self.seq_lens_tensor[:self.num_prefills], max_query_len=self.max_query_len,
                max_prefill_seq_len=self.max_prefill_seq_len, max_decode_seq_len=0,
                query_start_loc=None if self.query_start_loc is None else self.query_start_loc[:self.num_prefills + 1],
                seq_start_loc=None,
                context_lens_tensor=None if self.context_lens_tensor is None else self.context_lens_tensor[:self.num_prefills],
                block_tables=None if self.block_tables is None else self.block_tables[:self.num_prefills],
                use_cuda_graph=False, extend_seq_list=[], **self._carry())
        return self._cached_prefill_metadata

    @property
    def decode_metadata(self) -> Optional["VTensorMetadata"]:
        # xformers.py:176-211
        if self.num_decode_tokens == 0:
            return None
        if self._cached_decode_metadata is None:
            self._cached_decode_metadata = VTensorMetadata(
                num_prefills=0, num_prefill_tokens=0, num_decode_tokens=self.num_decode_tokens,
                slot_mapping=self.slot_mapping[self.num_prefills:], seq_lens=None,
                seq_lens_tensor=self.seq_lens_tensor[self.num_prefills:],
                max_query_len=None, max_prefill_seq_len=0, max_decode_seq_len=self.max_decode_seq_len,
                query_start_loc=None, seq_start_loc=None, context_lens_tensor=None,
                block_tables=None if self.block_tables is None else self.block_tables[self.num_prefills:],
                use_cuda_graph=self.use_cuda_graph, extend_seq_list=self.extend_seq_list, **self._carry())
        return self._cached_decode_metadata


class VTensorImpl(AttentionImpl[VTensorMetadata]):
    """xformers.py:214-433 with the external flash-decoding call replaced by the in-tree kernel."""

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: Optional[int] = None,
                 alibi_slopes: Optional[List[float]] = None, sliding_window: Optional[int] = None,
                 kv_cache_dtype: str = "auto") -> None:
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        if alibi_slopes is not None:
            alibi_slopes = torch.tensor(alibi_slopes, dtype=torch.float32)
        self.alibi_slopes = alibi_slopes
        self.sliding_window = sliding_window
        self.kv_cache_dtype = kv_cache_dtype
        assert self.num_heads % self.num_kv_heads == 0
        self.num_queries_per_kv = self.num_heads // self.num_kv_heads
        supported = PagedAttention.get_supported_head_sizes()
        if head_size not in supported:
            raise ValueError(f"Head size {head_size} is not supported by PagedAttention. "
                             f"Supported head sizes are: {supported}.")
        if sliding_window is not None:
            raise ValueError("sliding-window attention is not supported by the vtensor backend")
        # one launch for cache write + attention in pure decode steps; False = two launches
        self.fuse_decode_append = True

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, key_cache, value_cache,
                attn_metadata: VTensorMetadata, kv_scale: float = 1.0, v_scale: Optional[float] = None) -> torch.Tensor:
        """query [N, Hq*D], key/value [N, Hkv*D]; key_cache / value_cache are the per-layer
        ``KV_cache`` handles (xformers.py:269-278), or None in the engine's profiling run; returns
        [N, Hq*D].  The token batch holds the prompt tokens of ``num_prefills`` sequences first, then one
        token of each decode sequence (xformers.py:314-329); per-sequence metadata (``slot_mapping``,
        ``slot_m``, ``seq_lens_tensor``) is ordered the same way."""
        from ... import _custom_ops as ops

        if query.dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise ValueError(f"the vtensor backend runs bfloat16, float16 and float32 models, not {query.dtype}")
        # (float32 models run the separate calls over a float32 cache: the one-launch step is built for 16-bit models)
        fuse = self.fuse_decode_append and query.dtype != torch.float32
        query = query.view(-1, self.num_heads, self.head_size)
        key = key.view(-1, self.num_kv_heads, self.head_size)
        value = value.view(-1, self.num_kv_heads, self.head_size)
        vs = kv_scale if v_scale is None else v_scale
        meta = attn_metadata
        num_prefill_tokens = meta.num_prefill_tokens
        num_decode_tokens = meta.num_decode_tokens
        n_pre = meta.num_prefills
        assert key.shape[0] == num_prefill_tokens + num_decode_tokens
        assert value.shape[0] == num_prefill_tokens + num_decode_tokens

        if key_cache is None:
            # xformers.py:336-343 with kv_caches = [None] * layers (worker.py:157, model_runner.py:846): the
            # engine's profiling run.  Nothing is cached; the prompts attend over their own key/value rows.
            if num_decode_tokens:
                raise ValueError("decode tokens need a KV cache")
            output = torch.empty_like(query)
            if num_prefill_tokens:
                self._attend_packed(output, query, key, value, list(meta.seq_lens[:n_pre]))
            return output.view(-1, self.num_heads * self.head_size)

        k_table = meta.k_cache_segment_ptr_list[key_cache.layer_index]
        v_table = meta.v_cache_segment_ptr_list[value_cache.layer_index]
        output = torch.empty_like(query)

        if n_pre > 0:
            # xformers.py:290-312, prompt form: every prompt writes its new rows (all of its rows, or the
            # query_lens rows that follow what is cached already) behind the bytes its range holds ...
            rows_t = meta.query_lens_tensor if meta.query_lens is not None else meta.seq_lens_tensor[:n_pre]
            PagedAttention.write_to_paged_cache(
                key[:num_prefill_tokens], value[:num_prefill_tokens], k_table, v_table, meta.slot_m[:n_pre],
                meta.slot_mapping[:n_pre], rows_t, meta.cache_seq_lens[:n_pre], meta.max_query_len,
                self.num_kv_heads, self.head_size, self.kv_cache_dtype, kv_scale, vs)
            # ... and xformers.py:331-386: the reference attends over the key/value tensors (plain prompt)
            # or over the cache through an external kernel (cached prefix); with the rows in the cache both
            # are one causal attention over the ranges.
            seq_lens = list(meta.seq_lens[:n_pre])
            query_lens = list(meta.query_lens[:n_pre]) if meta.query_lens is not None else seq_lens
            ops.prefill_attention(
                output[:num_prefill_tokens], query[:num_prefill_tokens], k_table, v_table, self.num_kv_heads,
                self.scale, query_lens, seq_lens, meta.slot_mapping[:n_pre], self.alibi_slopes, self.kv_cache_dtype,
                kv_scale, vs)

        if num_decode_tokens > 0:
            # xformers.py:388-431: one query token per decode sequence over its whole range.
            if n_pre == 0:  # the common case, a pure decode step: no views to make
                d_query, d_key, d_value, d_out = query, key, value, output
                d_slots, d_lens = meta.slot_mapping, meta.seq_lens_tensor
            else:
                d_query = query[num_prefill_tokens:]
                d_key, d_value = key[num_prefill_tokens:], value[num_prefill_tokens:]
                d_slots = meta.slot_mapping[n_pre:]
                d_lens = meta.seq_lens_tensor[n_pre:]
                d_out = output[num_prefill_tokens:]
            max_len = meta.max_decode_seq_len if n_pre > 0 and meta.max_decode_seq_len else meta.max_seq_len
            if fuse and (self.head_size == 128 or self.kv_cache_dtype == "auto"):
                # the cache write (xformers.py:310-312) and the decode attention (:357-371) in one launch.
                # The row goes to position seq_len - 1 of each range, which is where slot_m points in the
                # reference's flow (llama.py:340: the bytes used before this step).  Where the metadata also
                # holds the lengths on the host (model_runner.py:607 passes both), up to 512 of them travel
                # with the kernel arguments, which spares the kernel a dependent load at its start.
                # prepare_step makes that array once per step for all layers; a step that is recorded into a graph
                # (use_cuda_graph, or a stream that is capturing) reads the device lengths, since values passed as
                # kernel arguments would be frozen into the recording.
                host_lens = meta._host_decode_lens
                if (host_lens is not None and len(host_lens) == num_decode_tokens and not meta.use_cuda_graph
                        and not torch.cuda.is_current_stream_capturing()):
                    d_lens = host_lens
                ops.decode_append_attention(
                    d_out, d_query, d_key, d_value, k_table, v_table, self.num_kv_heads, self.scale, d_lens, max_len,
                    self.alibi_slopes, d_slots, kv_cache_dtype=self.kv_cache_dtype, kv_scale=kv_scale, v_scale=vs)
            else:
                PagedAttention.write_to_paged_cache(
                    d_key, d_value, k_table, v_table, meta.slot_m[n_pre:], d_slots, None, None, 1,
                    self.num_kv_heads, self.head_size, self.kv_cache_dtype, kv_scale, vs)
                ops.paged_attention_v1(d_out, d_query, k_table, v_table, self.num_kv_heads, self.scale, d_lens, 1,
                                       max_len, self.alibi_slopes, self.kv_cache_dtype, kv_scale, d_slots, vs)
        return output.view(-1, self.num_heads * self.head_size)

    def _attend_packed(self, output: torch.Tensor, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                       seq_lens: List[int]) -> None:
        """Causal self-attention of packed prompts over their own key/value rows, without a cache: sequence
        b's rows [start_b, start_b + len_b) of ``key`` / ``value`` already are a token-major [T, Hkv, D]
        range, so the prompt kernel runs on them through a pointer table made for the call."""
        from ... import _custom_ops as ops

        key, value = key.contiguous(), value.contiguous()
        row = self.num_kv_heads * self.head_size * key.element_size()
        starts, at = [], 0
        for n in seq_lens:
            starts.append(at)
            at += n
        if at != query.shape[0]:
            raise ValueError(f"seq_lens add up to {at} tokens, the batch holds {query.shape[0]}")
        dev = query.device
        k_table = torch.tensor([key.data_ptr() + s * row for s in starts], dtype=torch.int64, device=dev)
        v_table = torch.tensor([value.data_ptr() + s * row for s in starts], dtype=torch.int64, device=dev)
        slots = torch.arange(len(seq_lens), dtype=torch.int64, device=dev)
        # the rows are in the model's dtype whatever the cache would hold
        ops.prefill_attention(output, query, k_table, v_table, self.num_kv_heads, self.scale, seq_lens, seq_lens,
                              slots, self.alibi_slopes, "auto", 1.0, 1.0)
