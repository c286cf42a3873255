"""``PagedAttention`` helper with the static methods of the reference's
``vllm/attention/ops/paged_attn.py`` (:30-225) for the contiguous-range (vTensor) cache."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch

from ... import _custom_ops as ops

_PARTITION_SIZE = 512  # paged_attn.py:10


@dataclass
class PagedAttentionMetadata:
    """paged_attn.py:13-27"""
    seq_lens_tensor: Optional[torch.Tensor]
    max_decode_seq_len: int
    block_tables: Optional[torch.Tensor]


class PagedAttention:
    @staticmethod
    def get_supported_head_sizes() -> List[int]:
        return [64, 80, 96, 112, 128, 256]  # paged_attn.py:33-34

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, ...]:
        return (2, num_blocks, block_size * num_kv_heads * head_size)  # paged_attn.py:36-43

    @staticmethod
    def split_kv_cache(kv_cache: torch.Tensor, num_kv_heads: int, head_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
        # paged_attn.py:45-59 (upstream paged layout, used by the paged scatter only)
        x = 16 // kv_cache.element_size()
        num_blocks = kv_cache.shape[1]
        key_cache = kv_cache[0].view(num_blocks, num_kv_heads, head_size // x, -1, x)
        value_cache = kv_cache[1].view(num_blocks, num_kv_heads, head_size, -1)
        return key_cache, value_cache

    @staticmethod
    def write_to_paged_cache(key, value, key_cache, value_cache, slot_m, slot_mapping, seq_lens, cache_seq_lens,
                             max_seq_len: int, num_kv_heads: int, head_size: int, kv_cache_dtype: str = "auto",
                             k_scale: float = 1.0, v_scale: float = 1.0) -> None:
        # paged_attn.py:61-87
        ops.reshape_and_cache(key, value, key_cache, value_cache, slot_m, slot_mapping, seq_lens, cache_seq_lens,
                              max_seq_len, num_kv_heads, head_size, kv_cache_dtype, k_scale, v_scale)

    @staticmethod
    def forward_decode(query, key_cache, value_cache, seq_lens, max_seq_len: int, kv_cache_dtype: str,
                       num_kv_heads: int, scale: float, alibi_slopes, kv_scale: float, slot_mapping,
                       v_scale: Optional[float] = None) -> torch.Tensor:
        # paged_attn.py:89-166.  The reference chooses between v1 and v2 by a heuristic that it
        # then overrides with v1 (:116-119); here one split-K kernel serves every length.
        output = torch.empty_like(query)
        ops.paged_attention_v1(output, query, key_cache, value_cache, num_kv_heads, scale, seq_lens, 1, max_seq_len,
                               alibi_slopes, kv_cache_dtype, kv_scale, slot_mapping, v_scale)
        return output

    @staticmethod
    def swap_blocks(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, src_to_dst: torch.Tensor) -> None:
        # paged_attn.py:203-216
        ops.swap_blocks(src_kv_cache[0], dst_kv_cache[0], src_to_dst)
        ops.swap_blocks(src_kv_cache[1], dst_kv_cache[1], src_to_dst)

    @staticmethod
    def copy_blocks(kv_caches: List[torch.Tensor], src_to_dists: torch.Tensor) -> None:
        # paged_attn.py:218-225
        ops.copy_blocks([kv[0] for kv in kv_caches], [kv[1] for kv in kv_caches], src_to_dists)
