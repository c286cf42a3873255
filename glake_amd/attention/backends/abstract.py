"""Attention backend interface, same shape as the reference's
``vllm/attention/backends/abstract.py`` (:9-127) so an engine written against it can select
this package's backend without changes."""
from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass, fields
from typing import Any, Dict, Generic, List, Optional, Set, Tuple, Type, TypeVar

import torch


class AttentionBackend(ABC):
    @staticmethod
    @abstractmethod
    def get_name() -> str: ...

    @staticmethod
    @abstractmethod
    def get_impl_cls() -> Type["AttentionImpl"]: ...

    @staticmethod
    @abstractmethod
    def make_metadata(*args, **kwargs) -> "AttentionMetadata": ...

    @staticmethod
    @abstractmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, ...]: ...

    @staticmethod
    @abstractmethod
    def swap_blocks(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, src_to_dst: torch.Tensor) -> None: ...

    @staticmethod
    @abstractmethod
    def copy_blocks(kv_caches: List[torch.Tensor], src_to_dists: torch.Tensor) -> None: ...


@dataclass
class AttentionMetadata:
    """Prefill and decode metadata batched together (abstract.py:55-96)."""
    num_prefills: int
    num_prefill_tokens: int
    num_decode_tokens: int
    slot_mapping: torch.Tensor

    @property
    @abstractmethod
    def prefill_metadata(self) -> Optional["AttentionMetadata"]: ...

    @property
    @abstractmethod
    def decode_metadata(self) -> Optional["AttentionMetadata"]: ...

    def asdict_zerocopy(self, skip_fields: Optional[Set[str]] = None) -> Dict[str, Any]:
        skip_fields = skip_fields or set()
        return {f.name: getattr(self, f.name) for f in fields(self) if f.name not in skip_fields}


T = TypeVar("T", bound=AttentionMetadata)


class AttentionImpl(ABC, Generic[T]):
    @abstractmethod
    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: Optional[int] = None,
                 alibi_slopes: Optional[List[float]] = None, sliding_window: Optional[int] = None,
                 kv_cache_dtype: str = "auto") -> None: ...

    @abstractmethod
    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, kv_cache, attn_metadata: T,
                kv_scale: float = 1.0) -> torch.Tensor: ...
