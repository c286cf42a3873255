"""Deterministic inputs of the golden cases: pure integer arithmetic, so every numpy version
and every machine produces the same arrays (nothing random is stored in the fixtures but the
expected outputs)."""
from __future__ import annotations

import numpy as np

LENS = [1, 15, 16, 17, 511, 512, 513, 1025]  # straddle the 16-token block and the 512-token partition
BLOCK_SIZE = 16
HEAD_SIZE = 128

# name -> (dtype, version, num_heads, num_kv_heads, alibi)
ATTENTION_CASES = {
    "f32_v1_gqa4": ("f32", 1, 8, 2, False),
    "f32_v2_gqa4": ("f32", 2, 8, 2, False),
    "f32_v1_gqa8": ("f32", 1, 8, 1, False),
    "f32_v2_mha": ("f32", 2, 4, 4, False),
    "f32_v1_alibi": ("f32", 1, 8, 2, True),
    "f32_v2_alibi": ("f32", 2, 8, 2, True),
    "bf16_v1_gqa4": ("bf16", 1, 8, 2, False),
    "bf16_v2_gqa4": ("bf16", 2, 8, 2, False),
    "bf16_v1_gqa8": ("bf16", 1, 8, 1, False),
    "bf16_v2_alibi": ("bf16", 2, 8, 2, True),
    # the other head sizes of the reference (vllm/attention/ops/paged_attn.py:33-34); a sixth field is the head size
    "bf16_v1_d64": ("bf16", 1, 8, 2, False, 64),
    "f32_v1_d80": ("f32", 1, 8, 2, False, 80),
    "bf16_v2_d96": ("bf16", 2, 8, 1, False, 96),
    "f32_v2_d112_alibi": ("f32", 2, 8, 2, True, 112),
    "bf16_v1_d256": ("bf16", 1, 4, 4, False, 256),
}


def _mix(i: np.ndarray, seed: int) -> np.ndarray:
    """splitmix64 finaliser on uint64 (wrap-around arithmetic)."""
    with np.errstate(over="ignore"):
        h = (i + np.uint64(seed)) * np.uint64(0x9E3779B97F4A7C15)
        h ^= h >> np.uint64(30)
        h *= np.uint64(0xBF58476D1CE4E5B9)
        h ^= h >> np.uint64(27)
        h *= np.uint64(0x94D049BB133111EB)
        h ^= h >> np.uint64(31)
    return h


def lattice(shape, seed: int) -> np.ndarray:
    """float32 multiples of 1/8 in [-2, 2] (exact in bf16), pseudo-random, variance ~1.4."""
    n = int(np.prod(shape))
    h = _mix(np.arange(n, dtype=np.uint64), seed)
    return (((h >> np.uint64(40)) % np.uint64(33)).astype(np.float32) / 8.0 - 2.0).reshape(shape)


def permutation(n: int, seed: int) -> np.ndarray:
    return np.argsort(_mix(np.arange(n, dtype=np.uint64), seed), kind="stable").astype(np.int32)


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    return (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)  # lattice values are exact in bf16


def attention_case(name: str):
    """Inputs of one attention case in the reference's paged layout (block 16)."""
    dtype, version, hq, hkv, alibi = ATTENTION_CASES[name][:5]
    seed = sum(ord(c) for c in name) * 1000
    d, bs = (ATTENTION_CASES[name][5] if len(ATTENTION_CASES[name]) > 5 else HEAD_SIZE), BLOCK_SIZE
    x = 4 if dtype == "f32" else 8
    lens = np.array(LENS, np.int32)
    nblk = (lens + bs - 1) // bs
    total = int(nblk.sum())
    num_blocks = total + 7  # a few unused blocks
    perm = permutation(num_blocks, seed + 1)
    block_tables = np.zeros((len(lens), int(nblk.max())), np.int32)
    at = 0
    for b, n in enumerate(nblk):
        block_tables[b, :n] = perm[at:at + n]
        at += n
    k = lattice((num_blocks, hkv, d // x, bs, x), seed + 2)
    v = lattice((num_blocks, hkv, d, bs), seed + 3)
    q = lattice((len(lens), hq, d), seed + 4)
    slopes = (lattice((hq,), seed + 5) / 16.0).astype(np.float32) if alibi else None
    if dtype == "bf16":
        k, v, q = f32_to_bf16_bits(k), f32_to_bf16_bits(v), f32_to_bf16_bits(q)
    return dict(dtype=dtype, version=version, q=q, k_cache=k, v_cache=v, block_tables=block_tables, seq_lens=lens,
                scale=float(d) ** -0.5, alibi_slopes=slopes, num_kv_heads=hkv)


def cache_case(dtype: str):
    """Inputs of the paged reshape_and_cache / copy_blocks cases (tests/kernels/test_cache.py shapes, smaller)."""
    seed = 77000 + (0 if dtype == "f32" else 1)
    num_tokens, heads, d, bs, num_blocks = 42, 8, HEAD_SIZE, BLOCK_SIZE, 64
    x = 4 if dtype == "f32" else 8
    slots = permutation(bs * num_blocks, seed)[:num_tokens].astype(np.int64)
    slots[5] = -1  # padded token: must be skipped
    qkv = lattice((num_tokens, 3, heads, d), seed + 1)  # key/value are strided views of a fused tensor
    k_cache = lattice((num_blocks, heads, d // x, bs, x), seed + 2)
    v_cache = lattice((num_blocks, heads, d, bs), seed + 3)
    pairs = permutation(num_blocks, seed + 4)
    mapping = np.stack([pairs[:16], pairs[16:32]], axis=1).astype(np.int64)  # disjoint sources and destinations
    if dtype == "bf16":
        qkv, k_cache, v_cache = f32_to_bf16_bits(qkv), f32_to_bf16_bits(k_cache), f32_to_bf16_bits(v_cache)
    return dict(dtype=dtype, qkv=qkv, k_cache=k_cache, v_cache=v_cache, slot_mapping=slots, mapping=mapping)
