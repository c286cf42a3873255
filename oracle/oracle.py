"""TEST INFRASTRUCTURE - numpy front end of the CPU oracle (``liboracle.so``) and of the
compiled reference CPU twin (``_ref/libref_cpu.so``).

Only tests, the smoke test and the CPU-baseline leg of the benchmark may import this
module; the product package never does.  bf16 arrays are carried as ``numpy.uint16``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
F32, BF16 = 0, 1
PAGED, VTENSOR = 0, 1
PARTITION_SIZE = 512  # csrc/cpu/attention.cpp:648


class _Cache(C.Structure):
    _fields_ = [
        ("layout", C.c_int), ("dtype", C.c_int),
        ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("block_tables", C.c_void_p), ("max_num_blocks_per_seq", C.c_int), ("block_size", C.c_int),
        ("kv_block_stride", C.c_int64), ("kv_head_stride", C.c_int64),
        ("k_ptrs", C.c_void_p), ("v_ptrs", C.c_void_p), ("slot_mapping", C.c_void_p),
        ("num_kv_heads", C.c_int), ("head_size", C.c_int),
    ]


def build(force: bool = False) -> None:
    """Compile liboracle.so (and _ref/ when the reference tree is present)."""
    if force or not os.path.exists(os.path.join(_HERE, "liboracle.so")):
        subprocess.check_call(["make", "-C", _HERE, "liboracle.so"])


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(os.path.join(_HERE, "liboracle.so"))
        _lib.oracle_fp8_e4m3fn_decode.restype = C.c_float
        _lib.oracle_fp8_e4m3fn_decode.argtypes = [C.c_uint8]
        _lib.oracle_fp8_e4m3fn_encode.restype = C.c_uint8
        _lib.oracle_fp8_e4m3fn_encode.argtypes = [C.c_float]
    return _lib


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _dt(a: np.ndarray) -> int:
    if a.dtype == np.float32:
        return F32
    if a.dtype == np.uint16:
        return BF16
    raise TypeError(f"oracle carries fp32 as float32 and bf16 as uint16, got {a.dtype}")


# ----------------------------------------------------------------------------- bf16 helpers
def f32_to_bf16(a: np.ndarray, round_nearest: bool = True) -> np.ndarray:
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    if not round_nearest:
        return (u >> 16).astype(np.uint16)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def bf16_to_f32(a: np.ndarray) -> np.ndarray:
    return (a.astype(np.uint32) << 16).view(np.float32)


# ----------------------------------------------------------------------------- cache descriptors
class PagedCache:
    """K [nb,Hkv,D/x,bs,x], V [nb,Hkv,D,bs] + int32 block tables (paged_attn.py:47-59)."""

    def __init__(self, k_cache: np.ndarray, v_cache: np.ndarray, block_tables: np.ndarray):
        assert k_cache.flags.c_contiguous and v_cache.flags.c_contiguous
        self.k, self.v = k_cache, v_cache
        self.bt = np.ascontiguousarray(block_tables, dtype=np.int32)
        nb, hkv, dx, bs, x = k_cache.shape
        self.c = _Cache(PAGED, _dt(k_cache), _p(k_cache), _p(v_cache), _p(self.bt), self.bt.shape[1], bs,
                        hkv * dx * bs * x, dx * bs * x, None, None, None, hkv, dx * x)


class VTensorCache:
    """Per-slot contiguous [T,Hkv,D] ranges addressed through base-pointer tables."""

    def __init__(self, k_bufs: Sequence[np.ndarray], v_bufs: Sequence[np.ndarray], slot_mapping, num_kv_heads: int,
                 head_size: int):
        self.k_bufs, self.v_bufs = list(k_bufs), list(v_bufs)
        self.k_ptrs = np.array([b.ctypes.data for b in self.k_bufs], dtype=np.int64)
        self.v_ptrs = np.array([b.ctypes.data for b in self.v_bufs], dtype=np.int64)
        self.slots = np.ascontiguousarray(slot_mapping, dtype=np.int64)
        self.c = _Cache(VTENSOR, _dt(self.k_bufs[0]), None, None, None, 0, 1, 0, 0, _p(self.k_ptrs), _p(self.v_ptrs),
                        _p(self.slots), num_kv_heads, head_size)


# ----------------------------------------------------------------------------- attention
def paged_attention_v1(q: np.ndarray, cache, scale: float, seq_lens, alibi_slopes=None, bf16_round: bool = True):
    q = np.ascontiguousarray(q)
    num_seqs, num_heads, d = q.shape
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    al = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, dtype=np.float32)
    out = np.zeros_like(q)
    rc = lib().oracle_paged_attention_v1(_p(out), _p(q), _dt(q), C.c_int64(num_heads * d), C.byref(cache.c),
                                         C.c_float(scale), _p(sl), num_seqs, num_heads, _p(al), int(bf16_round))
    assert rc == 0
    return out


def paged_attention_v2(q: np.ndarray, cache, scale: float, seq_lens, alibi_slopes=None, bf16_round: bool = True,
                       return_partials: bool = False):
    q = np.ascontiguousarray(q)
    num_seqs, num_heads, d = q.shape
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    al = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, dtype=np.float32)
    npart = max(1, (int(sl.max()) + PARTITION_SIZE - 1) // PARTITION_SIZE)
    out = np.zeros_like(q)
    exp_sums = np.zeros((num_seqs, num_heads, npart), np.float32)
    max_logits = np.zeros_like(exp_sums)
    tmp_out = np.zeros((num_seqs, num_heads, npart, d), q.dtype)
    rc = lib().oracle_paged_attention_v2(_p(out), _p(exp_sums), _p(max_logits), _p(tmp_out), _p(q), _dt(q),
                                         C.c_int64(num_heads * d), C.byref(cache.c), C.c_float(scale), _p(sl),
                                         num_seqs, num_heads, npart, _p(al), int(bf16_round))
    assert rc == 0
    return (out, exp_sums, max_logits, tmp_out) if return_partials else out


# ----------------------------------------------------------------------------- cache ops
def reshape_and_cache_paged(key, value, k_cache, v_cache, slot_mapping, key_stride=None, value_stride=None):
    num_tokens, hkv, d = key.shape
    nb, _, dx, bs, x = k_cache.shape
    sm = np.ascontiguousarray(slot_mapping, dtype=np.int64)
    ks = key.strides[0] // key.itemsize if key_stride is None else key_stride
    vs = value.strides[0] // value.itemsize if value_stride is None else value_stride
    rc = lib().oracle_reshape_and_cache_paged(C.c_void_p(key.ctypes.data), C.c_void_p(value.ctypes.data),
                                              _p(k_cache), _p(v_cache), _p(sm), num_tokens, C.c_int64(ks),
                                              C.c_int64(vs), hkv, d, bs, x, key.itemsize)
    assert rc == 0


def reshape_and_cache_vtensor(key, value, k_ptrs, v_ptrs, slot_m, slot_ids, seq_lens, cache_seq_lens, max_seq_len,
                              num_heads, head_size):
    """Host-memory restatement of the vTensor scatter; *_ptrs hold host addresses."""
    slot_m = np.ascontiguousarray(slot_m, dtype=np.int64)
    slot_ids = np.ascontiguousarray(slot_ids, dtype=np.int64)
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    cs = np.ascontiguousarray(cache_seq_lens, dtype=np.int32)
    rc = lib().oracle_reshape_and_cache_vtensor(
        C.c_void_p(key.ctypes.data), C.c_void_p(value.ctypes.data), _p(k_ptrs), _p(v_ptrs), _p(slot_m), _p(slot_ids),
        _p(sl), _p(cs), len(slot_m), int(max_seq_len), num_heads, head_size,
        C.c_int64(key.strides[0] // key.itemsize), C.c_int64(value.strides[0] // value.itemsize), key.itemsize)
    assert rc == 0


def reshape_and_cache_vtensor_fp8(key, value, k_ptrs, v_ptrs, slot_m, slot_ids, num_heads, head_size, k_scale,
                                  v_scale):
    slot_m = np.ascontiguousarray(slot_m, dtype=np.int64)
    slot_ids = np.ascontiguousarray(slot_ids, dtype=np.int64)
    rc = lib().oracle_reshape_and_cache_vtensor_fp8(
        C.c_void_p(key.ctypes.data), C.c_void_p(value.ctypes.data), _dt(key), _p(k_ptrs), _p(v_ptrs), _p(slot_m),
        _p(slot_ids), len(slot_m), num_heads, head_size, C.c_int64(key.strides[0] // key.itemsize),
        C.c_int64(value.strides[0] // value.itemsize), C.c_float(k_scale), C.c_float(v_scale))
    assert rc == 0


def copy_blocks(key_caches, value_caches, mapping):
    m = np.ascontiguousarray(mapping, dtype=np.int64).reshape(-1, 2)
    n = len(key_caches)
    kp = (C.c_void_p * n)(*[k.ctypes.data for k in key_caches])
    vp = (C.c_void_p * n)(*[v.ctypes.data for v in value_caches])
    block_bytes = key_caches[0][0].nbytes
    assert lib().oracle_copy_blocks(kp, vp, n, _p(m), len(m), C.c_int64(block_bytes)) == 0


def swap_blocks(src, dst, mapping):
    m = np.ascontiguousarray(mapping, dtype=np.int64).reshape(-1, 2)
    assert lib().oracle_swap_blocks(_p(src), _p(dst), _p(m), len(m), C.c_int64(src[0].nbytes)) == 0


# ----------------------------------------------------------------------------- fp8 e4m3fn
def fp8_encode(x: np.ndarray, scale: float = 1.0) -> np.ndarray:
    """code = e4m3fn(x / scale), RNE, saturating; x is float32 or bf16-as-uint16."""
    x = np.ascontiguousarray(x)
    out = np.empty(x.shape, np.uint8)
    assert lib().oracle_convert_to_fp8(_p(out), _p(x), _dt(x), C.c_int64(x.size), C.c_float(scale)) == 0
    return out


def fp8_decode(codes: np.ndarray, scale: float = 1.0, to_bf16: bool = False) -> np.ndarray:
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, np.uint16 if to_bf16 else np.float32)
    assert lib().oracle_convert_from_fp8(_p(out), _p(codes), BF16 if to_bf16 else F32, C.c_int64(codes.size),
                                         C.c_float(scale)) == 0
    return out


# ----------------------------------------------------------------------------- compiled reference CPU twin
_ref = None


def ref_available() -> bool:
    path = os.path.join(_HERE, "_ref", "libref_cpu.so")
    if not os.path.exists(path):
        return False
    try:
        with open("/proc/cpuinfo") as f:
            flags = f.read()
    except OSError:
        return False
    return all(f in flags for f in ("avx512f", "avx512bw", "avx512vl", "avx512dq"))


def ref():
    """The reference's csrc/cpu kernels compiled in place (needs torch's shared libraries)."""
    global _ref
    if _ref is None:
        import torch  # noqa: F401  (loads libtorch so the reference object resolves its symbols)
        _ref = C.CDLL(os.path.join(_HERE, "_ref", "libref_cpu.so"))
    return _ref


def ref_paged_attention(version: int, q, k_cache, v_cache, block_tables, seq_lens, scale, alibi_slopes=None):
    q = np.ascontiguousarray(q)
    num_seqs, num_heads, d = q.shape
    nb, hkv, dx, bs, x = k_cache.shape
    bt = np.ascontiguousarray(block_tables, dtype=np.int32)
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    al = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, dtype=np.float32)
    max_len = int(sl.max())
    npart = max(1, (max_len + PARTITION_SIZE - 1) // PARTITION_SIZE)
    out = np.zeros_like(q)
    es = np.zeros((num_seqs, num_heads, npart), np.float32)
    ml = np.zeros_like(es)
    to = np.zeros((num_seqs, num_heads, npart, d), q.dtype)
    rc = ref().ref_paged_attention(version, _p(out), _p(q), _p(k_cache), _p(v_cache), _dt(q), num_seqs, num_heads, hkv,
                                   d, nb, bs, C.c_float(scale), _p(bt), bt.shape[1], _p(sl), max_len, _p(al), _p(es),
                                   _p(ml), _p(to), npart)
    assert rc == 0
    return out


def ref_reshape_and_cache(key, value, k_cache, v_cache, slot_mapping):
    num_tokens, hkv, d = key.shape
    nb, _, dx, bs, x = k_cache.shape
    sm = np.ascontiguousarray(slot_mapping, dtype=np.int64)
    rc = ref().ref_reshape_and_cache(C.c_void_p(key.ctypes.data), C.c_void_p(value.ctypes.data), _p(k_cache),
                                     _p(v_cache), _dt(k_cache), num_tokens, hkv, d,
                                     C.c_long(key.strides[0] // key.itemsize),
                                     C.c_long(value.strides[0] // value.itemsize), nb, bs, _p(sm))
    assert rc == 0


def ref_copy_blocks(key_caches, value_caches, mapping):
    m = np.ascontiguousarray(mapping, dtype=np.int64).reshape(-1, 2)
    n = len(key_caches)
    kp = (C.c_void_p * n)(*[k.ctypes.data for k in key_caches])
    vp = (C.c_void_p * n)(*[v.ctypes.data for v in value_caches])
    nb = key_caches[0].shape[0]
    rc = ref().ref_copy_blocks(kp, vp, n, _dt(key_caches[0]), nb, C.c_long(key_caches[0][0].size), _p(m), len(m))
    assert rc == 0


# ----------------------------------------------------------------------------- textbook (float64) reference
def textbook_attention(q_f, k_rows, v_rows, scale, alibi_slope=None):
    """softmax(scale * q.K^T [+ alibi]) V in float64 for one head.
    q_f [D], k_rows/v_rows [T,D] (tests/kernels/test_attention.py:43-55,97-108)."""
    q_f = q_f.astype(np.float64)
    s = scale * (k_rows.astype(np.float64) @ q_f)
    if alibi_slope is not None:
        t = k_rows.shape[0]
        s = s + alibi_slope * (np.arange(t) - t + 1)
    s -= s.max()
    p = np.exp(s)
    p /= p.sum()
    return p @ v_rows.astype(np.float64)


def prefill_attention(q: np.ndarray, cache: "VTensorCache", scale: float, query_lens, seq_lens, alibi_slopes=None,
                      bf16_round: bool = True):
    """Causal attention of packed prompt tokens over the contiguous cache, which already holds their
    rows: the token at position t of its sequence attends to rows 0..t.  This is what both prompt-run
    branches of the reference backend compute (vllm/attention/backends/xformers.py:331-386; mask
    convention of tests/kernels/test_prefix_prefill.py:182-192, BlockDiagonalCausalFromBottomRightMask: the
    queries are the last query_len
    positions of the sequence).  Restated through the pinned decode oracle: one query token at position
    t is a decode step over a context of t + 1 rows.
    q [sum(query_lens), Hq, D]; returns the same shape."""
    slots, lens = [], []
    for b, (ql, sl) in enumerate(zip(query_lens, seq_lens)):
        for i in range(ql):
            slots.append(cache.slots[b])
            lens.append(sl - ql + i + 1)
    per_token = VTensorCache(cache.k_bufs, cache.v_bufs, np.array(slots, np.int64), cache.c.num_kv_heads,
                             cache.c.head_size)
    return paged_attention_v1(q, per_token, scale, np.array(lens, np.int32), alibi_slopes, bf16_round)


def textbook_causal_attention(q_f, k_rows, v_rows, scale, context_len: int, alibi_slope=None):
    """Whole-matrix form in float64 for one head of one sequence: q_f [Q, D] are the queries at
    positions context_len .. context_len+Q-1, k_rows / v_rows [context_len+Q, D]; lower-right aligned
    causal mask, optional ALiBi bias slope * (key position - query position)."""
    q64, k64, v64 = (x.astype(np.float64) for x in (q_f, k_rows, v_rows))
    nq, nk = q64.shape[0], k64.shape[0]
    assert nk == context_len + nq
    s = scale * (q64 @ k64.T)
    qpos = context_len + np.arange(nq)[:, None]
    kpos = np.arange(nk)[None, :]
    if alibi_slope is not None:
        s = s + alibi_slope * (kpos - qpos)
    s = np.where(kpos <= qpos, s, -np.inf)
    s -= s.max(axis=1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=1, keepdims=True)
    return p @ v64
