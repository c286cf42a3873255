"""Pins for the three oracle entry points that the GPU tests use as their only expectation: the scaled fp8
encode, the fp8 vTensor scatter and swap_blocks.  Each is checked against something that is not the oracle:
torch's float8_e4m3fn cast of an IEEE quotient (a library routine), the address formula of
csrc/cache_kernels.cu:176-199 written out in numpy, and `want[d] = src[s]` on the reference's own block
pairs (tests/worker/test_swap.py:57-89).  The scales are the reference's own per-layer e4m3fn scales
(tests/fp8_kv/llama2-{7b,70b}-fp8-kv/kv_cache_scales.json, committed as data under tests/golden/fp8_kv/)
plus a few of other magnitudes."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_kv")


def reference_scales():
    out = []
    for name in ("llama2-7b_kv_cache_scales.json", "llama2-70b_kv_cache_scales.json"):
        with open(os.path.join(GOLDEN, name)) as f:
            doc = json.load(f)
        assert doc["kv_cache"]["dtype"] == "float8_e4m3fn"
        for layers in doc["kv_cache"]["scaling_factor"].values():
            out += [float(s) for s in layers.values()]
    return out


def torch_codes(x_f32: np.ndarray, scale: float) -> np.ndarray:
    """e4m3fn(x / scale) by the library: IEEE fp32 division (numpy), then torch's cast (round to nearest even).
    Only meaningful where the quotient lies inside the finite range (torch does not saturate)."""
    with np.errstate(over="ignore"):
        quot = (x_f32 / np.float32(scale)).astype(np.float32)
    return torch.from_numpy(quot).to(torch.float8_e4m3fn).view(torch.uint8).numpy(), quot


def exact_ties():
    """Every positive value that lies exactly half-way between two neighbouring e4m3fn values."""
    codes = np.arange(0, 0x7f, dtype=np.uint8)  # 0 .. 448
    vals = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    return ((vals[:-1] + vals[1:]) / 2).astype(np.float32)


SCALES = sorted(set(reference_scales()))
OTHER_SCALES = [6.0 / 448, 0.0123, 0.0171, 1.0, 0.5, 3.0, 1e-3, 1.0 / 3.0]


def test_reference_scale_fixtures_are_what_the_reference_holds():
    s = reference_scales()
    assert len(s) == 32 + 80
    assert min(s) == pytest.approx(0.0152239128947258) and max(s) == pytest.approx(0.0853097140789032)


def test_scaled_encode_of_every_bf16_value_against_torch():
    """fp8_encode(x, s) bit for bit over all 65 536 bf16 inputs, for the reference's 112 scales and eight others.
    A reciprocal multiply in place of the IEEE division, a truncating rounding or a wrong saturation point
    each fail this."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = O.bf16_to_f32(bits)
    finite = np.isfinite(x)
    for s in SCALES + OTHER_SCALES:
        got = O.fp8_encode(bits, s)
        want, quot = torch_codes(x[finite], s)
        inside = np.abs(quot) <= 448
        assert np.array_equal(got[finite][inside], want[inside]), s
        # beyond the finite range: saturate (nvidia/quant_utils.cuh:481-490, SATFINITE), sign kept
        over = ~inside
        assert np.array_equal(got[finite][over], np.where(quot[over] < 0, 0xFE, 0x7E).astype(np.uint8)), s
        assert np.all((got[np.isnan(x)] & 0x7F) == 0x7F)


def test_scaled_encode_of_fp32_values_and_exact_ties_against_torch():
    rng = np.random.default_rng(5)
    ties = exact_ties()
    n_ties = 0
    for s in SCALES[::7] + OTHER_SCALES:
        s32 = np.float32(s)
        x = np.concatenate([
            rng.standard_normal(1 << 18).astype(np.float32) * np.float32(6.0),          # what a KV tensor holds
            (rng.standard_normal(1 << 17).astype(np.float32) * np.float32(200.0) * s32),  # the whole code range
            rng.uniform(-2.0 ** -5, 2.0 ** -5, 1 << 16).astype(np.float32) * s32,         # codes below 2^-6
        ])
        # inputs whose quotient is an exact tie: x = fl(tie * s), kept where fl(x / s) lands on the tie again
        cand = np.concatenate([ties * s32, -ties * s32]).astype(np.float32)
        hit = np.isin(np.abs(cand / s32), ties)
        n_ties += int(hit.sum())
        x = np.concatenate([x, cand[hit]]).astype(np.float32)
        want, quot = torch_codes(x, s)
        inside = np.abs(quot) <= 448
        assert np.array_equal(O.fp8_encode(x, s)[inside], want[inside]), s
    assert n_ties > 500  # the tie cases are really there (a power-of-two scale alone gives 252)


def test_encode_differs_from_a_reciprocal_multiply_somewhere():
    """The test above can tell x / s from x * (1 / s): with the reference's scales the two disagree on some
    inputs, and the oracle sides with the division."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = O.bf16_to_f32(bits)
    x = x[np.isfinite(x)]
    differ = 0
    x = x[np.abs(x) < 1e3]
    for s in SCALES:
        s32 = np.float32(s)
        a = torch.from_numpy((x / s32).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        b = torch.from_numpy((x * (np.float32(1) / s32)).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        ok = np.abs(x / s32) <= 448
        differ += int(np.count_nonzero(a[ok] != b[ok]))
    assert differ > 0


@pytest.mark.parametrize("src", ["bf16", "f32"])
def test_fp8_vtensor_scatter_against_the_address_formula(src):
    """oracle.reshape_and_cache_vtensor_fp8 against numpy: the code of element i of row b goes to byte
    k_ptrs[slot_ids[b]] + slot_m[b] + i (csrc/cache_kernels.cu:176-199 with one byte per element), codes by
    torch's cast of the IEEE quotient; rows with a negative offset are skipped; strided (fused qkv) sources."""
    rng = np.random.default_rng(11)
    hkv, d = 3, 16
    row = hkv * d
    k_scale, v_scale = SCALES[0], SCALES[-1]
    bufs_k = [np.full(64 * row, 0xAB, np.uint8) for _ in range(4)]
    bufs_v = [np.full(64 * row, 0xCD, np.uint8) for _ in range(4)]
    kp = np.array([b.ctypes.data for b in bufs_k], np.int64)
    vp = np.array([b.ctypes.data for b in bufs_v], np.int64)
    batch = 5
    fused = (rng.standard_normal((batch, 3, hkv, d)) * 3).astype(np.float32)
    fused[0, 1, 0, 0] = 1e6     # saturates
    fused[0, 2, 0, 1] = -1e6
    if src == "bf16":
        fused = O.f32_to_bf16(fused)
    key, value = fused[:, 1], fused[:, 2]  # rows 3*row elements apart
    slot_m = np.array([7 * row, -1, 0, 63 * row, 5 * row + 0], np.int64)
    slot_ids = np.array([2, 1, 0, 3, 2], np.int64)
    O.reshape_and_cache_vtensor_fp8(key, value, kp, vp, slot_m, slot_ids, hkv, d, k_scale, v_scale)

    def codes(rows, s):
        xf = O.bf16_to_f32(rows) if src == "bf16" else rows
        c, quot = torch_codes(np.ascontiguousarray(xf, dtype=np.float32), s)
        return np.where(np.abs(quot) > 448, np.where(quot < 0, 0xFE, 0x7E), c).astype(np.uint8)

    want_k = [np.full(64 * row, 0xAB, np.uint8) for _ in range(4)]
    want_v = [np.full(64 * row, 0xCD, np.uint8) for _ in range(4)]
    for b in range(batch):
        if slot_m[b] < 0:
            continue
        want_k[slot_ids[b]][slot_m[b]:slot_m[b] + row] = codes(key[b], k_scale).reshape(-1)
        want_v[slot_ids[b]][slot_m[b]:slot_m[b] + row] = codes(value[b], v_scale).reshape(-1)
    for i in range(4):
        assert np.array_equal(bufs_k[i], want_k[i]) and np.array_equal(bufs_v[i], want_v[i])
    assert np.all(bufs_k[1] == 0xAB) and np.all(bufs_v[1] == 0xCD)  # the skipped row's slot is untouched
    assert bufs_k[2][7 * row] == 0x7E and bufs_v[2][7 * row + 1] == 0xFE


# tests/worker/test_swap.py:57-89: the reference's fixed block pairs, swap-in and swap-out
REFERENCE_PAIRS = [[(3, 72), (56, 35), (84, 34)], [(19, 45), (67, 23), (12, 78), (40, 99), (1, 71)]]


@pytest.mark.parametrize("pairs", REFERENCE_PAIRS)
@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.float32])
def test_swap_blocks_is_want_d_equals_src_s(pairs, dtype):
    """oracle.swap_blocks against numpy fancy indexing (csrc/cache_kernels.cu:24-69: block src -> block dst,
    nothing else touched), on the reference's pairs and on random ones."""
    rng = np.random.default_rng(3)
    shape = (100, 2, 4, 16)
    src = rng.integers(0, 200, shape).astype(dtype)
    dst0 = rng.integers(0, 200, shape).astype(dtype)
    for mapping in (pairs, list(zip(rng.permutation(100)[:17].tolist(), rng.permutation(100)[:17].tolist()))):
        dst = dst0.copy()
        O.swap_blocks(src, dst, np.array(mapping, np.int64))
        want = dst0.copy()
        s, d = zip(*mapping)
        want[list(d)] = src[list(s)]
        assert np.array_equal(dst, want)
        untouched = np.setdiff1d(np.arange(100), d)
        assert np.array_equal(dst[untouched], dst0[untouched])
