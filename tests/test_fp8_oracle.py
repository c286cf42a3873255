"""fp8 e4m3fn: the oracle's encode/decode against a library routine (torch's float8_e4m3fn
casts, OCP format), exhaustively where the domain is small enough."""
import numpy as np
import pytest
import torch

from oracle import oracle as O


def test_decode_all_256_codes_against_torch():
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = O.fp8_decode(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))


def test_encode_every_bf16_value_against_torch():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = O.bf16_to_f32(bits)
    got = O.fp8_encode(bits)
    finite = np.isfinite(x)
    inside = finite & (np.abs(x) <= 448)
    want = torch.from_numpy(x[inside]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got[inside], want)
    # outside the finite range the reference saturates (nvidia/quant_utils.cuh:481-490, SATFINITE)
    over = (np.abs(x) > 448) & ~np.isnan(x)
    assert np.array_equal(got[over], np.where(x[over] < 0, 0xFE, 0x7E).astype(np.uint8))
    assert np.all((got[np.isnan(x)] & 0x7F) == 0x7F)


def test_encode_random_fp32_and_ties_against_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(1 << 20).astype(np.float32) * 40,
        rng.uniform(-2.0 ** -5, 2.0 ** -5, 1 << 18).astype(np.float32),   # subnormal range of e4m3
        (np.float32(2.0) ** rng.integers(-12, 9, 1 << 16) * rng.choice(np.arange(16, 33) / 16.0, 1 << 16)).astype(np.float32),  # exact ties
    ])
    x = x[np.abs(x) <= 448].astype(np.float32)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(O.fp8_encode(x), want)


def test_scaled_round_trip_like_the_reference_test():
    # tests/kernels/test_cache.py:347-380: uniform(-224, 224), atol 1e-3, rtol 0.1
    rng = np.random.default_rng(1)
    x = rng.uniform(-224, 224, 100000).astype(np.float32)
    back = O.fp8_decode(O.fp8_encode(x))
    assert np.all(np.abs(back - x) <= 1e-3 + 0.1 * np.abs(x))
    scale = np.abs(x).max() / 448
    back = O.fp8_decode(O.fp8_encode(x, scale), scale)
    assert np.all(np.abs(back - x) <= 1e-3 + 0.0625 * np.abs(x) + scale * 2.0 ** -9)
