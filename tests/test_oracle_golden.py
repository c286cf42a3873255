"""The oracle against the REFERENCE's own CPU kernels: tests/golden/reference_cpu.npz holds what
GLakeServe/csrc/cpu/{attention,cache}.cpp (compiled in place) returned on the deterministic inputs
of tests/golden/gen_inputs.py.  When the compiled reference is present (build container) the same
comparison is also made live on fresh random inputs."""
import hashlib
import os

import numpy as np
import pytest

from golden import gen_inputs as G
from oracle import oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_cpu.npz"))


def sha(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def bf16_steps(a_bits, b_bits):
    def key(bits):
        b = bits.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def run_oracle(c):
    cache = O.PagedCache(c["k_cache"], c["v_cache"], c["block_tables"])
    fn = O.paged_attention_v1 if c["version"] == 1 else O.paged_attention_v2
    # the compiled reference stores bf16 by truncation (gcc 11 cannot build its AVX512-BF16 branch)
    return fn(c["q"], cache, c["scale"], c["seq_lens"], c["alibi_slopes"], bf16_round=False)


def compare(got, want, dtype):
    if dtype == "f32":
        # same arithmetic, different summation trees (AVX-512 lanes vs scalar loops)
        assert np.all(np.abs(got - want) <= 2e-6 + 1e-5 * np.abs(want)), np.abs(got - want).max()
    else:
        steps = bf16_steps(got, want)
        assert steps.max() <= 1, f"max {steps.max()} bf16 steps"
        assert (steps == 0).mean() >= 0.995, f"only {(steps == 0).mean():.4f} bit-equal"


@pytest.mark.parametrize("name", sorted(G.ATTENTION_CASES))
def test_attention_against_reference_fixture(name):
    c = G.attention_case(name)
    compare(run_oracle(c), GOLD["attn_" + name], c["dtype"])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_paged_scatter_against_reference_fixture(dtype):
    c = G.cache_case(dtype)
    kc, vc = c["k_cache"].copy(), c["v_cache"].copy()
    O.reshape_and_cache_paged(c["qkv"][:, 1], c["qkv"][:, 2], kc, vc, c["slot_mapping"])
    assert sha(kc, vc) == str(GOLD["reshape_sha_" + dtype])
    # and the closed form of the reference's own test (tests/kernels/test_cache.py:170-180)
    ek, ev = c["k_cache"].copy(), c["v_cache"].copy()
    bs = ek.shape[3]
    for i, slot in enumerate(c["slot_mapping"]):
        if slot < 0:
            continue
        ek[slot // bs, :, :, slot % bs, :] = c["qkv"][i, 1].reshape(ek[0, :, :, 0, :].shape)
        ev[slot // bs, :, :, slot % bs] = c["qkv"][i, 2]
    assert np.array_equal(kc, ek) and np.array_equal(vc, ev)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_copy_blocks_against_reference_fixture(dtype):
    c = G.cache_case(dtype)
    ks = [c["k_cache"].copy(), c["v_cache"].copy()]
    vs = [c["v_cache"].copy(), c["k_cache"].copy().reshape(c["v_cache"].shape)]
    want_k = [k.copy() for k in ks]
    O.copy_blocks(ks, vs, c["mapping"])
    assert sha(*ks, *vs) == str(GOLD["copy_sha_" + dtype])
    for src, dst in c["mapping"]:
        for k in want_k:
            k[dst] = k[src]
    assert all(np.array_equal(a, b) for a, b in zip(ks, want_k))


@pytest.mark.skipif(not O.ref_available(), reason="compiled reference CPU kernels not present on this machine")
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("version", [1, 2])
def test_live_against_compiled_reference(dtype, version):
    rng = np.random.default_rng(5 + version)
    b, hq, hkv, d, bs = 6, 32, 8, 128, 16
    x = 4 if dtype == "f32" else 8
    lens = np.array([3, 16, 100, 640, 1024, 1500], np.int32)
    nb = 300
    k = rng.standard_normal((nb, hkv, d // x, bs, x)).astype(np.float32)
    v = rng.standard_normal((nb, hkv, d, bs)).astype(np.float32)
    q = rng.standard_normal((b, hq, d)).astype(np.float32)
    bt = rng.integers(0, nb, (b, (lens.max() + bs - 1) // bs)).astype(np.int32)
    if dtype == "bf16":
        k, v, q = O.f32_to_bf16(k), O.f32_to_bf16(v), O.f32_to_bf16(q)
    want = O.ref_paged_attention(version, q, k, v, bt, lens, d ** -0.5)
    c = dict(k_cache=k, v_cache=v, block_tables=bt, version=version, q=q, scale=d ** -0.5, seq_lens=lens,
             alibi_slopes=None)
    compare(run_oracle(c), want, dtype)
