"""Writes tests/golden/reference_cpu.npz: outputs of the REFERENCE's own CPU kernels
(GLakeServe/csrc/cpu/attention.cpp, cache.cpp, compiled in place into oracle/_ref by
`make -C oracle ref`) on the deterministic inputs of gen_inputs.py.

Run in the build container, where /root/reference exists:  python tests/golden/make_golden.py
Attention outputs are stored whole; the bit-exact cache ops are stored as SHA-256 of the
resulting cache bytes.
"""
from __future__ import annotations

import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

import gen_inputs as G  # noqa: E402
from oracle import oracle as O  # noqa: E402


def sha(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def main() -> None:
    assert O.ref_available(), "build the reference CPU kernels first: make -C oracle ref"
    out = {}
    for name in G.ATTENTION_CASES:
        c = G.attention_case(name)
        out["attn_" + name] = O.ref_paged_attention(c["version"], c["q"], c["k_cache"], c["v_cache"],
                                                    c["block_tables"], c["seq_lens"], c["scale"], c["alibi_slopes"])
    for dtype in ("f32", "bf16"):
        c = G.cache_case(dtype)
        key, value = c["qkv"][:, 1], c["qkv"][:, 2]
        kc, vc = c["k_cache"].copy(), c["v_cache"].copy()
        O.ref_reshape_and_cache(key, value, kc, vc, c["slot_mapping"])
        out["reshape_sha_" + dtype] = np.array(sha(kc, vc))
        kc2, vc2 = [c["k_cache"].copy(), c["v_cache"].copy()], [c["v_cache"].copy(), c["k_cache"].copy().reshape(c["v_cache"].shape)]
        O.ref_copy_blocks(kc2, vc2, c["mapping"])
        out["copy_sha_" + dtype] = np.array(sha(*kc2, *vc2))
    path = os.path.join(HERE, "reference_cpu.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "entries")


if __name__ == "__main__":
    main()
