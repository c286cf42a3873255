"""A seeded random sweep of decode and prompt attention against the oracle: head counts (GQA groups 1 to
16, odd head counts), batch sizes, length mixes (all short, mixed, one very long sequence among short
ones), fixed partitions and stream-K spans, ALiBi, fp8, and the three merge modes and tile orders.  Every case
builds its own sequence slots and destroys them again.  Same tolerances as the dedicated tests; with ALiBi the check
on bf16 steps is left out (slopes drawn from N(0,1) times positions in the thousands give biases whose
fp32 rounding alone exceeds a bf16 step of a small output, inside the tolerance on the fp32 values)."""
import numpy as np
import pytest

import test_gpu_attention as A
import test_gpu_attention_fp8 as F
import test_gpu_prefill_attention as P

pytestmark = pytest.mark.gpu

HEADS = [(32, 8), (64, 8), (8, 8), (16, 1), (12, 4), (8, 2), (16, 16), (48, 8), (128, 8), (7, 7), (10, 2)]
# fp8 rows: an even number of kv heads with groups up to 8 takes the kernel variants that stream two kv
# heads per workgroup, everything else (odd counts, one kv head, groups above 8) the one-head variants
HEADS_FP8 = HEADS + [(6, 3), (40, 8), (32, 2), (18, 2), (2, 2), (24, 6), (64, 4)]


@pytest.mark.parametrize("seed", [101, 202, 303])
def test_random_sweep(gpu_pool, seed):
    from glake_amd import _C

    lib = _C.lib()
    rng = np.random.default_rng(seed)
    try:
        for case in range(40):
            hq, hkv = HEADS[rng.integers(len(HEADS))]
            b = int(rng.integers(1, 24))
            kind = rng.integers(4)
            if kind == 0:
                lens = rng.integers(1, 40, b)
            elif kind == 1:
                lens = rng.integers(1, 700, b)
            elif kind == 2:
                lens = rng.integers(1, 3000, max(1, b // 3))
            else:
                lens = np.concatenate([rng.integers(1, 20, b), rng.integers(2000, 6000, 1)])
            lens = [int(x) for x in lens]
            pt = int(rng.choice([0, 0, 0, 64, 128, 256, 512, 1024]))
            alibi = bool(rng.integers(4) == 0)
            merge = int(rng.integers(-1, 2))
            sub = int(rng.integers(1 << 30))
            order = (sub >> 3) % 3 - 1  # tile order: -1 the library's choice, 0 sequence-major, 1 head-major where possible
            _C.check(lib.vtkv_set_fused_merge(merge))
            _C.check(lib.vtkv_set_head_major(order))
            print(f"decode case {case}: seed {sub} heads {hq}/{hkv} lens {lens} partition {pt} alibi {alibi} merge {merge} "
                  f"order {order}", flush=True)
            A.run_case(gpu_pool, sub, lens, hq, hkv, partition_tokens=pt, alibi=alibi, bf16_step_check=not alibi)
            if rng.integers(3) == 0:
                seq = [int(x) for x in rng.integers(1, 600, int(rng.integers(1, 6)))]
                ql = [int(rng.integers(1, s + 1)) if rng.integers(2) else s for s in seq]
                fp8, al = bool(rng.integers(4) == 0), bool(rng.integers(4) == 0)
                print(f"prompt case {case}: seed {sub} heads {hq}/{hkv} queries {ql} rows {seq} fp8 {fp8} alibi {al}", flush=True)
                P.run_case(gpu_pool, sub, ql, seq, hq, hkv, alibi=al, fp8=fp8, tol=3e-2 if fp8 else 2e-3)
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
        _C.check(lib.vtkv_set_head_major(-1))


@pytest.mark.parametrize("seed", [404, 505])
def test_random_sweep_fp8_decode(gpu_pool, seed):
    from glake_amd import _C

    lib = _C.lib()
    rng = np.random.default_rng(seed)
    try:
        for case in range(40):
            hq, hkv = HEADS_FP8[rng.integers(len(HEADS_FP8))]
            b = int(rng.integers(1, 24))
            kind = rng.integers(4)
            if kind == 0:
                lens = rng.integers(1, 40, b)
            elif kind == 1:
                lens = rng.integers(1, 700, b)
            elif kind == 2:
                lens = rng.integers(1, 3000, max(1, b // 3))
            else:
                lens = np.concatenate([rng.integers(1, 20, b), rng.integers(2000, 6000, 1)])
            lens = [int(x) for x in lens]
            pt = int(rng.choice([0, 0, 0, 64, 128, 256, 512, 1024]))
            alibi = bool(rng.integers(4) == 0)
            merge = int(rng.integers(-1, 2))
            sub = int(rng.integers(1 << 30))
            order = (sub >> 3) % 3 - 1
            _C.check(lib.vtkv_set_fused_merge(merge))
            _C.check(lib.vtkv_set_head_major(order))
            print(f"fp8 decode case {case}: seed {sub} heads {hq}/{hkv} lens {lens} partition {pt} alibi {alibi} "
                  f"merge {merge} order {order}", flush=True)
            F.run_case(gpu_pool, sub, lens, hq, hkv, alibi=alibi, partition_tokens=pt)
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
        _C.check(lib.vtkv_set_head_major(-1))


@pytest.mark.parametrize("seed", [606, 707])
def test_random_sweep_over_head_sizes_and_types(gpu_pool, seed):
    """The same sweep over the other head sizes (64, 80, 96, 112, 256, and 128 in fp16), fp16 and bf16, plain and
    fp8 caches, the plain entry point with stream-K or fixed partitions and the split-K interface; for half of
    the cases also the fused append on the same shape (where it exists) and a batch of prompts (some behind cached
    rows) through the prompt kernel of that shape."""
    sweep_head_sizes(gpu_pool, seed, HEADS, 40, always_f16_at_128=True)


# more than 16 query heads per kv head: served in parts of 16, 15 + 11, 10, 9 + 8, 12, 13 + 12, 16 heads
HEADS_MANY = [(64, 1), (48, 1), (71, 1), (40, 2), (17, 1), (96, 4), (100, 4), (128, 2)]


@pytest.mark.parametrize("seed", [808])
def test_random_sweep_with_many_query_heads_per_kv_head(gpu_pool, seed):
    """The sweep over head sizes and types on multi-query shapes (head size 128 in bf16 included)."""
    sweep_head_sizes(gpu_pool, seed, HEADS_MANY, 40, always_f16_at_128=False)


def sweep_head_sizes(gpu_pool, seed, heads, cases, always_f16_at_128):
    import test_gpu_head_sizes as H
    from glake_amd import _C

    lib = _C.lib()
    rng = np.random.default_rng(seed)
    rng_append = np.random.default_rng(seed + 1)  # (its own stream: the cases above it stay what they were)
    try:
        for case in range(cases):
            hq, hkv = heads[rng.integers(len(heads))]
            d = int(rng.choice(H.HEAD_SIZES))
            dtype = "f16" if ((d == 128 and always_f16_at_128) or rng.integers(2)) else "bf16"
            b = int(rng.integers(1, 16))
            kind = rng.integers(3)
            if kind == 0:
                lens = rng.integers(1, 40, b)
            elif kind == 1:
                lens = rng.integers(1, 900, b)
            else:
                lens = np.concatenate([rng.integers(1, 20, b), rng.integers(2000, 5000, 1)])
            lens = [int(x) for x in lens]
            fp8, alibi = bool(rng.integers(3) == 0), bool(rng.integers(4) == 0)
            version = "v2" if rng.integers(4) == 0 else "v1"
            pt = int(rng.choice([0, 0, 64, 256, 512])) if version == "v1" else 0
            merge = int(rng.integers(-1, 2))
            sub = int(rng.integers(1 << 30))
            _C.check(lib.vtkv_set_fused_merge(merge))
            print(f"case {case}: seed {sub} heads {hq}/{hkv} d {d} {dtype} fp8 {fp8} lens {lens} {version} partition {pt} "
                  f"alibi {alibi} merge {merge}", flush=True)
            H.run_case(gpu_pool, sub, lens, hq, hkv, d, dtype, fp8=fp8, alibi=alibi, version=version, partition_tokens=pt)
            # the one-launch decode step on the same shape, where it exists: any cache at head size 128, 16-bit caches
            # elsewhere
            if (d == 128 or not fp8) and rng_append.integers(2) == 0:
                src = "host" if rng_append.integers(2) else "device"
                print(f"append case {case}: lengths from the {src}", flush=True)
                H.run_append_case(gpu_pool, sub, lens, hq, hkv, d, dtype, fp8=fp8, lens_from=src, alibi=alibi,
                                  partition_tokens=pt)
            if rng.integers(2) == 0:
                seq = [int(x) for x in rng.integers(1, 700, int(rng.integers(1, 6)))]
                ql = [int(rng.integers(1, s + 1)) if rng.integers(2) else s for s in seq]
                pf8, pal = bool(rng.integers(3) == 0), bool(rng.integers(3) == 0)
                print(f"prompt case {case}: seed {sub} heads {hq}/{hkv} d {d} {dtype} queries {ql} rows {seq} fp8 {pf8} "
                      f"alibi {pal}", flush=True)
                H.run_prompt_case(gpu_pool, sub, ql, seq, hq, hkv, d, dtype, fp8=pf8, alibi=pal)
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
