"""More than 16 query heads per kv head (multi-query models: 48, 64 or 71 query heads over one kv head; the
reference's kernels take any ratio, csrc/attention/attention_kernels.cu:625, and tests/kernels/
test_prefix_prefill.py:14 runs 64 per kv head).  The MFMA layouts of the kernels hold 16 heads of a group, so a kv
head with more is served as several virtual kv heads over the same rows, the last of which may hold fewer heads
(71 = 4 x 15 + 11).  Every path that indexes query heads is run on such shapes against the oracle: decode (v1,
the split-K interface with its side buffers in tests/test_gpu_reference_configs.py, fixed partitions, both merge
forms, both tile orders, ALiBi, fp16, fp8 rows, other head sizes), the fused append, and prompts."""
import numpy as np
import pytest

import test_gpu_append_attention as A
import test_gpu_attention as D
import test_gpu_head_sizes as H

pytestmark = pytest.mark.gpu

EDGE = [1, 15, 16, 17, 64, 65, 257, 1025, 3000]
# (query heads, kv heads): 64 = 4 x 16, 48 = 3 x 16, 71 = 4 x 15 + 11, 40 over 2 = 2 x 10 each, 17 = 9 + 8, 96 over 4
SHAPES = [(64, 1), (48, 1), (71, 1), (40, 2), (17, 1), (96, 4)]


@pytest.mark.parametrize("hq,hkv", SHAPES)
def test_decode_attention(gpu_pool, hq, hkv):
    D.run_case(gpu_pool, hq, EDGE, hq, hkv)
    D.run_case(gpu_pool, hq + 1, [20000, 3, 700], hq, hkv)                                  # many workgroups per segment
    D.run_case(gpu_pool, hq + 3, [33, 400, 1000], hq, hkv, alibi=True)
    D.run_case(gpu_pool, hq + 2, [700, 64, 1500, 2049], hq, hkv, partition_tokens=128)


@pytest.mark.parametrize("merge,head_major", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_both_merge_forms_and_tile_orders(gpu_pool, merge, head_major):
    from glake_amd import _C

    lib = _C.lib()
    _C.check(lib.vtkv_set_fused_merge(merge))
    _C.check(lib.vtkv_set_head_major(head_major))
    try:
        rng = np.random.default_rng(9)
        D.run_case(gpu_pool, 61, EDGE, 71, 1)
        D.run_case(gpu_pool, 62, [30000, 3, 9000, 700], 64, 2)
        D.run_case(gpu_pool, 63, rng.integers(1, 600, 300).tolist(), 48, 1)       # several segments per workgroup
        A.run_case(gpu_pool, 64, rng.integers(1, 3000, 40).tolist(), 71, 1, lens_from="device")
    finally:
        _C.check(lib.vtkv_set_fused_merge(-1))
        _C.check(lib.vtkv_set_head_major(-1))


@pytest.mark.parametrize("hq,hkv,d,dtype,fp8", [(64, 1, 128, "f16", False), (71, 1, 64, "bf16", False),
                                                (48, 1, 256, "f16", True), (40, 2, 80, "bf16", True),
                                                (71, 1, 128, "bf16", True), (64, 2, 96, "f16", False)])
def test_other_types_and_head_sizes(gpu_pool, hq, hkv, d, dtype, fp8):
    H.run_case(gpu_pool, hq + d, [1, 17, 513, 2500, 64], hq, hkv, d, dtype, fp8=fp8, alibi=(d == 128))
    H.run_case(gpu_pool, hq + d + 1, [513, 2000, 100], hq, hkv, d, dtype, fp8=fp8, version="v2")


@pytest.mark.parametrize("hq,hkv", [(64, 1), (71, 1), (40, 2)])
@pytest.mark.parametrize("fp8", [False, True])
def test_fused_append(gpu_pool, hq, hkv, fp8):
    """Every virtual kv head of a kv head stores the new row: the same bytes at the same place."""
    A.run_case(gpu_pool, hq + 5 * fp8, [1, 2, 16, 17, 18, 1025, 1026, 5000], hq, hkv, lens_from="host", fp8=fp8)
    A.run_case(gpu_pool, hq + 5 * fp8 + 1, [300, 1, 2049, 77], hq, hkv, lens_from="device", fp8=fp8, alibi=True,
               value_skew=256)


@pytest.mark.parametrize("hq,hkv,d,dtype,fp8,alibi", [(64, 1, 128, "bf16", False, False), (71, 1, 128, "bf16", False, True),
                                                      (48, 1, 128, "f16", True, False), (40, 2, 64, "f16", False, False),
                                                      (17, 1, 256, "bf16", True, True), (96, 4, 96, "bf16", False, False)])
def test_prompts(gpu_pool, hq, hkv, d, dtype, fp8, alibi):
    """Plain prompts and prompts behind cached rows; a unit holds 8 tokens of 16 (or 15, 10, 9) heads."""
    H.run_prompt_case(gpu_pool, hq + d, [300, 20, 1, 130], [300, 33, 1, 700], hq, hkv, d, dtype, fp8, alibi)


@pytest.mark.parametrize("hq,hkv,fp8", [(71, 1, False), (48, 2, True)])
def test_through_the_attention_backend(gpu_pool, hq, hkv, fp8):
    """prepare_step + VTensorImpl.forward of a multi-query model: prompts, prompts behind cached rows, mixed
    batches and both decode paths (the fused append and the separate operators)."""
    from test_gpu_backend_modes import BackendSim

    sim = BackendSim(hq=hq, hkv=hkv, fp8=fp8, max_seqs=5, layers=2, seed=hq)
    sim.step(prompt_slots=[3, 0], query_lens=[300, 17])
    sim.step(prompt_slots=[0, 3], query_lens=[40, 129])                       # continue both
    sim.step(prompt_slots=[1], query_lens=[90], decode_slots=[3, 0], fuse=True)
    sim.step(decode_slots=[0, 1, 3], fuse=False)
    sim.step(decode_slots=[3, 1, 0], fuse=True)
    sim.close()
