"""The attention backend driven the way the reference's model code drives it
(llama.py:307-351 -> xformers.py:269-433): per-step bookkeeping, then per layer a cache write and
decode attention, over several steps and layers; checked against the oracle."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fuse", [True, False])
def test_backend_decode_steps_match_oracle(gpu_pool, fuse):
    import torch

    from glake_amd import _C
    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step import prepare_step

    assert VTensorBackend.get_name() == "vtensor-hip"
    layers, hq, hkv, d, max_seqs = 2, 32, 8, 128, 6
    row = hkv * d * 2
    rng = np.random.default_rng(0)
    eng = CacheEngine(layers, hkv, d, torch.bfloat16, max_seqs, 4096)
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    impl.fuse_decode_append = fuse                      # one launch per layer, or cache write + attention
    slots = [4, 1, 5]                                   # three running sequences in slots 4, 1, 5
    lens = [1023, 37, 600]                              # the first crosses a 2 MiB boundary at step 2
    hist_k = {(l, s): [] for l in range(layers) for s in slots}
    hist_v = {(l, s): [] for l in range(layers) for s in slots}
    for s, n in zip(slots, lens):                       # "prefill": rows already in the cache
        seg = eng.vmm_kvcache_segment[s]
        seg.copy_kv_cache(n * row, row)
        for l in range(layers):
            k, v = O.f32_to_bf16(rng.standard_normal((n, hkv, d)).astype(np.float32)), O.f32_to_bf16(
                rng.standard_normal((n, hkv, d)).astype(np.float32))
            _C.check(_C.lib().vtkv_memcpy_h2d(seg.getKeyDevicePtr(l), k.ctypes.data_as(C.c_void_p), k.nbytes))
            _C.check(_C.lib().vtkv_memcpy_h2d(seg.getValueDevicePtr(l), v.ctypes.data_as(C.c_void_p), v.nbytes))
            hist_k[(l, s)].append(k)
            hist_v[(l, s)].append(v)
    dev = torch.device("cuda")
    for step in range(4):
        lens = [n + 1 for n in lens]
        meta = VTensorBackend.make_metadata(
            num_prefills=0, num_prefill_tokens=0, num_decode_tokens=len(slots),
            slot_mapping=torch.tensor(slots, dtype=torch.int64, device=dev), seq_lens=None,
            seq_lens_tensor=torch.tensor(lens, dtype=torch.int32, device=dev), max_query_len=None,
            max_prefill_seq_len=0, max_decode_seq_len=max(lens), query_start_loc=None, seq_start_loc=None,
            context_lens_tensor=None, block_tables=None, is_extend=0, kv_batch_stride=eng.kv_batch_stride,
            kv_num_heads=hkv, kv_head_size=d, max_seq_len=max(lens), slot_mapping_list=slots,
            set_used_size=[0] * len(slots), extend_seq_list=[-1] * len(slots), use_cuda_graph=False)
        meta.k_cache_segment_ptr_list = eng.k_cache_ptr
        meta.v_cache_segment_ptr_list = eng.v_cache_ptr
        meta.kvcache_segment = [eng.vmm_kvcache_segment[s] for s in slots]
        prepare_step(meta, eng.gpu_cache)
        assert meta.slot_m.tolist() == [(n - 1) * row for n in lens]
        for l in range(layers):
            q = O.f32_to_bf16(rng.standard_normal((len(slots), hq * d)).astype(np.float32))
            k = O.f32_to_bf16(rng.standard_normal((len(slots), hkv * d)).astype(np.float32))
            v = O.f32_to_bf16(rng.standard_normal((len(slots), hkv * d)).astype(np.float32))
            for i, s in enumerate(slots):
                hist_k[(l, s)].append(k[i].reshape(1, hkv, d))
                hist_v[(l, s)].append(v[i].reshape(1, hkv, d))
            kc, vc = eng.gpu_cache[l]
            out = impl.forward(torch_bf16_from_bits(q), torch_bf16_from_bits(k), torch_bf16_from_bits(v), kc, vc, meta)
            assert out.shape == (len(slots), hq * d) and out.dtype == torch.bfloat16
            kb = [np.zeros((1, hkv, d), np.uint16)] * max_seqs
            vb = list(kb)
            for s in slots:
                kb[s], vb[s] = np.concatenate(hist_k[(l, s)]), np.concatenate(hist_v[(l, s)])
            want = O.paged_attention_v1(q.reshape(len(slots), hq, d), O.VTensorCache(kb, vb, slots, hkv, d), d ** -0.5, lens)
            got = bits_from_torch_bf16(out).reshape(len(slots), hq, d)
            diff = np.abs(O.bf16_to_f32(got) - O.bf16_to_f32(want))
            # both sides are bf16 tensors: one bf16 step (2^-7 relative) on top of the 2e-3 bound
            assert np.all(diff <= 2e-3 + (2e-3 + 2.0 ** -7) * np.abs(O.bf16_to_f32(want)))
    assert eng.vmm_kvcache_segment[4].actual_size == 2 * (2 << 20)   # crossed into its second chunk
    eng.close()


def test_backend_prompt_run_then_decode(gpu_pool):
    """A prompt run through the backend (cache write + causal attention over the ranges), then decode
    steps that read what the prompt run cached."""
    import torch

    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step import prepare_step

    hq, hkv, d, max_seqs = 32, 8, 128, 4
    row = hkv * d * 2
    rng = np.random.default_rng(3)
    eng = CacheEngine(1, hkv, d, torch.bfloat16, max_seqs, 4096)
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    slots = [2, 0, 3]
    lens = [37, 1000, 5]
    dev = torch.device("cuda")
    n_tok = sum(lens)

    def metadata(prefill: bool, lens):
        starts = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        meta = VTensorBackend.make_metadata(
            num_prefills=len(slots) if prefill else 0, num_prefill_tokens=n_tok if prefill else 0,
            num_decode_tokens=0 if prefill else len(slots),
            slot_mapping=torch.tensor(slots, dtype=torch.int64, device=dev), seq_lens=list(lens) if prefill else None,
            seq_lens_tensor=torch.tensor(lens, dtype=torch.int32, device=dev), max_query_len=max(lens) if prefill else None,
            max_prefill_seq_len=max(lens) if prefill else 0, max_decode_seq_len=0 if prefill else max(lens),
            query_start_loc=torch.tensor(starts, device=dev) if prefill else None, seq_start_loc=None,
            context_lens_tensor=None, block_tables=None, is_extend=0, kv_batch_stride=eng.kv_batch_stride,
            kv_num_heads=hkv, kv_head_size=d, max_seq_len=max(lens), slot_mapping_list=slots,
            set_used_size=[0] * len(slots), extend_seq_list=[-1] * len(slots), use_cuda_graph=False)
        if prefill:  # first source row of each prompt in the packed key/value tensors (model_runner.py:366-370)
            meta.cache_seq_lens = torch.tensor(starts[:-1], dtype=torch.int32, device=dev)
        meta.k_cache_segment_ptr_list = eng.k_cache_ptr
        meta.v_cache_segment_ptr_list = eng.v_cache_ptr
        meta.kvcache_segment = [eng.vmm_kvcache_segment[s] for s in slots]
        prepare_step(meta, eng.gpu_cache)
        return meta

    kc, vc = eng.gpu_cache[0]
    q = O.f32_to_bf16(rng.standard_normal((n_tok, hq * d)).astype(np.float32))
    k = O.f32_to_bf16(rng.standard_normal((n_tok, hkv * d)).astype(np.float32))
    v = O.f32_to_bf16(rng.standard_normal((n_tok, hkv * d)).astype(np.float32))
    meta = metadata(True, lens)
    assert meta.slot_m.tolist() == [0, 0, 0]
    out = impl.forward(torch_bf16_from_bits(q), torch_bf16_from_bits(k), torch_bf16_from_bits(v), kc, vc, meta)
    kb = [np.zeros((1, hkv, d), np.uint16)] * max_seqs
    vb = list(kb)
    row0 = 0
    for s, n in zip(slots, lens):
        kb[s], vb[s] = k[row0:row0 + n].reshape(n, hkv, d), v[row0:row0 + n].reshape(n, hkv, d)
        row0 += n
    want = O.prefill_attention(q.reshape(n_tok, hq, d), O.VTensorCache(kb, vb, slots, hkv, d), d ** -0.5, lens, lens)
    got = bits_from_torch_bf16(out).reshape(n_tok, hq, d)
    diff = np.abs(O.bf16_to_f32(got) - O.bf16_to_f32(want))
    assert np.all(diff <= 2e-3 + (2e-3 + 2.0 ** -7) * np.abs(O.bf16_to_f32(want)))
    for step in range(2):
        lens = [n + 1 for n in lens]
        meta = metadata(False, lens)
        assert meta.slot_m.tolist() == [(n - 1) * row for n in lens]
        q1 = O.f32_to_bf16(rng.standard_normal((len(slots), hq * d)).astype(np.float32))
        k1 = O.f32_to_bf16(rng.standard_normal((len(slots), hkv * d)).astype(np.float32))
        v1 = O.f32_to_bf16(rng.standard_normal((len(slots), hkv * d)).astype(np.float32))
        out = impl.forward(torch_bf16_from_bits(q1), torch_bf16_from_bits(k1), torch_bf16_from_bits(v1), kc, vc, meta)
        for i, s in enumerate(slots):
            kb[s] = np.concatenate([kb[s], k1[i].reshape(1, hkv, d)])
            vb[s] = np.concatenate([vb[s], v1[i].reshape(1, hkv, d)])
        want = O.paged_attention_v1(q1.reshape(len(slots), hq, d), O.VTensorCache(kb, vb, slots, hkv, d), d ** -0.5, lens)
        got = bits_from_torch_bf16(out).reshape(len(slots), hq, d)
        diff = np.abs(O.bf16_to_f32(got) - O.bf16_to_f32(want))
        assert np.all(diff <= 2e-3 + (2e-3 + 2.0 ** -7) * np.abs(O.bf16_to_f32(want)))
    eng.close()
