"""The attention backend in the batch shapes the reference engine feeds it (xformers.py:269-433): the profiling
run without a KV cache (worker.py:157, model_runner.py:846), prompts behind cached rows, batches that mix prompt
and decode tokens, and an fp8 cache through ``prepare_step`` + ``forward``.  A host mirror of every slot's rows
(in the cache's own format) is kept beside the GPU; after every call the cache bytes must equal the mirror bit
for bit and the outputs must match the oracle run on the mirror (bf16: 2e-3 + one bf16 step; fp8: the
reference's protocol, tests/kernels/test_attention.py:233-252,271-274, of dequantising to bf16 first, 3e-2)."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


class BackendSim:
    """Drives VTensorImpl.forward the way the model code does and mirrors the cache on the host."""

    def __init__(self, hq=32, hkv=8, d=128, max_seqs=6, fp8=False, layers=1, max_tokens=4096, seed=0):
        import torch

        from glake_amd.attention.backends.vtensor import VTensorBackend
        from glake_amd.worker.cache_engine import CacheEngine

        self.torch = torch
        self.hq, self.hkv, self.d, self.fp8, self.layers, self.max_seqs = hq, hkv, d, fp8, layers, max_seqs
        self.rng = np.random.default_rng(seed)
        self.eng = CacheEngine(layers, hkv, d, torch.uint8 if fp8 else torch.bfloat16, max_seqs, max_tokens)
        self.k_scale, self.v_scale = (0.011, 0.017) if fp8 else (1.0, 1.0)
        self.impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "fp8" if fp8 else "auto")
        self.backend = VTensorBackend
        self.row = hkv * d * (1 if fp8 else 2)
        self.cdtype = np.uint8 if fp8 else np.uint16
        self.mirror_k = {(l, s): np.zeros((0, hkv, d), self.cdtype) for l in range(layers) for s in range(max_seqs)}
        self.mirror_v = {(l, s): np.zeros((0, hkv, d), self.cdtype) for l in range(layers) for s in range(max_seqs)}
        self.dev = torch.device("cuda")

    def rows_in_cache(self, slot):
        return self.mirror_k[(0, slot)].shape[0]

    def _encode(self, x_bits, scale):
        """What the cache holds for bf16 input rows."""
        if not self.fp8:
            return x_bits
        return O.fp8_encode(O.bf16_to_f32(x_bits), scale)

    def metadata(self, prompt_slots, query_lens, decode_slots, with_query_lens):
        torch, eng = self.torch, self.eng
        slots = list(prompt_slots) + list(decode_slots)
        n_pre = len(prompt_slots)
        seq_lens = [self.rows_in_cache(s) + q for s, q in zip(prompt_slots, query_lens)] + \
                   [self.rows_in_cache(s) + 1 for s in decode_slots]
        cached = [self.rows_in_cache(s) for s in slots]
        n_ptok = int(sum(query_lens))
        meta = self.backend.make_metadata(
            num_prefills=n_pre, num_prefill_tokens=n_ptok, num_decode_tokens=len(decode_slots),
            slot_mapping=torch.tensor(slots, dtype=torch.int64, device=self.dev), seq_lens=list(seq_lens),
            seq_lens_tensor=torch.tensor(seq_lens, dtype=torch.int32, device=self.dev),
            max_query_len=max(query_lens) if n_pre else None,
            max_prefill_seq_len=max(seq_lens[:n_pre]) if n_pre else 0,
            max_decode_seq_len=max(seq_lens[n_pre:]) if decode_slots else 0, query_start_loc=None, seq_start_loc=None,
            context_lens_tensor=None, block_tables=None, is_extend=0, kv_batch_stride=eng.kv_batch_stride,
            kv_num_heads=self.hkv, kv_head_size=self.d, max_seq_len=max(seq_lens), slot_mapping_list=slots,
            set_used_size=cached if with_query_lens else [0] * len(slots), extend_seq_list=[-1] * len(slots),
            use_cuda_graph=False)
        if with_query_lens:
            meta.query_lens = list(query_lens)
        meta.k_cache_segment_ptr_list = eng.k_cache_ptr
        meta.v_cache_segment_ptr_list = eng.v_cache_ptr
        meta.kvcache_segment = [eng.vmm_kvcache_segment[s] for s in slots]
        return meta, slots, seq_lens

    def step(self, prompt_slots=(), query_lens=(), decode_slots=(), with_query_lens=None, fuse=True):
        """One model step: prologue, then every layer's forward; checks cache bytes and outputs."""
        from glake_amd.worker.step import prepare_step

        if with_query_lens is None:
            with_query_lens = any(self.rows_in_cache(s) for s in prompt_slots)
        meta, slots, seq_lens = self.metadata(prompt_slots, query_lens, decode_slots, with_query_lens)
        before = [self.rows_in_cache(s) for s in slots]
        prepare_step(meta, self.eng.gpu_cache)
        assert meta.slot_m.tolist() == [n * self.row for n in before]
        self.impl.fuse_decode_append = fuse
        n_tok = int(sum(query_lens)) + len(decode_slots)
        rows_new = list(query_lens) + [1] * len(decode_slots)
        hq, hkv, d = self.hq, self.hkv, self.d
        for l in range(self.layers):
            q = O.f32_to_bf16(self.rng.standard_normal((n_tok, hq * d)).astype(np.float32))
            k = O.f32_to_bf16(self.rng.standard_normal((n_tok, hkv * d)).astype(np.float32))
            v = O.f32_to_bf16(self.rng.standard_normal((n_tok, hkv * d)).astype(np.float32))
            at = 0
            for s, n in zip(slots, rows_new):
                kk = self._encode(k[at:at + n].reshape(n, hkv, d), self.k_scale)
                vv = self._encode(v[at:at + n].reshape(n, hkv, d), self.v_scale)
                self.mirror_k[(l, s)] = np.concatenate([self.mirror_k[(l, s)], kk])
                self.mirror_v[(l, s)] = np.concatenate([self.mirror_v[(l, s)], vv])
                at += n
            kc, vc = self.eng.gpu_cache[l]
            out = self.impl.forward(torch_bf16_from_bits(q), torch_bf16_from_bits(k), torch_bf16_from_bits(v), kc, vc,
                                    meta, self.k_scale, self.v_scale)
            self.torch.cuda.synchronize()
            assert out.shape == (n_tok, hq * d) and out.dtype == self.torch.bfloat16
            self.check_cache(l, slots)
            self.check_output(l, q.reshape(n_tok, hq, d), bits_from_torch_bf16(out).reshape(n_tok, hq, d),
                              list(prompt_slots), list(query_lens), list(decode_slots), seq_lens)
        return meta

    def check_cache(self, layer, slots):
        from glake_amd import _C

        for s in slots:
            seg = self.eng.vmm_kvcache_segment[s]
            for mirror, ptr in ((self.mirror_k, seg.getKeyDevicePtr(layer)), (self.mirror_v, seg.getValueDevicePtr(layer))):
                want = mirror[(layer, s)]
                got = np.empty_like(want)
                _C.check(_C.lib().vtkv_memcpy_d2h(got.ctypes.data_as(C.c_void_p), ptr, want.nbytes))
                assert np.array_equal(got, want), f"cache bytes of slot {s}, layer {layer} differ from the mirror"
            assert seg.used_size == self.mirror_k[(layer, s)].shape[0] * self.row

    def oracle_cache(self, layer, slots):
        empty = np.zeros((1, self.hkv, self.d), np.uint16)
        kb, vb = [empty] * self.max_seqs, [empty] * self.max_seqs
        for s in range(self.max_seqs):
            k, v = self.mirror_k[(layer, s)], self.mirror_v[(layer, s)]
            if k.shape[0] == 0:
                continue
            if self.fp8:  # the reference's test protocol: back to the model dtype with the scale applied
                k, v = O.fp8_decode(k, self.k_scale, to_bf16=True), O.fp8_decode(v, self.v_scale, to_bf16=True)
            kb[s], vb[s] = k, v
        return kb, vb

    def check_output(self, layer, q, got, prompt_slots, query_lens, decode_slots, seq_lens):
        kb, vb = self.oracle_cache(layer, prompt_slots + decode_slots)
        n_ptok, n_pre = int(sum(query_lens)), len(prompt_slots)
        scale = self.d ** -0.5
        tol = 3e-2 if self.fp8 else 2e-3
        parts = []
        if n_pre:
            parts.append(O.prefill_attention(q[:n_ptok], O.VTensorCache(kb, vb, prompt_slots, self.hkv, self.d), scale,
                                             query_lens, seq_lens[:n_pre]))
        if decode_slots:
            parts.append(O.paged_attention_v1(q[n_ptok:], O.VTensorCache(kb, vb, decode_slots, self.hkv, self.d), scale,
                                              seq_lens[n_pre:]))
        want = O.bf16_to_f32(np.concatenate(parts))
        diff = np.abs(O.bf16_to_f32(got) - want)
        # both sides are bf16 tensors: one bf16 step (2^-7 relative) on top of the bound
        assert np.all(diff <= tol + (tol + 2.0 ** -7) * np.abs(want)), f"max err {diff.max():.3e}"

    def close(self):
        self.eng.close()


def test_profiling_run_without_a_kv_cache(gpu_pool):
    """kv_caches = [None] * layers: prepare_step does nothing, forward attends over the key/value tensors
    themselves (xformers.py:336-343) and caches nothing.  Checked against the prompt oracle on the same rows, with
    key/value as strided slices of a fused qkv tensor as the model hands them over (llama.py:172-174)."""
    import torch

    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.worker.step import prepare_step

    hq, hkv, d = 32, 8, 128
    rng = np.random.default_rng(11)
    lens = [700, 1, 33, 256]
    n_tok = sum(lens)
    qkv = O.f32_to_bf16(rng.standard_normal((n_tok, (hq + 2 * hkv) * d)).astype(np.float32))
    qkv_t = torch_bf16_from_bits(qkv)
    q_t, k_t, v_t = qkv_t.split([hq * d, hkv * d, hkv * d], dim=-1)
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    dev = torch.device("cuda")
    free0 = gpu_pool.showFreeBlocks()
    meta = VTensorBackend.make_metadata(
        num_prefills=len(lens), num_prefill_tokens=n_tok, num_decode_tokens=0,
        slot_mapping=torch.zeros(len(lens), dtype=torch.int64, device=dev), seq_lens=lens,
        seq_lens_tensor=torch.tensor(lens, dtype=torch.int32, device=dev), max_query_len=max(lens),
        max_prefill_seq_len=max(lens), max_decode_seq_len=0, query_start_loc=None, seq_start_loc=None,
        context_lens_tensor=None, block_tables=None, is_extend=0, kv_batch_stride=None, kv_num_heads=None,
        kv_head_size=None, max_seq_len=max(lens), slot_mapping_list=[0] * len(lens), set_used_size=[0] * len(lens),
        extend_seq_list=[], use_cuda_graph=False)
    prepare_step(meta, [None])                      # model_runner.py:846
    out = impl.forward(q_t, k_t, v_t, None, None, meta)
    torch.cuda.synchronize()
    assert out.shape == (n_tok, hq * d) and gpu_pool.showFreeBlocks() == free0
    k = qkv[:, hq * d:(hq + hkv) * d].reshape(n_tok, hkv, d)
    v = qkv[:, (hq + hkv) * d:].reshape(n_tok, hkv, d)
    starts = np.concatenate([[0], np.cumsum(lens)])
    kb = [np.ascontiguousarray(k[starts[i]:starts[i + 1]]) for i in range(len(lens))]
    vb = [np.ascontiguousarray(v[starts[i]:starts[i + 1]]) for i in range(len(lens))]
    want = O.prefill_attention(np.ascontiguousarray(qkv[:, :hq * d]).reshape(n_tok, hq, d),
                               O.VTensorCache(kb, vb, np.arange(len(lens)), hkv, d), d ** -0.5, lens, lens)
    got = bits_from_torch_bf16(out).reshape(n_tok, hq, d)
    diff = np.abs(O.bf16_to_f32(got) - O.bf16_to_f32(want))
    assert np.all(diff <= 2e-3 + (2e-3 + 2.0 ** -7) * np.abs(O.bf16_to_f32(want)))
    with pytest.raises(ValueError):                 # a decode token cannot do without a cache
        meta.num_decode_tokens, meta.num_prefill_tokens = 1, n_tok - 1
        impl.forward(q_t, k_t, v_t, None, None, meta)


@pytest.mark.parametrize("fp8", [False, True])
def test_prompts_behind_cached_rows_in_one_batch(gpu_pool, fp8):
    """Several prompts in one batch, each continuing behind rows its slot already holds (a chunked prompt,
    a reused prefix): forward must scatter query_len rows per prompt, not seq_len, and advance used by them."""
    sim = BackendSim(fp8=fp8, max_seqs=5, seed=21)
    sim.step(prompt_slots=[3, 0, 4], query_lens=[300, 17, 1])                 # plain prompts
    sim.step(prompt_slots=[0, 4, 3], query_lens=[40, 200, 129])               # continue all three, other order
    sim.step(prompt_slots=[1, 3], query_lens=[5, 1], with_query_lens=True)    # a fresh prompt beside a continued one
    sim.step(decode_slots=[3, 1, 0, 4])
    assert sim.rows_in_cache(3) == 300 + 129 + 1 + 1
    sim.close()


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("fuse", [True, False])
def test_prompt_and_decode_tokens_in_one_batch(gpu_pool, fp8, fuse):
    """xformers.py:314-433 serves prompt tokens and decode tokens of one batch in one call."""
    sim = BackendSim(fp8=fp8, max_seqs=6, layers=2, seed=31)
    sim.step(prompt_slots=[2, 5], query_lens=[1023, 64], fuse=fuse)
    sim.step(prompt_slots=[0], query_lens=[90], decode_slots=[5, 2], fuse=fuse)   # slot 2 crosses into chunk 2
    sim.step(prompt_slots=[1, 0], query_lens=[7, 30], decode_slots=[2], fuse=fuse)
    sim.step(decode_slots=[0, 1, 2, 5], fuse=fuse)
    sim.close()


def test_fp8_cache_through_prepare_step_and_forward(gpu_pool):
    """An fp8 cache holds one byte per element: the prologue must count rows of Hkv*D bytes (not the two
    bytes per element the reference hard-codes, llama.py:315), or an unfused decode step writes at twice
    the right offset.  Prompt, chunked prompt, then both decode paths; a sequence grows past the first
    chunk (2048 fp8 rows per 2 MiB at Hkv = 8)."""
    sim = BackendSim(fp8=True, max_seqs=4, seed=41, max_tokens=8192)
    sim.step(prompt_slots=[1, 2], query_lens=[2040, 100])
    sim.step(prompt_slots=[2], query_lens=[60])
    for fuse in (False, True, False, True):
        sim.step(decode_slots=[2, 1], fuse=fuse)
    assert sim.eng.vmm_kvcache_segment[1].used_size == 2044 * 1024   # 1024 bytes per row, not 2048
    for fuse in (False, True, False, True, False, True):
        sim.step(decode_slots=[1], fuse=fuse)
    assert sim.eng.vmm_kvcache_segment[1].actual_size == 2 * (2 << 20)
    sim.close()
