"""Prefix reuse end to end: the radix tree (glake_amd/core/radix_cache.py) finds the longest cached prefix of a
prompt, its holders are cache-engine slots cut from one another with KVcacheSegment.share_prefix (whole chunks
mapped a second time, the partly filled chunk copied), and the prompt's remaining tokens run through
prepare_step + VTensorImpl.forward behind the shared rows.  Three prompts with nested common prefixes: 2500 rows
(ends inside the third chunk) and 1024 rows (ends on a chunk boundary; the V rows' 256-byte offset spills into the
next chunk).  Checked: the number of physical chunks mapped more than once against its closed form, the cache
bytes of every running slot against the rows fed (shared part included), the attention output of the new tokens
against the oracle over all rows, and the pool's balance after eviction."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

from kvharness import bits_from_torch_bf16, torch_bf16_from_bits

pytestmark = pytest.mark.gpu


def test_three_prompts_with_nested_shared_prefixes(gpu_pool):
    import torch

    from glake_amd import _C
    from glake_amd.attention.backends.vtensor import VTensorBackend
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.prefix_store import PrefixStore
    from glake_amd.worker.step import prepare_step

    vmm = gpu_pool
    vmm.trim()
    free0 = vmm.showFreeBlocks()
    layers, hq, hkv, d, max_seqs = 2, 32, 8, 128, 8
    row = hkv * d * 2                                     # 1024 rows per 2 MiB chunk
    rng = np.random.default_rng(5)
    eng = CacheEngine(layers, hkv, d, torch.bfloat16, max_seqs, 4096)
    store = PrefixStore(eng, cache_slots=[3, 4, 5, 6, 7])     # five holders: A, B, C and the two cuts
    impl = VTensorBackend.get_impl_cls()(hq, d, d ** -0.5, hkv, None, None, "auto")
    dev = torch.device("cuda")

    def rand_rows(n):
        return [(O.f32_to_bf16(rng.standard_normal((n, hkv, d)).astype(np.float32)),
                 O.f32_to_bf16(rng.standard_normal((n, hkv, d)).astype(np.float32))) for _ in range(layers)]

    def extend(rows, n_keep, n_new):
        fresh = rand_rows(n_new)
        return [(np.concatenate([k[:n_keep], fk]), np.concatenate([v[:n_keep], fv])) for (k, v), (fk, fv) in zip(rows, fresh)]

    tok_a = list(range(3000))
    tok_b = tok_a[:2500] + list(range(50000, 50500))
    tok_c = tok_a[:1024] + list(range(70000, 70300))
    rows_a = rand_rows(3000)
    rows_b = extend(rows_a, 2500, 500)                   # same tokens -> same KV rows for the common part
    rows_c = extend(rows_a, 1024, 300)

    def run_prompt(tokens, rows, run_slot, expect_cached):
        cache_slot, cached = store.lookup(tokens)
        assert cached == expect_cached
        if cached:
            store.start_from(run_slot, cache_slot, cached)
        store.end_step()                                  # (a lookup keeps its holder from eviction until then)
        n, nq = len(tokens), len(tokens) - cached
        meta = VTensorBackend.make_metadata(
            num_prefills=1, num_prefill_tokens=nq, num_decode_tokens=0,
            slot_mapping=torch.tensor([run_slot], dtype=torch.int64, device=dev), seq_lens=[n],
            seq_lens_tensor=torch.tensor([n], dtype=torch.int32, device=dev), max_query_len=nq, max_prefill_seq_len=n,
            max_decode_seq_len=0, query_start_loc=None, seq_start_loc=None, context_lens_tensor=None, block_tables=None,
            is_extend=0, kv_batch_stride=eng.kv_batch_stride, kv_num_heads=hkv, kv_head_size=d, max_seq_len=n,
            slot_mapping_list=[run_slot], set_used_size=[cached], extend_seq_list=[-1], use_cuda_graph=False)
        meta.query_lens = [nq]
        meta.k_cache_segment_ptr_list, meta.v_cache_segment_ptr_list = eng.k_cache_ptr, eng.v_cache_ptr
        meta.kvcache_segment = [eng.vmm_kvcache_segment[run_slot]]
        prepare_step(meta, eng.gpu_cache)
        assert meta.slot_m.tolist() == [cached * row]
        seg = eng.vmm_kvcache_segment[run_slot]
        for l in range(layers):
            k, v = rows[l]
            q = O.f32_to_bf16(rng.standard_normal((nq, hq * d)).astype(np.float32))
            kc, vc = eng.gpu_cache[l]
            out = impl.forward(torch_bf16_from_bits(q), torch_bf16_from_bits(k[cached:].reshape(nq, hkv * d)),
                               torch_bf16_from_bits(v[cached:].reshape(nq, hkv * d)), kc, vc, meta)
            torch.cuda.synchronize()
            for want, ptr in ((k, seg.getKeyDevicePtr(l)), (v, seg.getValueDevicePtr(l))):
                back = np.empty_like(want)
                _C.check(_C.lib().vtkv_memcpy_d2h(back.ctypes.data_as(C.c_void_p), ptr, want.nbytes))
                assert np.array_equal(back, want), ("cache bytes", run_slot, l)
            tail = min(nq, 40)                            # the last query positions see all rows
            kb = [np.zeros((1, hkv, d), np.uint16)] * max_seqs
            vb = list(kb)
            kb[run_slot], vb[run_slot] = k, v
            want = O.prefill_attention(q.reshape(nq, hq, d)[nq - tail:], O.VTensorCache(kb, vb, [run_slot], hkv, d),
                                       d ** -0.5, [tail], [n])
            got = O.bf16_to_f32(bits_from_torch_bf16(out).reshape(nq, hq, d)[nq - tail:])
            diff = np.abs(got - O.bf16_to_f32(want))
            assert np.all(diff <= 2e-3 + (2e-3 + 2.0 ** -7) * np.abs(O.bf16_to_f32(want)))
        return seg

    def finish(tokens, run_slot, known):
        assert store.keep(tokens, run_slot) == known
        torch.cuda.synchronize()
        eng.vmm_kvcache_segment[run_slot].release_seq(run_slot)

    per_prefix_chunk = 2 * layers                        # a K and a V chunk in every layer
    # A: nothing cached.  Keeping it maps its two whole chunks (2048 of 3000 rows) a second time.
    run_prompt(tok_a, rows_a, 0, 0)
    assert vmm.sharedBlocks() == 0
    assert store.keep(tok_a, 0) == 0 and vmm.sharedBlocks() == 2 * per_prefix_chunk
    torch.cuda.synchronize()
    eng.vmm_kvcache_segment[0].release_seq(0)
    assert vmm.sharedBlocks() == 0                       # one user left
    # B: 2500 rows in common.  The tree cuts a 2500-row holder from A's (two whole chunks shared, 452 rows
    # copied), B's slot starts from it (the same two chunks, a third user).
    free_before = vmm.showFreeBlocks()
    run_prompt(tok_b, rows_b, 1, 2500)
    assert vmm.sharedBlocks() == 2 * per_prefix_chunk
    # chunks taken from the pool: the cut holder's own third chunk, and B's own third and fourth (rows
    # 2048..2999 and the slack of 100 rows: 3100 rows pass the 3072 that three chunks hold)
    assert free_before - vmm.showFreeBlocks() == 3 * per_prefix_chunk
    finish(tok_b, 1, 2500)
    assert vmm.sharedBlocks() == 2 * per_prefix_chunk    # A's, the cut's and B's holders share chunks 0 and 1
    # C: 1024 rows in common: exactly chunk 0.  The new holder shares chunk 0 and owns one more chunk for the
    # last 256 bytes of the V rows, which sit 256 bytes into their range.
    free_before = vmm.showFreeBlocks()
    seg = run_prompt(tok_c, rows_c, 2, 1024)
    assert vmm.sharedBlocks() == 2 * per_prefix_chunk
    assert seg.actual_size == 2 * (2 << 20)              # 1324 rows + slack: two chunks, the first one shared
    assert free_before - vmm.showFreeBlocks() == 2 * per_prefix_chunk   # one own chunk each: the cut and C
    finish(tok_c, 2, 1024)
    # a fourth lookup of a cached prompt in full runs its last token only
    slot, n = store.lookup(tok_a)
    assert n == len(tok_a) - 1 and store.rows[slot] == len(tok_a)
    # B's and C's holders go; not the one the lookup handed out, nor the cuts that lead to it
    assert store.evict(10 ** 9) == 3000 + 1324
    store.end_step()
    # eviction frees every holder; shared chunks go back with their last user
    assert store.evict(10 ** 9) == 3000 + 2500 + 1024
    assert vmm.sharedBlocks() == 0 and sorted(store.free_slots) == [3, 4, 5, 6, 7]
    eng.close()
    assert vmm.showFreeBlocks() == free0
