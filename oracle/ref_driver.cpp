// TEST INFRASTRUCTURE - NOT PRODUCT CODE.
//
// C entry points around the reference's own CPU kernels, so that tests can call the
// real reference (compiled from its sources where they lie, never copied) without its
// Python package.  The reference functions called here are defined in
//   GLakeServe/csrc/cpu/attention.cpp:415-430  paged_attention_v1
//   GLakeServe/csrc/cpu/attention.cpp:730-746  paged_attention_v2
//   GLakeServe/csrc/cpu/cache.cpp:84-101       copy_blocks
//   GLakeServe/csrc/cpu/cache.cpp:103-128      reshape_and_cache
// This file only wraps caller-owned host buffers as tensors and forwards.
#include <torch/torch.h>

#include <string>
#include <vector>

void paged_attention_v1(torch::Tensor &out, torch::Tensor &query, torch::Tensor &key_cache,
                        torch::Tensor &value_cache, int num_kv_heads, float scale, torch::Tensor &block_tables,
                        torch::Tensor &seq_lens, int block_size, int max_seq_len,
                        const c10::optional<torch::Tensor> &alibi_slopes, const std::string &kv_cache_dtype,
                        float kv_scale);
void paged_attention_v2(torch::Tensor &out, torch::Tensor &exp_sums, torch::Tensor &max_logits,
                        torch::Tensor &tmp_out, torch::Tensor &query, torch::Tensor &key_cache,
                        torch::Tensor &value_cache, int num_kv_heads, float scale, torch::Tensor &block_tables,
                        torch::Tensor &seq_lens, int block_size, int max_seq_len,
                        const c10::optional<torch::Tensor> &alibi_slopes, const std::string &kv_cache_dtype,
                        float kv_scale);
void copy_blocks(std::vector<torch::Tensor> &key_caches, std::vector<torch::Tensor> &value_caches,
                 const torch::Tensor &block_mapping);
void reshape_and_cache(torch::Tensor &key, torch::Tensor &value, torch::Tensor &key_cache,
                       torch::Tensor &value_cache, torch::Tensor &slot_mapping, const std::string &kv_cache_dtype,
                       float kv_scale);

namespace {
torch::ScalarType st(int dtype) { return dtype == 0 ? torch::kFloat32 : torch::kBFloat16; }
torch::Tensor blob(void *p, std::vector<int64_t> shape, torch::ScalarType t) {
  return torch::from_blob(p, shape, torch::TensorOptions().dtype(t));
}
}  // namespace

extern "C" {

int ref_num_threads() { return at::get_num_threads(); }

// dtype: 0 = fp32, 1 = bf16.  Cache shapes: K [nb,Hkv,D/x,bs,x], V [nb,Hkv,D,bs], x = 16/elem.
int ref_paged_attention(int version, void *out, void *q, void *k_cache, void *v_cache, int dtype, int num_seqs,
                        int num_heads, int num_kv_heads, int head_size, int num_blocks, int block_size, float scale,
                        int *block_tables, int max_blocks_per_seq, int *seq_lens, int max_seq_len,
                        float *alibi_slopes, float *exp_sums, float *max_logits, void *tmp_out,
                        int max_num_partitions) {
  try {
    const int x = dtype == 0 ? 4 : 8;
    auto t = st(dtype);
    auto o = blob(out, {num_seqs, num_heads, head_size}, t);
    auto qq = blob(q, {num_seqs, num_heads, head_size}, t);
    auto kc = blob(k_cache, {num_blocks, num_kv_heads, head_size / x, block_size, x}, t);
    auto vc = blob(v_cache, {num_blocks, num_kv_heads, head_size, block_size}, t);
    auto bt = blob(block_tables, {num_seqs, max_blocks_per_seq}, torch::kInt32);
    auto sl = blob(seq_lens, {num_seqs}, torch::kInt32);
    c10::optional<torch::Tensor> al;
    if (alibi_slopes) al = blob(alibi_slopes, {num_heads}, torch::kFloat32);
    if (version == 1) {
      paged_attention_v1(o, qq, kc, vc, num_kv_heads, scale, bt, sl, block_size, max_seq_len, al, "auto", 1.0f);
    } else {
      auto es = blob(exp_sums, {num_seqs, num_heads, max_num_partitions}, torch::kFloat32);
      auto ml = blob(max_logits, {num_seqs, num_heads, max_num_partitions}, torch::kFloat32);
      auto to = blob(tmp_out, {num_seqs, num_heads, max_num_partitions, head_size}, t);
      paged_attention_v2(o, es, ml, to, qq, kc, vc, num_kv_heads, scale, bt, sl, block_size, max_seq_len, al, "auto",
                         1.0f);
    }
    return 0;
  } catch (const std::exception &e) {
    fprintf(stderr, "ref_paged_attention: %s\n", e.what());
    return -1;
  }
}

int ref_reshape_and_cache(void *key, void *value, void *k_cache, void *v_cache, int dtype, int num_tokens,
                          int num_heads, int head_size, long key_stride, long value_stride, int num_blocks,
                          int block_size, long *slot_mapping) {
  try {
    const int x = dtype == 0 ? 4 : 8;
    auto t = st(dtype);
    auto opt = torch::TensorOptions().dtype(t);
    auto k = torch::from_blob(key, {num_tokens, num_heads, head_size}, {key_stride, head_size, 1}, opt);
    auto v = torch::from_blob(value, {num_tokens, num_heads, head_size}, {value_stride, head_size, 1}, opt);
    auto kc = blob(k_cache, {num_blocks, num_heads, head_size / x, block_size, x}, t);
    auto vc = blob(v_cache, {num_blocks, num_heads, head_size, block_size}, t);
    auto sm = blob(slot_mapping, {num_tokens}, torch::kInt64);
    reshape_and_cache(k, v, kc, vc, sm, "auto", 1.0f);
    return 0;
  } catch (const std::exception &e) {
    fprintf(stderr, "ref_reshape_and_cache: %s\n", e.what());
    return -1;
  }
}

int ref_copy_blocks(void **key_caches, void **value_caches, int num_layers, int dtype, int num_blocks,
                    long block_elems, long *mapping, int num_pairs) {
  try {
    auto t = st(dtype);
    std::vector<torch::Tensor> ks, vs;
    for (int l = 0; l < num_layers; ++l) {
      ks.push_back(blob(key_caches[l], {num_blocks, block_elems}, t));
      vs.push_back(blob(value_caches[l], {num_blocks, block_elems}, t));
    }
    auto m = blob(mapping, {num_pairs, 2}, torch::kInt64);
    copy_blocks(ks, vs, m);
    return 0;
  } catch (const std::exception &e) {
    fprintf(stderr, "ref_copy_blocks: %s\n", e.what());
    return -1;
  }
}
}
