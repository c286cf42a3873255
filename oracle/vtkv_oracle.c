/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's KV-cache hot path, used only as the
 * checker in tests, in the smoke test and as the timed CPU baseline.  Nothing
 * in the shipped library calls into this file.
 *
 * Each function names the reference file:line whose algorithm it follows
 * (paths relative to the reference's GLakeServe/ directory).
 *
 * Numeric conventions restated from the reference's CPU twin:
 *   - bf16 inputs are widened to fp32 exactly (csrc/cpu/cpu_types.hpp:259-261);
 *   - all arithmetic is fp32 (csrc/cpu/attention.cpp:22-39 KernelVecType);
 *   - softmax divides by the exact sum, no epsilon (csrc/cpu/attention.cpp:43-67);
 *   - fp32 -> bf16 on store TRUNCATES in the build without AVX512-BF16
 *     (csrc/cpu/cpu_types.hpp:332-346) and rounds to nearest even in the build
 *     with it (csrc/cpu/cpu_types.hpp:315-330); `bf16_round` selects which.
 *
 * Pinning status (what checks each function against something other than itself):
 *   oracle_paged_attention_v1 / _v2 : compiled reference CPU twin (oracle/_ref),
 *       float64 textbook softmax(QK^T)V, T=1 closed form, block-id permutation
 *       invariance, v1 == v2 partition invariance.
 *   oracle_reshape_and_cache_paged  : compiled reference CPU twin, closed-form index
 *       formula of tests/kernels/test_cache.py:170-180.
 *   oracle_copy_blocks              : compiled reference CPU twin, identity.
 *   oracle_reshape_and_cache_vtensor: brute-force address formula; equals the paged
 *       variant at block_size 1 up to the [T,Hkv,D] collapse.
 *   oracle_fp8_e4m3fn_*, oracle_convert_to_fp8 : torch.float8_e4m3fn casts (library routine),
 *       exhaustive over the 256 codes and all 65536 bf16 inputs at scale 1, and with a
 *       scale (torch's cast of the IEEE quotient x / scale) over all bf16 inputs for each of
 *       the 112 scales of the reference's tests/fp8_kv/.../kv_cache_scales.json and eight
 *       others, random fp32 inputs and inputs whose quotient is an exact tie.
 *   oracle_reshape_and_cache_vtensor_fp8 : the same cast plus the address formula of
 *       csrc/cache_kernels.cu:176-199 in numpy, skipped rows and strided sources included.
 *   oracle_swap_blocks              : want[dst] = src[src] by numpy indexing on the block
 *       pairs of the reference's tests/worker/test_swap.py:57-89 and on random pairs.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_DTYPE_F32 0
#define ORACLE_DTYPE_BF16 1
#define ORACLE_LAYOUT_PAGED 0   /* K [nb,Hkv,D/x,bs,x], V [nb,Hkv,D,bs]  (vllm/attention/ops/paged_attn.py:47-59) */
#define ORACLE_LAYOUT_VTENSOR 1 /* per-sequence base pointer, [T,Hkv,D]   (csrc/cache_kernels.cu:176-199)          */

static inline float bf16_to_f32(uint16_t v) {
  uint32_t u = ((uint32_t)v) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* csrc/cpu/cpu_types.hpp:332-346 (truncate) or :315-330 (round to nearest even) */
static inline uint16_t f32_to_bf16(float f, int round_nearest) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if (!round_nearest) return (uint16_t)(u >> 16);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

static inline float load_elem(const void *base, int64_t idx, int dtype) {
  return dtype == ORACLE_DTYPE_F32 ? ((const float *)base)[idx] : bf16_to_f32(((const uint16_t *)base)[idx]);
}

static inline void store_elem(void *base, int64_t idx, float v, int dtype, int bf16_round) {
  if (dtype == ORACLE_DTYPE_F32)
    ((float *)base)[idx] = v;
  else
    ((uint16_t *)base)[idx] = f32_to_bf16(v, bf16_round);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------------- */
/* Cache layout description shared by the attention restatements.            */
typedef struct {
  int layout;               /* ORACLE_LAYOUT_* */
  int dtype;                /* ORACLE_DTYPE_*  */
  const void *k_cache;      /* paged: base of K blocks                         */
  const void *v_cache;      /* paged: base of V blocks                         */
  const int32_t *block_tables; /* paged: [num_seqs, max_num_blocks_per_seq]    */
  int max_num_blocks_per_seq;
  int block_size;           /* paged: tokens per block                         */
  int64_t kv_block_stride;  /* paged: elements between blocks  (key_cache.stride(0)) */
  int64_t kv_head_stride;   /* paged: elements between heads   (key_cache.stride(1)) */
  const int64_t *k_ptrs;    /* vtensor: per-slot base addresses                */
  const int64_t *v_ptrs;
  const int64_t *slot_mapping; /* vtensor: [num_seqs] slot of each sequence    */
  int num_kv_heads;
  int head_size;
} oracle_cache_t;

/* Gather 16 tokens (one reference BLOCK_SIZE worth) of K and V for one kv head into
 * fp32 scratch rows k[16][D], v[16][D].  Addressing:
 *   paged   : csrc/cpu/attention.cpp:266-269 (K block ptr), :119-195 (x-interleaved K),
 *             :197-211 (V rows of block_size), layout vllm/attention/ops/paged_attn.py:47-59
 *   vtensor : csrc/attention/attention_kernels.cu:194,221-224 with BLOCK_SIZE=1 collapsing
 *             to token-major [T,Hkv,D] (csrc/cache_kernels.cu:176-199) */
static void gather_tokens(const oracle_cache_t *c, int seq_idx, int kv_head, int tok0, int ntok, float *k, float *v) {
  const int D = c->head_size;
  if (c->layout == ORACLE_LAYOUT_PAGED) {
    const int x = c->dtype == ORACLE_DTYPE_F32 ? 4 : 8; /* 16 / sizeof(scalar_t), csrc/cpu/attention.cpp:236 */
    const int bs = c->block_size;
    for (int i = 0; i < ntok; ++i) {
      const int t = tok0 + i;
      const int64_t blk = c->block_tables[(int64_t)seq_idx * c->max_num_blocks_per_seq + t / bs];
      const int off = t % bs;
      const int64_t base = blk * c->kv_block_stride + (int64_t)kv_head * c->kv_head_stride;
      for (int d = 0; d < D; ++d) {
        k[i * D + d] = load_elem(c->k_cache, base + (int64_t)(d / x) * bs * x + (int64_t)off * x + d % x, c->dtype);
        v[i * D + d] = load_elem(c->v_cache, base + (int64_t)d * bs + off, c->dtype);
      }
    }
  } else {
    const int64_t slot = c->slot_mapping[seq_idx];
    const void *kb = (const void *)(intptr_t)c->k_ptrs[slot];
    const void *vb = (const void *)(intptr_t)c->v_ptrs[slot];
    for (int i = 0; i < ntok; ++i) {
      const int64_t row = ((int64_t)(tok0 + i) * c->num_kv_heads + kv_head) * D;
      for (int d = 0; d < D; ++d) {
        k[i * D + d] = load_elem(kb, row + d, c->dtype);
        v[i * D + d] = load_elem(vb, row + d, c->dtype);
      }
    }
  }
}

/* csrc/cpu/attention.cpp:119-195 reduceQKBlockKernel: q.k per token, x partial lanes
 * (d % x) accumulated over d / x steps, then summed; result times scale. */
static void qk_block(const float *q, const float *k, int D, int x, int ntok, float scale, float *logits) {
  for (int i = 0; i < ntok; ++i) {
    float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int d0 = 0; d0 < D; d0 += x)
      for (int j = 0; j < x; ++j) lanes[j] = lanes[j] + q[d0 + j] * k[i * D + d0 + j];
    float dot = 0.f;
    for (int j = 0; j < x; ++j) dot += lanes[j];
    logits[i] = dot * scale;
  }
}

/* csrc/cpu/attention.cpp:43-67 reduceSoftmax and :69-98 reduceSoftmaxAlibi.
 * Returns max and sum through pointers; data[0..size) becomes exp(x-max)/sum,
 * data[size..capacity) is zeroed. */
static void reduce_softmax(float *data, int size, int capacity, const float *alibi_slope, int start_index, int seq_len,
                           float *out_max, float *out_sum) {
  if (alibi_slope) {
    for (int i = 0; i < size; ++i) data[i] = data[i] + (*alibi_slope) * (float)(start_index + i - seq_len + 1);
  }
  float mx = data[0];
  for (int i = 1; i < size; ++i) mx = mx >= data[i] ? mx : data[i];
  float sum = 0.f;
  for (int i = 0; i < size; ++i) {
    data[i] = expf(data[i] - mx);
    sum += data[i];
  }
  for (int i = 0; i < size; ++i) data[i] /= sum;
  for (int i = size; i < capacity; ++i) data[i] = 0.f;
  *out_max = mx;
  *out_sum = sum;
}

/* csrc/cpu/attention.cpp:197-211 reduceValueBlock + :300-330: per head element an
 * accumulator with 16 lanes (lane = token offset inside the 16-token block), summed
 * at the end (reduce_sum). */
static void pv_accumulate(const float *prob16, const float *v, int D, int ntok, float *acc /* [D][16] */) {
  for (int d = 0; d < D; ++d)
    for (int i = 0; i < ntok; ++i) acc[d * 16 + i] = acc[d * 16 + i] + prob16[i] * v[i * D + d];
}

/* One (sequence, head, token range) work item: logits -> softmax -> P.V.
 * Shared by v1 (whole sequence, csrc/cpu/attention.cpp:246-332) and by v2's first
 * phase (one 512-token partition, csrc/cpu/attention.cpp:463-580). */
static void attend_range(const oracle_cache_t *c, const void *q, int q_dtype, int64_t q_off, int seq_idx, int head_idx,
                         int num_queries_per_kv, float scale, const float *alibi_slope, int start_tok, int ntok,
                         int seq_len, float *logits /* >= round16(ntok) */, float *out_f32 /* [D] */, float *out_max,
                         float *out_sum) {
  const int D = c->head_size;
  const int x = c->dtype == ORACLE_DTYPE_F32 ? 4 : 8;
  const int kv_head = head_idx / num_queries_per_kv;
  const int nblk = (ntok + 15) / 16;
  float *qf = (float *)malloc(sizeof(float) * D);
  float *kbuf = (float *)malloc(sizeof(float) * 16 * D * 2);
  float *vbuf = kbuf + 16 * D;
  float *acc = (float *)calloc((size_t)D * 16, sizeof(float));
  for (int d = 0; d < D; ++d) qf[d] = load_elem(q, q_off + d, q_dtype);
  for (int b = 0; b < nblk; ++b) {
    const int n = (b == nblk - 1) ? ntok - b * 16 : 16;
    gather_tokens(c, seq_idx, kv_head, start_tok + b * 16, n, kbuf, vbuf);
    qk_block(qf, kbuf, D, x, n, scale, logits + b * 16);
  }
  reduce_softmax(logits, ntok, nblk * 16, alibi_slope, start_tok, seq_len, out_max, out_sum);
  for (int b = 0; b < nblk; ++b) {
    const int n = (b == nblk - 1) ? ntok - b * 16 : 16;
    gather_tokens(c, seq_idx, kv_head, start_tok + b * 16, n, kbuf, vbuf);
    pv_accumulate(logits + b * 16, vbuf, D, n, acc);
  }
  for (int d = 0; d < D; ++d) {
    float s = 0.f;
    for (int i = 0; i < 16; ++i) s += acc[d * 16 + i];
    out_f32[d] = s;
  }
  free(acc);
  free(kbuf);
  free(qf);
}

/* csrc/cpu/attention.cpp:216-338 paged_attention_v1_impl::call.
 * out/q: [num_seqs, num_heads, D] in `q_dtype`; out rows are contiguous, q has
 * row stride q_stride elements (csrc/cpu/attention.cpp:253-254, :283-285). */
int oracle_paged_attention_v1(void *out, const void *q, int q_dtype, int64_t q_stride, const oracle_cache_t *cache,
                              float scale, const int32_t *seq_lens, int num_seqs, int num_heads,
                              const float *alibi_slopes, int bf16_round) {
  const int D = cache->head_size;
  if (num_heads % cache->num_kv_heads != 0) return -1;
  const int qpk = num_heads / cache->num_kv_heads;
  int max_len = 0;
  for (int s = 0; s < num_seqs; ++s) max_len = seq_lens[s] > max_len ? seq_lens[s] : max_len;
  const int padded = (max_len + 15) & ~15;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < num_seqs; ++s) {
    for (int h = 0; h < num_heads; ++h) {
      const int seq_len = seq_lens[s];
      if (seq_len <= 0) continue;
      float *logits = (float *)malloc(sizeof(float) * (size_t)(padded + 16));
      float *o = (float *)malloc(sizeof(float) * D);
      float mx, sum;
      attend_range(cache, q, q_dtype, (int64_t)s * q_stride + (int64_t)h * D, s, h, qpk, scale,
                   alibi_slopes ? &alibi_slopes[h] : NULL, 0, seq_len, seq_len, logits, o, &mx, &sum);
      for (int d = 0; d < D; ++d) store_elem(out, ((int64_t)s * num_heads + h) * D + d, o[d], q_dtype, bf16_round);
      free(o);
      free(logits);
    }
  }
  return 0;
}

/* csrc/cpu/attention.cpp:100-117 reducePartitonSoftmax */
static void reduce_partition_softmax(const float *max_data, float *sum_data, int size) {
  float mx = max_data[0];
  for (int i = 1; i < size; ++i) mx = mx >= max_data[i] ? mx : max_data[i];
  float rescaled_sum = 0.f;
  for (int i = 0; i < size; ++i) {
    float f = expf(max_data[i] - mx);
    rescaled_sum += f * sum_data[i];
    sum_data[i] *= f;
  }
  for (int i = 0; i < size; ++i) sum_data[i] = (float)((double)sum_data[i] / ((double)rescaled_sum + 1e-8));
}

/* csrc/cpu/attention.cpp:434-646 paged_attention_v2_impl::call, PARTITION_SIZE = 512
 * (:648).  exp_sums/max_logits: fp32 [num_seqs,num_heads,max_num_partitions];
 * tmp_out: q_dtype [num_seqs,num_heads,max_num_partitions,D] (stored in the model
 * dtype, so bf16 adds one rounding, :535-541, :569-573). */
int oracle_paged_attention_v2(void *out, float *exp_sums, float *max_logits, void *tmp_out, const void *q, int q_dtype,
                              int64_t q_stride, const oracle_cache_t *cache, float scale, const int32_t *seq_lens,
                              int num_seqs, int num_heads, int max_num_partitions, const float *alibi_slopes,
                              int bf16_round) {
  enum { PARTITION_SIZE = 512 };
  const int D = cache->head_size;
  if (num_heads % cache->num_kv_heads != 0) return -1;
  const int qpk = num_heads / cache->num_kv_heads;
  /* phase 1: per-partition attention, csrc/cpu/attention.cpp:463-580 */
#pragma omp parallel for collapse(3) schedule(static, 1)
  for (int s = 0; s < num_seqs; ++s) {
    for (int p = 0; p < max_num_partitions; ++p) {
      for (int h = 0; h < num_heads; ++h) {
        const int seq_len = seq_lens[s];
        const int start = p * PARTITION_SIZE;
        if (start >= seq_len) continue;
        const int partition_num = (seq_len + PARTITION_SIZE - 1) / PARTITION_SIZE;
        const int no_reduce = partition_num == 1;
        const int ntok = (seq_len < start + PARTITION_SIZE ? seq_len : start + PARTITION_SIZE) - start;
        float logits[PARTITION_SIZE];
        float o[256];
        float mx, sum;
        memset(logits, 0, sizeof(logits));
        attend_range(cache, q, q_dtype, (int64_t)s * q_stride + (int64_t)h * D, s, h, qpk, scale,
                     alibi_slopes ? &alibi_slopes[h] : NULL, start, ntok, seq_len, logits, o, &mx, &sum);
        if (!no_reduce) {
          const int64_t idx = ((int64_t)s * num_heads + h) * max_num_partitions + p;
          max_logits[idx] = mx;
          exp_sums[idx] = sum;
          for (int d = 0; d < D; ++d) store_elem(tmp_out, idx * D + d, o[d], q_dtype, bf16_round);
        } else {
          for (int d = 0; d < D; ++d)
            store_elem(out, ((int64_t)s * num_heads + h) * D + d, o[d], q_dtype, bf16_round);
        }
      }
    }
  }
  /* phase 2: rescale factors, csrc/cpu/attention.cpp:583-600 */
#pragma omp parallel for collapse(2) schedule(static, 1)
  for (int s = 0; s < num_seqs; ++s) {
    for (int h = 0; h < num_heads; ++h) {
      const int partition_num = (seq_lens[s] + PARTITION_SIZE - 1) / PARTITION_SIZE;
      if (partition_num <= 1) continue;
      const int64_t base = ((int64_t)s * num_heads + h) * max_num_partitions;
      reduce_partition_softmax(max_logits + base, exp_sums + base, partition_num);
    }
  }
  /* phase 3: weighted sum of partition outputs, csrc/cpu/attention.cpp:611-644 */
#pragma omp parallel for collapse(2) schedule(static, 1)
  for (int s = 0; s < num_seqs; ++s) {
    for (int h = 0; h < num_heads; ++h) {
      const int partition_num = (seq_lens[s] + PARTITION_SIZE - 1) / PARTITION_SIZE;
      if (partition_num <= 1) continue;
      const int64_t base = ((int64_t)s * num_heads + h) * max_num_partitions;
      for (int d = 0; d < D; ++d) {
        float acc = 0.f;
        for (int p = 0; p < partition_num; ++p) acc = acc + load_elem(tmp_out, (base + p) * D + d, q_dtype) * exp_sums[base + p];
        store_elem(out, ((int64_t)s * num_heads + h) * D + d, acc, q_dtype, bf16_round);
      }
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* csrc/cpu/cache.cpp:34-81 reshape_and_cache_cpu_impl (paged scatter).
 * key/value: [num_tokens, num_heads, head_size] with row strides key_stride /
 * value_stride (elements); slot < 0 skips the token (:46). elem_size in bytes. */
int oracle_reshape_and_cache_paged(const void *key, const void *value, void *key_cache, void *value_cache,
                                   const int64_t *slot_mapping, int num_tokens, int64_t key_stride,
                                   int64_t value_stride, int num_heads, int head_size, int block_size, int x,
                                   int elem_size) {
  const int64_t block_elem_num = (int64_t)num_heads * head_size * block_size;
  const char *kp = (const char *)key, *vp = (const char *)value;
  char *kc = (char *)key_cache, *vc = (char *)value_cache;
  if (head_size % x != 0) return -1;
#pragma omp parallel for collapse(2)
  for (int t = 0; t < num_tokens; ++t) {
    for (int h = 0; h < num_heads; ++h) {
      const int64_t slot = slot_mapping[t];
      if (slot < 0) continue;
      const int64_t blk = slot / block_size, off = slot % block_size;
      const int64_t src_k = t * key_stride + (int64_t)h * head_size;
      const int64_t src_v = t * value_stride + (int64_t)h * head_size;
      const int64_t dst_head = block_elem_num * blk + (int64_t)h * block_size * head_size;
      for (int d = 0; d < head_size; d += x) {
        const int64_t dst = dst_head + (int64_t)d * block_size + off * x;
        memcpy(kc + dst * elem_size, kp + (src_k + d) * elem_size, (size_t)x * elem_size);
      }
      for (int d = 0; d < head_size; ++d) {
        const int64_t dst = dst_head + (int64_t)d * block_size + off;
        memcpy(vc + dst * elem_size, vp + (src_v + d) * elem_size, (size_t)elem_size);
      }
    }
  }
  return 0;
}

/* csrc/cache_kernels.cu:153-200 reshape_and_cache_kernel (vTensor scatter).
 * For sequence b and token t of the launch grid (batch, max_seq_len):
 *   dst = ptr_table[slot_mapping[b]] + slot_m[b] + t * Hkv*D*elem   (:176-180)
 *   src = key + b*key_stride                      when max_seq_len == 1 (:184-186)
 *       = key + (cache_seq_lens[b] + t)*key_stride otherwise           (:187-190)
 * rows with slot_mapping[b] < 0 are skipped (:172-175); rows with t >= seq_lens[b]
 * are skipped in the multi-token case (:171).  The reference hard-codes 2-byte
 * elements (:179-180); elem_size generalises that for fp32 test configs.
 * NOTE the reference indexes BOTH the pointer table and the byte offset by the
 * same arrays it is handed: `slot_mapping` holds the per-sequence byte offsets
 * (python slot_m) and `slot_map_list` the slot ids (python slot_mapping), see
 * csrc/cache_kernels.cu:172,176 and vllm/attention/ops/paged_attn.py:75-87. */
int oracle_reshape_and_cache_vtensor(const void *key, const void *value, const int64_t *k_ptrs, const int64_t *v_ptrs,
                                     const int64_t *slot_m /* byte offsets */, const int64_t *slot_ids,
                                     const int32_t *seq_lens, const int32_t *cache_seq_lens, int batch,
                                     int max_seq_len, int num_heads, int head_size, int64_t key_stride,
                                     int64_t value_stride, int elem_size) {
  const int64_t row_bytes = (int64_t)num_heads * head_size * elem_size;
  for (int b = 0; b < batch; ++b) {
    for (int t = 0; t < max_seq_len; ++t) {
      if (max_seq_len != 1 && t >= seq_lens[b]) continue;
      const int64_t off = slot_m[b];
      if (off < 0) continue;
      char *kd = (char *)(intptr_t)k_ptrs[slot_ids[b]] + off + t * row_bytes;
      char *vd = (char *)(intptr_t)v_ptrs[slot_ids[b]] + off + t * row_bytes;
      const int64_t src_row = max_seq_len == 1 ? b : (int64_t)cache_seq_lens[b] + t;
      memcpy(kd, (const char *)key + src_row * key_stride * elem_size, (size_t)row_bytes);
      memcpy(vd, (const char *)value + src_row * value_stride * elem_size, (size_t)row_bytes);
    }
  }
  return 0;
}

/* csrc/cpu/cache.cpp:7-32 copy_blocks_cpu_impl: for every layer and (src,dst) pair
 * copy one block of K and one of V inside the same cache tensor. */
int oracle_copy_blocks(void **key_caches, void **value_caches, int num_layers, const int64_t *mapping_pairs,
                       int num_pairs, int64_t block_bytes) {
  for (int l = 0; l < num_layers; ++l)
    for (int p = 0; p < num_pairs; ++p) {
      const int64_t src = mapping_pairs[2 * p] * block_bytes, dst = mapping_pairs[2 * p + 1] * block_bytes;
      memcpy((char *)key_caches[l] + dst, (char *)key_caches[l] + src, (size_t)block_bytes);
      memcpy((char *)value_caches[l] + dst, (char *)value_caches[l] + src, (size_t)block_bytes);
    }
  return 0;
}

/* csrc/cache_kernels.cu:24-69 swap_blocks: one copy of block_bytes per (src,dst) row
 * of an int64 [n,2] mapping. */
int oracle_swap_blocks(const void *src, void *dst, const int64_t *mapping, int num_pairs, int64_t block_bytes) {
  for (int p = 0; p < num_pairs; ++p)
    memcpy((char *)dst + mapping[2 * p + 1] * block_bytes, (const char *)src + mapping[2 * p] * block_bytes,
           (size_t)block_bytes);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* fp8 e4m3fn (OCP: bias 7, no inf, NaN = S.1111.111, max 448).
 * Encode follows csrc/quantization/fp8/nvidia/quant_utils.cuh:481-490:
 *   code = cvt_float_to_fp8(x / scale, SATFINITE, E4M3)
 * i.e. IEEE fp32 division, round to nearest even, finite overflow clamps to +-448,
 * NaN -> 0x7f.  Decode follows :406-417 (code -> float, times scale). */
uint8_t oracle_fp8_e4m3fn_encode(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);      /* NaN */
  if (a >= 0x43e80000u) return (uint8_t)(sign | 0x7eu);      /* >= 464 (midpoint 448..480) or inf: saturate to 448 */
  if (a < 0x3c800000u) {                                     /* < 2^-6: subnormal range, quantum 2^-9 */
    float f;
    memcpy(&f, &a, 4);
    float r = nearbyintf(f * 512.0f); /* exact scaling; default rounding mode = nearest even */
    return (uint8_t)(sign | (uint8_t)r); /* r in 0..8; 8 encodes as exp=1,mant=0 = 2^-6 */
  }
  /* normal: keep 3 mantissa bits, RNE on the 20 dropped bits */
  uint32_t lsb = (a >> 20) & 1u;
  uint32_t r = a + 0x7ffffu + lsb;
  uint32_t e = (r >> 23) - 127u + 7u;
  uint32_t m = (r >> 20) & 7u;
  uint32_t code = (e << 3) | m;
  if (code > 0x7eu) code = 0x7eu;
  return (uint8_t)(sign | code);
}

float oracle_fp8_e4m3fn_decode(uint8_t c) {
  const int sign = c & 0x80;
  const int e = (c >> 3) & 0xf, m = c & 7;
  float v;
  if (e == 0xf && m == 7)
    v = NAN;
  else if (e == 0)
    v = ldexpf((float)m, -9);
  else
    v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return sign ? -v : v;
}

/* csrc/cache_kernels.cu:346-357 convert_fp8_kernel, both directions, elementwise.
 * wide_dtype: ORACLE_DTYPE_F32 or ORACLE_DTYPE_BF16. */
int oracle_convert_to_fp8(uint8_t *dst, const void *src, int wide_dtype, int64_t n, float scale) {
  for (int64_t i = 0; i < n; ++i) dst[i] = oracle_fp8_e4m3fn_encode(load_elem(src, i, wide_dtype) / scale);
  return 0;
}

int oracle_convert_from_fp8(void *dst, const uint8_t *src, int wide_dtype, int64_t n, float scale) {
  for (int64_t i = 0; i < n; ++i) store_elem(dst, i, oracle_fp8_e4m3fn_decode(src[i]) * scale, wide_dtype, 1);
  return 0;
}

/* vTensor scatter with fp8 quantisation of bf16/fp32 sources: the layout rule of
 * csrc/cache_kernels.cu:176-199 with the element conversion of
 * csrc/quantization/fp8/nvidia/quant_utils.cuh:469-490 applied per element
 * (one code byte per element, so the row is Hkv*D bytes). Decode-step form only. */
int oracle_reshape_and_cache_vtensor_fp8(const void *key, const void *value, int src_dtype, const int64_t *k_ptrs,
                                         const int64_t *v_ptrs, const int64_t *slot_m, const int64_t *slot_ids,
                                         int batch, int num_heads, int head_size, int64_t key_stride,
                                         int64_t value_stride, float k_scale, float v_scale) {
  const int n = num_heads * head_size;
  for (int b = 0; b < batch; ++b) {
    if (slot_m[b] < 0) continue;
    uint8_t *kd = (uint8_t *)(intptr_t)k_ptrs[slot_ids[b]] + slot_m[b];
    uint8_t *vd = (uint8_t *)(intptr_t)v_ptrs[slot_ids[b]] + slot_m[b];
    for (int i = 0; i < n; ++i) {
      kd[i] = oracle_fp8_e4m3fn_encode(load_elem(key, b * key_stride + i, src_dtype) / k_scale);
      vd[i] = oracle_fp8_e4m3fn_encode(load_elem(value, b * value_stride + i, src_dtype) / v_scale);
    }
  }
  return 0;
}
