// Decode attention for float32 models: float32 queries over float32 K and V rows in the per-sequence contiguous
// ranges.  The reference runs its paged attention in float as well (tests/kernels/test_attention.py:23 DTYPES;
// csrc/cpu/attention.cpp has the float instantiations); nothing is deployed in float32, so this path is kept
// simple: it is the split-K form of the reference (csrc/attention/attention_kernels.cu:451-583,
// csrc/cpu/attention.cpp:434-746) with all arithmetic in fp32 on the vector unit.
//
//  * Kernel A: one workgroup per (query row, kv head, partition of `part_rows` rows).  A row of K or V for one kv
//    head is D floats; 32 lanes take 16 bytes each (two pieces each for D = 256), so a wave holds two rows at a
//    time and a workgroup eight.  Each half-wave walks over its rows four at a time (eight 16-byte loads in flight
//    per lane), computes the group's logits with a butterfly sum over its 32 lanes, and keeps an online softmax
//    per query head.  The eight partial results of a workgroup are merged through LDS; the partition's normalised
//    result, its maximum and its sum of exponentials go to the caller's buffers (split-K interface) or to the
//    workspace, or straight to `out` when no sequence of the call has more than one partition.
//  * Kernel B merges the partitions of a (query row, head) by the reference's rule.
//  * A kv head's query heads are taken up to eight at a time; larger groups make further passes over the rows.
//  * The same kernel serves prompt tokens (causal attention over the ranges, one query row per token, its length
//    the token's position plus one): every token then streams its own rows, which is the arithmetic of the
//    reference's prompt path without its reuse of rows between tokens.
//
// HBM-bound like the 16-bit kernels, at twice their bytes per row; per byte the vector unit has about a quarter of
// what it can issue to do.
#include "vtkv_common.h"

#include <algorithm>
#include <cmath>
#include <cstdint>

namespace {

constexpr int kThreads = 256;
constexpr int kHalves = 8;   // half-waves per workgroup: rows in flight
constexpr int kUnroll = 4;   // rows per half-wave and step
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct F32Params {
  const float *q;
  const int64_t *k_ptrs, *v_ptrs, *slot_ids;
  const int32_t *seq_lens;  // decode: one query row per sequence
  const int32_t *units;     // prompts: [n][4] = {sequence, first query row, query tokens, position of the first}
  const float *alibi_slopes;
  float *out;
  float *part_out, *part_max, *part_sum;  // [rows, num_heads, parts_dim(, D)]
  int64_t q_stride;
  int num_heads, num_kv_heads, head_size;
  int part_rows, parts_dim, unit_tokens;
  int direct;  // no query row has more than one partition: kernel A writes `out`
  float scale_log2;
};

typedef float f4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) f4 *gf4;

__device__ __forceinline__ float sum32(float v) {
#pragma unroll
  for (int d = 16; d >= 1; d >>= 1) v += __shfl_xor(v, d, 32);
  return v;
}

// Which query row a workgroup of kernel A or B serves: its sequence (index into slot_ids), its place among the
// query rows and the number of rows it attends to.  false: nothing to do.
__device__ __forceinline__ bool query_row(const F32Params &p, int z, int &seq, int &row, int &len) {
  if (p.units) {
    const int u = z / p.unit_tokens, t = z % p.unit_tokens;
    if (t >= p.units[4 * u + 2]) return false;
    seq = p.units[4 * u];
    row = p.units[4 * u + 1] + t;
    len = p.units[4 * u + 3] + t + 1;
  } else {
    seq = row = z;
    len = p.seq_lens[z];
  }
  return len > 0;
}

// GC: query heads per pass (1, 2, 4 or 8); KP: 16-byte pieces of a row per lane (1: D <= 128, 2: D = 256)
template <int GC, int KP>
__global__ void __launch_bounds__(kThreads) decode_attn_f32_kernel(F32Params p) {
  __shared__ float sm_o[4][GC][KP * 128];
  __shared__ float sm_m[4][GC], sm_l[4][GC];
  const int part = blockIdx.x, kvh = blockIdx.y;
  int seq, qrow, len;
  if (!query_row(p, blockIdx.z, seq, qrow, len)) return;
  const int row0 = part * p.part_rows;
  if (row0 >= len) return;
  const int row1 = min(len, row0 + p.part_rows);
  const int D = p.head_size, G = p.num_heads / p.num_kv_heads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, hw = wave * 2 + (lane >> 5);
  const int64_t slot = p.slot_ids[seq];
  const int64_t row_bytes = (int64_t)p.num_kv_heads * D * 4;
  const char *k_base = (const char *)(uintptr_t)p.k_ptrs[slot] + (int64_t)kvh * D * 4;
  const char *v_base = (const char *)(uintptr_t)p.v_ptrs[slot] + (int64_t)kvh * D * 4;
  bool piece_live[KP];
  int piece_off[KP];
#pragma unroll
  for (int pp = 0; pp < KP; ++pp) {
    piece_live[pp] = 4 * l32 + 128 * pp < D;
    piece_off[pp] = piece_live[pp] ? 16 * l32 + 512 * pp : 0;
  }

  for (int h0 = 0; h0 < G; h0 += GC) {
    // this pass's query heads; heads past the group get q = 0 and store nothing
    f4 qv[GC][KP], acc[GC][KP];
    float m_run[GC], l_run[GC], slope[GC];
#pragma unroll
    for (int j = 0; j < GC; ++j) {
      const int head = kvh * G + min(h0 + j, G - 1);
      const float *qp = p.q + (int64_t)qrow * p.q_stride + (int64_t)head * D;
#pragma unroll
      for (int pp = 0; pp < KP; ++pp) {
        qv[j][pp] = (f4){0.f, 0.f, 0.f, 0.f};
        if (piece_live[pp] && h0 + j < G) qv[j][pp] = *reinterpret_cast<const f4 *>(qp + 4 * l32 + 128 * pp);
        acc[j][pp] = (f4){0.f, 0.f, 0.f, 0.f};
      }
      m_run[j] = -INFINITY;
      l_run[j] = 0.f;
      slope[j] = p.alibi_slopes ? p.alibi_slopes[head] * kLog2e : 0.f;
    }
    for (int base = row0 + hw; base < row1; base += kHalves * kUnroll) {
      f4 kk[kUnroll][KP], vv[kUnroll][KP];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        // (rows past the end read the last row again; their weight is zero)
        const int64_t off = (int64_t)min(base + kHalves * u, row1 - 1) * row_bytes;
#pragma unroll
        for (int pp = 0; pp < KP; ++pp) {
          kk[u][pp] = __builtin_nontemporal_load((gf4)(k_base + off + piece_off[pp]));
          vv[u][pp] = __builtin_nontemporal_load((gf4)(v_base + off + piece_off[pp]));
          if (!piece_live[pp]) kk[u][pp] = (f4){0.f, 0.f, 0.f, 0.f};
          if (!piece_live[pp]) vv[u][pp] = (f4){0.f, 0.f, 0.f, 0.f};
        }
      }
#pragma unroll
      for (int j = 0; j < GC; ++j) {
        float x[kUnroll];
        float m_new = m_run[j];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          float s = 0.f;
#pragma unroll
          for (int pp = 0; pp < KP; ++pp)
            s += qv[j][pp][0] * kk[u][pp][0] + qv[j][pp][1] * kk[u][pp][1] + qv[j][pp][2] * kk[u][pp][2] +
                 qv[j][pp][3] * kk[u][pp][3];
          s = sum32(s);
          const int r = base + kHalves * u;
          x[u] = s * p.scale_log2 + slope[j] * (float)(r - len + 1);
          if (r >= row1) x[u] = -INFINITY;
          m_new = fmaxf(m_new, x[u]);
        }
        // (the first row of the step is always inside the partition, so m_new is finite)
        const float alpha = __builtin_amdgcn_exp2f(m_run[j] - m_new);
        m_run[j] = m_new;
        l_run[j] *= alpha;
#pragma unroll
        for (int pp = 0; pp < KP; ++pp) acc[j][pp] *= alpha;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const float w = __builtin_amdgcn_exp2f(x[u] - m_new);
          l_run[j] += w;
#pragma unroll
          for (int pp = 0; pp < KP; ++pp) acc[j][pp] += w * vv[u][pp];
        }
      }
    }
    // ---- merge: the two halves of a wave by lane exchange, the four waves through LDS
#pragma unroll
    for (int j = 0; j < GC; ++j) {
      const float m_o = __shfl_xor(m_run[j], 32, 64), l_o = __shfl_xor(l_run[j], 32, 64);
      const float m = fmaxf(m_run[j], m_o);
      // (a half-wave without rows has m = -inf and contributes nothing; the workgroup as a whole has rows)
      const float a = m_run[j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run[j] - m);
      const float b = m_o == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_o - m);
      l_run[j] = l_run[j] * a + l_o * b;
#pragma unroll
      for (int pp = 0; pp < KP; ++pp)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float o = __shfl_xor(acc[j][pp][e], 32, 64);
          acc[j][pp][e] = acc[j][pp][e] * a + o * b;
        }
      m_run[j] = m;
    }
    __syncthreads();  // (the previous pass has read its results)
    if (lane < 32) {
#pragma unroll
      for (int j = 0; j < GC; ++j) {
#pragma unroll
        for (int pp = 0; pp < KP; ++pp)
          *reinterpret_cast<f4 *>(&sm_o[wave][j][4 * l32 + 128 * pp]) = acc[j][pp];
        if (l32 == 0) {
          sm_m[wave][j] = m_run[j];
          sm_l[wave][j] = l_run[j];
        }
      }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < GC * D; idx += kThreads) {
      const int j = idx / D, d = idx % D;
      if (h0 + j >= G) continue;
      float m = -INFINITY;
#pragma unroll
      for (int w = 0; w < 4; ++w) m = fmaxf(m, sm_m[w][j]);
      float lsum = 0.f, o = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float f = sm_m[w][j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sm_m[w][j] - m);
        lsum += sm_l[w][j] * f;
        o += sm_o[w][j][d] * f;
      }
      const int head = kvh * G + h0 + j;
      const float r = o / lsum;
      if (p.direct) {
        p.out[((int64_t)qrow * p.num_heads + head) * D + d] = r;
      } else {
        const int64_t pi = ((int64_t)qrow * p.num_heads + head) * p.parts_dim + part;
        p.part_out[pi * D + d] = r;
        if (d == 0) {
          p.part_max[pi] = m * kLn2;  // natural units, as the reference's max_logits
          p.part_sum[pi] = lsum;
        }
      }
    }
  }
}

// out = sum_j tmp_j w_j / sum_j w_j, w_j = exp_sum_j exp(max_j - max) (csrc/attention/attention_kernels.cu:515-582)
__global__ void __launch_bounds__(kThreads) merge_attn_f32_kernel(F32Params p) {
  int seq, qrow, len;
  if (!query_row(p, blockIdx.y, seq, qrow, len)) return;
  const int head = blockIdx.x, D = p.head_size;
  const int parts = (len + p.part_rows - 1) / p.part_rows;
  const int64_t pi = ((int64_t)qrow * p.num_heads + head) * p.parts_dim;
  float m = -INFINITY;
  for (int j = 0; j < parts; ++j) m = fmaxf(m, p.part_max[pi + j]);
  for (int d = threadIdx.x; d < D; d += kThreads) {
    float wsum = 0.f, o = 0.f;
    for (int j = 0; j < parts; ++j) {
      const float w = p.part_sum[pi + j] * __expf(p.part_max[pi + j] - m);
      wsum += w;
      o += p.part_out[(pi + j) * D + d] * w;
    }
    p.out[((int64_t)qrow * p.num_heads + head) * D + d] = o / wsum;
  }
}

template <int KP>
void launch_a(int gc, dim3 grid, hipStream_t st, const F32Params &p) {
  switch (gc) {
    case 1: hipLaunchKernelGGL((decode_attn_f32_kernel<1, KP>), grid, dim3(kThreads), 0, st, p); break;
    case 2: hipLaunchKernelGGL((decode_attn_f32_kernel<2, KP>), grid, dim3(kThreads), 0, st, p); break;
    case 4: hipLaunchKernelGGL((decode_attn_f32_kernel<4, KP>), grid, dim3(kThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((decode_attn_f32_kernel<8, KP>), grid, dim3(kThreads), 0, st, p); break;
  }
}

}  // namespace

namespace vtkv {

// Float32 attention of `num_rows` query rows (decode: one per sequence, lengths in seq_lens; prompts: `units` with
// up to unit_tokens tokens each, num_rows = num_units * unit_tokens).  exp_sums / max_logits / tmp_out: the caller's
// buffers of the split-K interface with `max_parts` partitions of 512 rows per query row, or null: the workspace
// holds the partial results (any partition size that fits it), or nothing is needed when no query row has more
// than one partition.
int attention_f32(float *out, const float *q, const int64_t *k_ptrs, const int64_t *v_ptrs, const int64_t *slot_ids,
                  const int32_t *seq_lens, const int32_t *units, int unit_tokens, int num_rows, int num_heads,
                  int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                  const float *alibi_slopes, float *exp_sums, float *max_logits, float *tmp_out, int max_parts,
                  void *workspace, int64_t workspace_bytes, void *stream) {
  VTKV_REQUIRE(out && q && k_ptrs && v_ptrs && slot_ids && (seq_lens || units), "null argument");
  VTKV_REQUIRE(num_rows >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0,
               "num_heads %d must be a positive multiple of num_kv_heads %d", num_heads, num_kv_heads);
  VTKV_REQUIRE(head_size == 64 || head_size == 80 || head_size == 96 || head_size == 112 || head_size == 128 ||
                   head_size == 256,
               "head_size %d is not supported (64, 80, 96, 112, 128, 256)", head_size);
  VTKV_REQUIRE(q_stride >= (int64_t)num_heads * head_size && q_stride % 4 == 0 && (uintptr_t)q % 16 == 0,
               "q rows must be 16-byte aligned and at least num_heads*head_size apart");
  VTKV_REQUIRE(max_seq_len > 0, "max_seq_len must be > 0");
  VTKV_REQUIRE(num_kv_heads <= 65535, "too many kv heads");
  if (num_rows == 0) return VTKV_OK;
  F32Params p;
  p.q = q;
  p.k_ptrs = k_ptrs;
  p.v_ptrs = v_ptrs;
  p.slot_ids = slot_ids;
  p.seq_lens = seq_lens;
  p.units = units;
  p.unit_tokens = unit_tokens > 0 ? unit_tokens : 1;
  p.alibi_slopes = alibi_slopes;
  p.out = out;
  p.q_stride = q_stride;
  p.num_heads = num_heads;
  p.num_kv_heads = num_kv_heads;
  p.head_size = head_size;
  p.scale_log2 = scale * kLog2e;
  const int64_t per_part = (int64_t)num_rows * num_heads * (head_size + 2) * (int64_t)sizeof(float);  // one partition of every row
  int parts;
  if (tmp_out) {
    VTKV_REQUIRE(exp_sums && max_logits, "null argument");
    p.part_rows = 512;  // vllm/attention/ops/paged_attn.py:10
    parts = (max_seq_len + 511) / 512;
    VTKV_REQUIRE(max_parts >= parts, "%d partitions do not hold %d rows", max_parts, max_seq_len);
    p.parts_dim = max_parts;
    p.part_out = tmp_out;
    p.part_max = max_logits;
    p.part_sum = exp_sums;
    p.direct = 0;
  } else {
    // Partitions of 512 rows, smaller while that leaves the part short of workgroups, larger where the workspace
    // does not hold that many partial results.
    const int64_t cap = workspace ? workspace_bytes / per_part : 0;
    int rows = 512;
    while (rows > 64 && (int64_t)num_rows * num_kv_heads * ((max_seq_len + rows - 1) / rows) < 2048) rows /= 2;
    parts = (max_seq_len + rows - 1) / rows;
    if (parts > 1 && parts > cap) {
      if (cap < 2) {
        rows = max_seq_len;
      } else {
        rows = (int)(((int64_t)max_seq_len + cap - 1) / cap);
      }
      parts = (max_seq_len + rows - 1) / rows;
    }
    p.part_rows = rows;
    p.parts_dim = parts;
    p.direct = parts == 1;
    p.part_out = (float *)workspace;
    p.part_max = p.part_out + (int64_t)num_rows * num_heads * parts * head_size;
    p.part_sum = p.part_max + (int64_t)num_rows * num_heads * parts;
    if (!p.direct) VTKV_REQUIRE((uintptr_t)workspace % 16 == 0, "workspace must be 16-byte aligned");
  }
  VTKV_REQUIRE(parts <= 65535 * 32, "too many partitions");
  const int group = num_heads / num_kv_heads;
  const int gc = group >= 8 ? 8 : group > 2 ? 4 : group;
  hipStream_t st = (hipStream_t)stream;
  // (the grid's z extent is limited to 65 535: more query rows run as consecutive launches, of whole units)
  const int per_launch = 65535 / p.unit_tokens * p.unit_tokens;
  for (int at = 0; at < num_rows; at += per_launch) {
    F32Params pc = p;
    const int n = std::min(per_launch, num_rows - at);
    // decode rows are addressed from the start of their arrays: a launch of later rows shifts the arrays; the query
    // rows of units are named by the units themselves
    if (units) {
      pc.units = units + 4 * (int64_t)(at / p.unit_tokens);
    } else {
      pc.seq_lens = seq_lens + at;
      pc.slot_ids = slot_ids + at;
      pc.q = q + (int64_t)at * q_stride;
      pc.out = out + (int64_t)at * num_heads * head_size;
      pc.part_out = p.part_out + (int64_t)at * num_heads * p.parts_dim * head_size;
      pc.part_max = p.part_max + (int64_t)at * num_heads * p.parts_dim;
      pc.part_sum = p.part_sum + (int64_t)at * num_heads * p.parts_dim;
    }
    const dim3 grid((unsigned)parts, (unsigned)num_kv_heads, (unsigned)n);
    if (head_size > 128)
      launch_a<2>(gc, grid, st, pc);
    else
      launch_a<1>(gc, grid, st, pc);
    if (!pc.direct)
      hipLaunchKernelGGL(merge_attn_f32_kernel, dim3((unsigned)num_heads, (unsigned)n), dim3(kThreads), 0, st, pc);
  }
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

}  // namespace vtkv
