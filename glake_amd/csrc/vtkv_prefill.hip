// Prompt (prefill) attention over per-sequence contiguous KV ranges for gfx950, bf16 or fp8-e4m3 cache.
//
// The query token at position t of its sequence attends to rows 0..t of the sequence's K and V
// ranges, which already hold the prompt's own rows.  Unlike decode this is not bound by HBM: a block
// of query tokens reuses every K/V row it reads, so the kernel is organised around reuse.
//
//  * A workgroup (four wave64) takes one unit = up to 128/G consecutive query tokens of one sequence
//    and one kv head, i.e. 128 columns (token, head of the group); a wave owns 32 of them as two
//    blocks of 16 and walks over ALL rows its columns may see, so there is nothing to merge at the end.
//  * K and V rows are loaded once per workgroup, 32 rows at a time, as whole rows with ordinary
//    (cached) loads into a double-buffered LDS stage in the swizzled tile layouts of the decode kernel;
//    every wave reads each 16-row tile from LDS once and uses it for both of its column blocks.
//  * S^T = K_tile . Q^T and O^T += V_tile^T . P^T run on v_mfma_f32_16x16x32_bf16 exactly as in the
//    decode kernel (P as bf16 head + tail in one K=32 MFMA, softmax statistics in registers, online
//    rescale), with each lane applying its column's causal limit to the logits of the tiles that reach it.
//  * The kv head is the fastest index of the grid: with 8 kv heads the workgroups of one kv head all land
//    on one XCD, whose L2 then serves the re-reads of that head's rows by later query blocks.
//
//  * fp8 cache: rows are e4m3fn codes (128 bytes per head row); they are widened to bf16 (exactly) on the
//    way into the LDS stage, so everything after the stage is the bf16 kernel; the K scale folds into the
//    logit scale and the V scale into the final normalisation.
//
// Numerics as in the decode kernel (vtkv_attention.hip); the reference computes this with xformers /
// an external flash-attention kernel (vllm/attention/backends/xformers.py:331-386).
#include "vtkv_attn_common.h"
#include "vtkv_common.h"

namespace {

using namespace vtkv_attn;

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
#ifndef VTKV_PREFILL_NB
#define VTKV_PREFILL_NB 2
#endif
#ifndef VTKV_PREFILL_KEYS
#define VTKV_PREFILL_KEYS 32
#endif
constexpr int kNB = VTKV_PREFILL_NB;          // column blocks of 16 per wave
constexpr int kCols = kWaves * kNB * 16;      // columns per workgroup
constexpr int kKeyBlock = VTKV_PREFILL_KEYS;  // rows per LDS stage (32 or 64)
static_assert(kKeyBlock == 32 || kKeyBlock == 64, "the stage loads cover 32 or 64 rows");
constexpr int kSub = kKeyBlock / kTile;       // 16-row tiles per stage
constexpr int kStageBytes = 2 * kKeyBlock * kRowBytes;  // K then V

struct PrefillParams {
  const uint16_t *q;
  const int64_t *k_ptrs, *v_ptrs, *slot_ids;
  const int32_t *units;  // [n][4] = {sequence, first query row, query tokens, position of the first}
  const float *alibi_slopes;
  void *out;
  int out_f32;
  int64_t q_stride;
  int num_heads, num_kv_heads, group;
  float scale_log2;  // scale * log2(e) [* k_scale for an fp8 cache]
  float v_scale;     // 1 for a bf16 cache
};

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

template <bool ALIBI, bool FP8>
__global__ void __launch_bounds__(kThreads) prefill_attn_kernel(PrefillParams p) {
  __shared__ __attribute__((aligned(16))) char smem[2 * kStageBytes];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int g = lane >> 4, n = lane & 15;
  const int G = p.group, Hkv = p.num_kv_heads;
  const int kvh = blockIdx.x % Hkv;
  const int unit = blockIdx.x / Hkv;
  const int u_seq = uniform(p.units[4 * unit]);
  const int u_row0 = uniform(p.units[4 * unit + 1]);
  const int u_ntok = uniform(p.units[4 * unit + 2]);
  const int u_pos0 = uniform(p.units[4 * unit + 3]);
  const int kv_len = u_pos0 + u_ntok;  // rows the unit's last token sees

  typedef const __attribute__((address_space(1))) char *gptr;
  typedef const __attribute__((address_space(1))) u32x4 *gvec;
  const int64_t slot = p.slot_ids[u_seq];
  constexpr int kKvRowBytes = FP8 ? kD : kRowBytes;  // bytes of one head row in the cache
  gptr k_base = (gptr)(uintptr_t)p.k_ptrs[slot] + kvh * kKvRowBytes;
  gptr v_base = (gptr)(uintptr_t)p.v_ptrs[slot] + kvh * kKvRowBytes;
  const uint32_t row_stride = (uint32_t)Hkv * kKvRowBytes;

  // ---- this wave's columns: block nb, column n -> (token, head); unused columns get q = 0
  bf16x8 qop[kNB][4];
  int limit[kNB];       // rows below this are visible to the lane's column
  int col_tok[kNB], col_head[kNB];
  float slope_log2[kNB];
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    const int c = (wave * kNB + nb) * 16 + n;
    const int tok = c / G, head = c % G;
    const bool valid = tok < u_ntok;
    col_tok[nb] = valid ? tok : -1;
    col_head[nb] = head;
    limit[nb] = valid ? u_pos0 + tok + 1 : 0x7fffffff;
    slope_log2[nb] = ALIBI && valid ? p.alibi_slopes[kvh * G + head] * kLog2e : 0.f;
    const uint16_t *qrow = p.q + (int64_t)(u_row0 + (valid ? tok : 0)) * p.q_stride + (int64_t)(kvh * G + head) * kD;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 raw = *reinterpret_cast<const u32x4 *>(qrow + ks * 32 + g * 8);
      if (!valid) raw = (u32x4){0, 0, 0, 0};
      qop[nb][ks] = __builtin_bit_cast(bf16x8, raw);
    }
  }
  // rows this wave needs: up to the limit of its last used column; its first column's limit says from
  // which tile on the mask matters
  const int tok_lo = (wave * kNB * 16) / G, tok_hi = ((wave + 1) * kNB * 16 - 1) / G;
  const int wave_end = tok_lo < u_ntok ? u_pos0 + min(tok_hi, u_ntok - 1) + 1 : 0;  // 0: no column in use
  const int wave_first_limit = u_pos0 + tok_lo + 1;

  f32x4 acc[kNB][8];
  float m_run[kNB], l_run[kNB];
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    m_run[nb] = -INFINITY;
    l_run[nb] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[nb][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // ---- cooperative stage loads of a block of kKeyBlock rows.  bf16 rows: thread t takes piece t%16 of
  // rows t/16 + 16j.  fp8 rows have 8 pieces of 16 codes: thread t takes piece t%8 of rows t/8 + 32j and
  // widens it to two bf16 pieces on the way into LDS.
  constexpr int kLd = FP8 ? kKeyBlock / 32 : kKeyBlock / 16;
  const int ld_piece = FP8 ? threadIdx.x & 7 : threadIdx.x & 15, ld_row = FP8 ? threadIdx.x >> 3 : threadIdx.x >> 4;
  const int nblocks = (kv_len + kKeyBlock - 1) / kKeyBlock;
  u32x4 kst[kLd], vst[kLd];
  auto gload = [&](int kb) {
#pragma unroll
    for (int j = 0; j < kLd; ++j) {
      // rows past the end are redirected to the last row; they are masked for every column in use
      const int row = min(kb * kKeyBlock + j * (kKeyBlock / kLd) + ld_row, kv_len - 1);
      const int64_t off = (int64_t)row * row_stride + ld_piece * 16;
      kst[j] = *(gvec)(k_base + off);
      vst[j] = *(gvec)(v_base + off);
    }
  };
  auto lstore = [&](int buf) {
    char *kb_ = smem + buf * kStageBytes, *vb_ = kb_ + kKeyBlock * kRowBytes;
#pragma unroll
    for (int j = 0; j < kLd; ++j) {
      if constexpr (FP8) {
        const int row = j * 32 + ld_row, tile = row >> 4, r = row & 15;
        char *kt = kb_ + tile * kTile * kRowBytes, *vt = vb_ + tile * kTile * kRowBytes;
        *reinterpret_cast<u32x4 *>(kt + k_lds_offset(r, 2 * ld_piece)) = fp8x8_to_bf16x8(kst[j][0], kst[j][1]);
        *reinterpret_cast<u32x4 *>(kt + k_lds_offset(r, 2 * ld_piece + 1)) = fp8x8_to_bf16x8(kst[j][2], kst[j][3]);
        *reinterpret_cast<u32x4 *>(vt + v_lds_offset(r, 2 * ld_piece)) = fp8x8_to_bf16x8(vst[j][0], vst[j][1]);
        *reinterpret_cast<u32x4 *>(vt + v_lds_offset(r, 2 * ld_piece + 1)) = fp8x8_to_bf16x8(vst[j][2], vst[j][3]);
      } else {
        *reinterpret_cast<u32x4 *>(kb_ + j * kTile * kRowBytes + k_lds_offset(ld_row, ld_piece)) = kst[j];
        *reinterpret_cast<u32x4 *>(vb_ + j * kTile * kRowBytes + v_lds_offset(ld_row, ld_piece)) = vst[j];
      }
    }
  };

  gload(0);
  lstore(0);
  __syncthreads();
  for (int kb = 0; kb < nblocks; ++kb) {
    gload(min(kb + 1, nblocks - 1));  // always issued: the last block is loaded once more and not used
    const char *kstage = smem + (kb & 1) * kStageBytes, *vstage = kstage + kKeyBlock * kRowBytes;
    for (int sub = 0; sub < kSub; ++sub) {
      const int t0 = kb * kKeyBlock + sub * kTile;
      if (t0 >= wave_end) break;  // wave-uniform: nothing this wave's columns may see
      const char *k_tile = kstage + sub * kTile * kRowBytes, *v_tile = vstage + sub * kTile * kRowBytes;
      // A operand of S^T = K.Q^T: lane (n, g) takes row n, bytes [16g, +16) of each 64-byte quarter
      u32x4 ka[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) ka[c] = *reinterpret_cast<const u32x4 *>(k_tile + k_lds_offset(n, 4 * c + g));
      const bool masked = t0 + kTile > wave_first_limit;  // wave-uniform: the tile reaches some column's limit
      // Order within the tile: all S MFMAs first, then per column block its softmax followed by its P.V
      // MFMAs, so that the matrix pipe works on one block's P.V while the vector unit does the next
      // block's softmax.
      f32x4 sacc[kNB];
#pragma unroll
      for (int nb = 0; nb < kNB; ++nb) {
        sacc[nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
          sacc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ka[ks]), qop[nb][ks], sacc[nb], 0,
                                                             0, 0);
      }
      // transposed V operands, read once for both column blocks
      u32x4 vop[8];
      {
        const int row = 4 * g + (n >> 2);
        const int base = row * kRowBytes + ((n & 1) << 3);
        const int swz = (row & 7) << 1;
#pragma unroll
        for (int db = 0; db < 8; ++db) {
          const int off = base + (((2 * db + ((n >> 1) & 1)) ^ swz) << 4);
          const s16x4 quad =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(v_tile + off));
          const u32x2 qd = __builtin_bit_cast(u32x2, quad);
          vop[db] = (u32x4){qd[0], qd[1], qd[0], qd[1]};
        }
      }
#pragma unroll
      for (int nb = 0; nb < kNB; ++nb) {
        const f32x4 s = sacc[nb];
        float x[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          x[r] = s[r] * p.scale_log2;
          if (ALIBI) x[r] += slope_log2[nb] * (float)(t0 + 4 * g + r - limit[nb] + 1);
        }
        if (masked) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (t0 + 4 * g + r >= limit[nb]) x[r] = -INFINITY;
        }
        const float tmax = max_over_row_groups(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])));
        // The reference point of the exponentials only follows the running maximum when that has grown by
        // more than 8 (a factor 256 in the weights, harmless in fp32): the rescale of the accumulators,
        // which otherwise runs whenever any of the wave's 32 columns sees a new maximum, becomes rare.
        const float m_new = tmax > m_run[nb] + 8.f ? tmax : m_run[nb];
        // (a column can have a whole tile masked; the reference point 0 keeps exp2(-inf - ref) = 0)
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[nb] - m_ref);
        m_run[nb] = m_new;
        float pr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pr[r] = __builtin_amdgcn_exp2f(x[r] - m_ref);
        l_run[nb] = l_run[nb] * alpha + ((pr[0] + pr[1]) + (pr[2] + pr[3]));
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
          for (int d = 0; d < 8; ++d) acc[nb][d] *= alpha;
        }
        // P^T as a bf16 head plus a bf16 tail in the two halves of the K=32 reduction (as in decode)
        float plo[4];
        u32x4 pb;
        pb[0] = pack_bf16x2(pr[0], pr[1]);
        pb[1] = pack_bf16x2(pr[2], pr[3]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const unsigned hi_bits = (r & 1) ? (pb[r >> 1] & 0xffff0000u) : (pb[r >> 1] << 16);
          plo[r] = pr[r] - __builtin_bit_cast(float, hi_bits);
        }
        pb[2] = pack_bf16x2(plo[0], plo[1]);
        pb[3] = pack_bf16x2(plo[2], plo[3]);
        const bf16x8 pop = __builtin_bit_cast(bf16x8, pb);
#pragma unroll
        for (int db = 0; db < 8; ++db)
          acc[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vop[db]), pop, acc[nb][db], 0,
                                                                0, 0);
      }
    }
    lstore((kb + 1) & 1);  // nobody reads that stage: its readers finished before the last barrier
    __syncthreads();
  }

  // ---- normalise and store: lane (n, g) holds O[column n][d = 16*db + 4g + i]
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    const float l = sum_over_row_groups(l_run[nb]);
    if (col_tok[nb] < 0) continue;
    const float inv = p.v_scale / l;
    const int64_t o0 = ((int64_t)(u_row0 + col_tok[nb]) * p.num_heads + kvh * G + col_head[nb]) * kD + 4 * g;
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const f32x4 r = acc[nb][db] * inv;
      if (p.out_f32) {
        *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.out) + o0 + db * 16) = r;
      } else {
        u32x2 w = {pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
        *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(p.out) + o0 + db * 16) = w;
      }
    }
  }
}

}  // namespace

extern "C" {

int vtkv_prefill_unit_tokens(int num_heads, int num_kv_heads, int kv_dtype) {
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0) return 0;
  const int group = num_heads / num_kv_heads;
  if (group > 16) return 0;
  (void)kv_dtype;  // the same kernel serves both cache types
  return kCols / group;
}

int vtkv_prefill_attention(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                           const int64_t *slot_ids, const int32_t *units, int num_units, int num_heads,
                           int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                           const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                           float v_scale, void *stream) {
  VTKV_REQUIRE(out && q && k_ptrs && v_ptrs && slot_ids && units, "null argument");
  VTKV_REQUIRE(num_units >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0,
               "num_heads %d must be a positive multiple of num_kv_heads %d", num_heads, num_kv_heads);
  VTKV_REQUIRE(head_size == kD, "head_size %d is not supported (only 128)", head_size);
  VTKV_REQUIRE(q_dtype == VTKV_BF16, "q_dtype must be BF16");
  VTKV_REQUIRE(out_dtype == VTKV_BF16 || out_dtype == VTKV_F32, "out_dtype must be BF16 or F32");
  VTKV_REQUIRE(kv_dtype == VTKV_BF16 || kv_dtype == VTKV_FP8_E4M3, "kv_dtype must be BF16 or FP8_E4M3");
  const bool fp8 = kv_dtype == VTKV_FP8_E4M3;
  if (fp8) VTKV_REQUIRE(k_scale > 0.f && v_scale > 0.f, "fp8 scales must be positive");
  const int group = num_heads / num_kv_heads;
  VTKV_REQUIRE(group <= 16, "num_heads/num_kv_heads = %d exceeds 16", group);
  VTKV_REQUIRE(q_stride >= (int64_t)num_heads * head_size && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
                   (uintptr_t)out % 16 == 0,
               "q rows must be 16-byte aligned and at least num_heads*head_size apart");
  VTKV_REQUIRE(max_seq_len > 0 && (int64_t)max_seq_len * num_kv_heads * head_size * 2 < (1ll << 40), "bad max_seq_len");
  VTKV_REQUIRE((int64_t)num_units * num_kv_heads < (1ll << 31), "too many units");
  if (num_units == 0) return VTKV_OK;
  PrefillParams p;
  p.q = (const uint16_t *)q;
  p.k_ptrs = k_ptrs;
  p.v_ptrs = v_ptrs;
  p.slot_ids = slot_ids;
  p.units = units;
  p.alibi_slopes = alibi_slopes;
  p.out = out;
  p.out_f32 = out_dtype == VTKV_F32;
  p.q_stride = q_stride;
  p.num_heads = num_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = group;
  p.scale_log2 = scale * kLog2e * (fp8 ? k_scale : 1.f);
  p.v_scale = fp8 ? v_scale : 1.f;
  const dim3 grid((unsigned)((int64_t)num_units * num_kv_heads)), block(kThreads);
  hipStream_t st = (hipStream_t)stream;
  if (alibi_slopes && fp8)
    hipLaunchKernelGGL((prefill_attn_kernel<true, true>), grid, block, 0, st, p);
  else if (alibi_slopes)
    hipLaunchKernelGGL((prefill_attn_kernel<true, false>), grid, block, 0, st, p);
  else if (fp8)
    hipLaunchKernelGGL((prefill_attn_kernel<false, true>), grid, block, 0, st, p);
  else
    hipLaunchKernelGGL((prefill_attn_kernel<false, false>), grid, block, 0, st, p);
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

}  // extern "C"
