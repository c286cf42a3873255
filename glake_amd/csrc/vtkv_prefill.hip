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
//  * S^T = K_tile . Q^T runs on v_mfma_f32_16x16x32_bf16 as in the decode kernel.  O^T += V^T . P^T runs
//    on v_mfma_f32_16x16x32_f16 over the stage's 32 rows at once: V is converted to fp16 on its way into
//    LDS and the softmax weights are rounded to fp16 (2^-12 relative per weight, 16 times finer than the
//    bf16 weights of flash-attention kernels; the decode kernel's bf16 head + tail is finer still but costs
//    twice the P.V MFMAs).  bf16 V values convert exactly for magnitudes in [2^-24, 65504]; smaller ones
//    lose low bits (absolute error below 2^-25); a larger one becomes infinity, the workgroup finds its
//    result non-finite at the end and computes the unit a second time with V kept in bf16 and the decode
//    kernel's bf16 head + tail of P, so prompt and decode attention agree for every bf16 input.  Softmax
//    statistics live in registers, each lane applies its column's causal limit to the logits of the stages
//    that reach it.
//  * The kv head is the fastest index of the grid: with 8 kv heads the workgroups of one kv head all land
//    on one XCD, whose L2 then serves the re-reads of that head's rows by later query blocks.
//
//  * fp8 cache: rows are e4m3fn codes (128 bytes per head row); on the way into the LDS stage K is widened
//    to bf16 and V to fp16 (both exactly), so everything after the stage is the bf16 kernel; the K scale
//    folds into the logit scale and the V scale into the final normalisation.
//
// Otherwise numerics as in the decode kernel (vtkv_attention.hip); the reference computes this with xformers /
// an external flash-attention kernel (vllm/attention/backends/xformers.py:331-386).
#include "vtkv_attn_common.h"
#include "vtkv_common.h"

#include <type_traits>

#ifdef VTKV_PREFILL_TRACE
// Tuning builds only: per workgroup of the last launch {XCC id, start, first stage in LDS, end of the stages, end,
// stages} on the 100 MHz wall clock.
__device__ unsigned long long g_prefill_trace[4096][6];
#endif

namespace {

using namespace vtkv_attn;

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
#ifndef VTKV_PREFILL_NB
#define VTKV_PREFILL_NB 2
#endif

constexpr int kNB = VTKV_PREFILL_NB;          // column blocks of 16 per wave (one for head sizes above 128)
constexpr int kKeyBlock = 32;                 // rows per LDS stage = rows of one P.V reduction (two 16-row tiles)
constexpr int col_blocks(int head_size) { return head_size > 128 ? 1 : kNB; }
constexpr int cols_per_group(int head_size) { return kWaves * col_blocks(head_size) * 16; }  // columns per workgroup

struct PrefillParams {
  const uint16_t *q;
  const int64_t *k_ptrs, *v_ptrs, *slot_ids;
  const int32_t *units;  // [n][4] = {sequence, first query row, query tokens, position of the first}
  const float *alibi_slopes;
  void *out;
  int out_f32;
  int64_t q_stride;
  int num_heads, num_kv_heads, group;  // (kv heads and heads of each as the kernel sees them: see first_head_of)
  int kv_split, group_real;
  float scale_log2;  // scale * log2(e) [* k_scale for an fp8 cache]
  float v_scale;     // 1 for a bf16 cache
};

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// Two floats to two fp16 in one register, round to nearest; a value beyond the fp16 range becomes infinity.
__device__ __forceinline__ unsigned pack_f16x2(float a, float b) {
  f16x2 v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(unsigned, v);
}
// Maxima as single instructions.  fmaxf() first quiets its operands (one more instruction each) wherever the
// compiler cannot prove them canonical, which it cannot after selects and lane swaps.
__device__ __forceinline__ float fmax2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float fmax3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// Maximum over the four row groups of a column: lanes n, n+16, n+32, n+48.
__device__ __forceinline__ float wave_max_over_row_groups(float v) {
  float a, b;
  swap_rows16(v, a, b);
  swap_rows32(fmax2(a, b), a, b);
  return fmax2(a, b);
}
// Eight bf16 values (one 16-byte piece of a V row) to eight fp16 values.  Exact for magnitudes in
// [2^-24, 65504]; a larger one becomes infinity, which makes the unit's result non-finite: the kernel sees that
// at the end and computes the unit again with V kept in bf16 (see WIDE).
__device__ __forceinline__ u32x4 bf16x8_to_f16x8(u32x4 v) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    r[i] = pack_f16x2(__builtin_bit_cast(float, v[i] << 16), __builtin_bit_cast(float, v[i] & 0xffff0000u));
  return r;
}
// F16: queries, rows and output are fp16 instead of bf16 (rows may still be e4m3fn codes).  S runs on the fp16
// MFMA and V needs no conversion on its way into LDS; nothing can leave the fp16 range, so there is no second pass.
// HS: the head size, 64, 80, 96, 112, 128 or 256.  The kernel was shaped for 128, where every constant below has
// the value it always had.  K rows are held in LDS padded to the MFMA depth of 32 (80 as 96, 112 as 128; the pad
// is cleared once and q is zero there); V and the output need no padding, every size being a multiple of 16.
// Above 128 a wave owns one block of 16 columns instead of two.
template <bool ALIBI, bool FP8, bool F16 = false, int HS = 128>
__global__ void __launch_bounds__(kThreads) prefill_attn_kernel(PrefillParams p) {
  constexpr int kD = HS;                              // (shadows the library-wide 128 inside this kernel)
  constexpr int kHD = (HS + 31) / 32 * 32;            // K row as held in LDS
  constexpr int kRowBytes = kHD * 2 < 256 ? 256 : kHD * 2;  // LDS pitch of a row (16-bit elements)
  constexpr int kKS = kHD / 32;                       // MFMA steps over d of S
  constexpr int kDB = HS / 16;                        // blocks of 16 output columns
  constexpr int kNB = col_blocks(HS);
  constexpr int kStageBytes = 2 * kKeyBlock * kRowBytes;  // K then V
  auto k_lds_offset = [](int row, int piece16) { return row * kRowBytes + ((piece16 ^ (row & 15)) << 4); };
  auto v_lds_offset = [](int row, int piece16) { return row * kRowBytes + ((piece16 ^ ((row & 7) << 1)) << 4); };
  __shared__ __attribute__((aligned(16))) char smem[2 * kStageBytes];
#ifdef VTKV_PREFILL_TRACE
  const unsigned long long trace_t0 = wall_clock64();
  unsigned long long trace_t1 = 0;
#endif
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
  constexpr int kKvRowBytes = FP8 ? kD : 2 * kD;  // bytes of one head row in the cache
  const int kv_real = real_kv_head(p, kvh);  // whose rows this workgroup reads
  gptr k_base = (gptr)(uintptr_t)p.k_ptrs[slot] + kv_real * kKvRowBytes;
  gptr v_base = (gptr)(uintptr_t)p.v_ptrs[slot] + kv_real * kKvRowBytes;
  const uint32_t row_stride = (uint32_t)(Hkv / p.kv_split) * kKvRowBytes;
  const int head0 = first_head_of(p, kvh), n_heads = heads_of(p, kvh);

  // ---- this wave's columns: block nb, column n -> (token, head); unused columns get q = 0
  u32x4 qop[kNB][kKS];
  int limit[kNB];       // rows below this are visible to the lane's column
  int col_tok[kNB], col_head[kNB];
  float slope_log2[kNB];
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    const int c = (wave * kNB + nb) * 16 + n;
    const int tok = c / G, head = c % G;
    const bool valid = tok < u_ntok && head < n_heads;
    col_tok[nb] = valid ? tok : -1;
    col_head[nb] = head;
    limit[nb] = valid ? u_pos0 + tok + 1 : 0x7fffffff;
    slope_log2[nb] = ALIBI && valid && p.alibi_slopes ? p.alibi_slopes[head0 + head] * kLog2e : 0.f;
    const uint16_t *qrow =
        p.q + (int64_t)(u_row0 + (valid ? tok : 0)) * p.q_stride + (int64_t)(head0 + (valid ? head : 0)) * kD;
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
      u32x4 raw = (u32x4){0, 0, 0, 0};
      if (kHD == kD || ks * 32 + g * 8 < kD) raw = *reinterpret_cast<const u32x4 *>(qrow + ks * 32 + g * 8);
      if (!valid) raw = (u32x4){0, 0, 0, 0};
      qop[nb][ks] = raw;
    }
  }
  // rows this wave needs: up to the limit of its last used column; its first column's limit says from
  // which tile on the mask matters
  const int tok_lo = (wave * kNB * 16) / G, tok_hi = ((wave + 1) * kNB * 16 - 1) / G;
  const int wave_end = tok_lo < u_ntok ? u_pos0 + min(tok_hi, u_ntok - 1) + 1 : 0;  // 0: no column in use
  const int wave_first_limit = u_pos0 + tok_lo + 1;

  f32x4 acc[kNB][kDB];
  // The normaliser of a column is one more row of its output: P^T times a column of ones, accumulated by the matrix
  // pipe like the others (every lane of the column ends up with the whole sum in each of its four slots), instead
  // of a chain of vector additions per stage.  m_off: what the exponent's fused multiply-add subtracts, kept with
  // the reference point it follows.
  f32x4 acc_l[kNB];
  float m_run[kNB], m_off[kNB];
  auto reset = [&]() {
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      m_run[nb] = -INFINITY;
      m_off[nb] = 0.f;
      acc_l[nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < kDB; ++i) acc[nb][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  };
  reset();

  // ---- cooperative stage loads of a block of kKeyBlock rows.  The 16-byte pieces of the block (kGp per row:
  // 16 for a bf16 row of 128, 8 for its fp8 codes) are dealt to the threads in order, piece 256 j + t to load j
  // of thread t; an fp8 piece carries 16 codes and is widened to two 16-bit pieces on the way into LDS.  A
  // thread's byte offset into the K range is also its offset into the V range; it advances by 32 rows per
  // stage and is clamped to the same piece of the last row (rows past the end are masked for every column in
  // use, so any finite in-bounds data will do).  Where the pieces do not fill the last load, its idle threads
  // fetch a piece again and store nothing.
  constexpr int kGp = FP8 ? kD / 16 : kD / 8;
  constexpr int kStagePieces = kKeyBlock * kGp;
  constexpr int kLd = (kStagePieces + kThreads - 1) / kThreads;
  constexpr bool kEvenLd = kStagePieces % kThreads == 0;
  int ld_row[kLd], ld_piece[kLd];
  bool ld_live[kLd];
#pragma unroll
  for (int j = 0; j < kLd; ++j) {
    const int idx = j * kThreads + (int)threadIdx.x;
    ld_live[j] = kEvenLd || idx < kStagePieces;
    ld_row[j] = ld_live[j] ? idx / kGp : 0;
    ld_piece[j] = ld_live[j] ? idx % kGp : 0;
  }
  const int nblocks = (kv_len + kKeyBlock - 1) / kKeyBlock;
  const uint32_t stage_step = kKeyBlock * row_stride;
  uint32_t ld_off[kLd], last_off[kLd];
#pragma unroll
  for (int j = 0; j < kLd; ++j) last_off[j] = (uint32_t)(kv_len - 1) * row_stride + ld_piece[j] * 16;
  auto rewind = [&]() {
#pragma unroll
    for (int j = 0; j < kLd; ++j) ld_off[j] = (uint32_t)ld_row[j] * row_stride + ld_piece[j] * 16;
  };
  rewind();
  u32x4 kst[kLd], vst[kLd];
  auto gload = [&]() {  // loads the next stage's rows and moves on
#pragma unroll
    for (int j = 0; j < kLd; ++j) {
      const uint32_t off = min(ld_off[j], last_off[j]);
      kst[j] = *(gvec)(k_base + off);
      vst[j] = *(gvec)(v_base + off);
      ld_off[j] += stage_step;
    }
  };
  if constexpr (kHD != kD) {
    // the pad pieces of the K rows of both stages: cleared once, no load ever writes them
    constexpr int kPad = (kHD - kD) / 8;
    for (int i = threadIdx.x; i < 2 * kKeyBlock * kPad; i += kThreads) {
      const int buf = i / (kKeyBlock * kPad), rem = i % (kKeyBlock * kPad), row = rem / kPad, pp = kD / 8 + rem % kPad;
      *reinterpret_cast<u32x4 *>(smem + buf * kStageBytes + (row >> 4) * kTile * kRowBytes + k_lds_offset(row & 15, pp)) =
          (u32x4){0, 0, 0, 0};
    }
  }
  // LDS byte offsets that do not depend on the stage, so that the stage's buffer and tile add as immediates
  int st_k[kLd], st_v[kLd];  // where lstore puts this thread's pieces (fp8: the first of each pair)
#pragma unroll
  for (int j = 0; j < kLd; ++j) {
    const int tile = ld_row[j] >> 4, r = ld_row[j] & 15, lp = FP8 ? 2 * ld_piece[j] : ld_piece[j];
    st_k[j] = tile * kTile * kRowBytes + k_lds_offset(r, lp);
    st_v[j] = kKeyBlock * kRowBytes + tile * kTile * kRowBytes + v_lds_offset(r, lp);
  }
  // WIDE (bf16 rows only): V stays bf16 in LDS and P.V runs on the bf16 MFMA with P as a bf16 head plus a bf16
  // tail, the decode kernel's arithmetic: twice the P.V MFMAs, no limit on |V|.  Used for a unit's second pass.
  auto lstore = [&](auto bufc, auto widec) {
    constexpr bool WIDE = decltype(widec)::value;
    char *base = smem + decltype(bufc)::value * kStageBytes;
#pragma unroll
    for (int j = 0; j < kLd; ++j) {
      if (!ld_live[j]) continue;
      if constexpr (FP8) {
        // pieces 2p and 2p+1 of a row sit 16 bytes apart before the swizzle, which flips bit 4 or leaves it
        *reinterpret_cast<u32x4 *>(base + st_k[j]) = fp8x8_widen<F16>(kst[j][0], kst[j][1]);
        *reinterpret_cast<u32x4 *>(base + (st_k[j] ^ 16)) = fp8x8_widen<F16>(kst[j][2], kst[j][3]);
        *reinterpret_cast<u32x4 *>(base + st_v[j]) = fp8x8_to_f16x8(vst[j][0], vst[j][1]);
        *reinterpret_cast<u32x4 *>(base + (st_v[j] ^ 16)) = fp8x8_to_f16x8(vst[j][2], vst[j][3]);
      } else {
        *reinterpret_cast<u32x4 *>(base + st_k[j]) = kst[j];
        *reinterpret_cast<u32x4 *>(base + st_v[j]) = (WIDE || F16) ? vst[j] : bf16x8_to_f16x8(vst[j]);
      }
    }
  };
  // A operands of S^T = K.Q^T: lane (n, g) takes row n, bytes [16g, +16) of each 64-byte quarter c
  int ka_off[kKS];
#pragma unroll
  for (int c = 0; c < kKS; ++c) ka_off[c] = k_lds_offset(n, 4 * c + g);
  // A operands of O^T += V^T.P^T: the lane's transposed quad of dims [16db, +16)
  int vq_off[kDB];
  {
    const int row = 4 * g + (n >> 2);
    const int base = kKeyBlock * kRowBytes + row * kRowBytes + ((n & 1) << 3);
    const int swz = (row & 7) << 1;
#pragma unroll
    for (int db = 0; db < kDB; ++db) vq_off[db] = base + (((2 * db + ((n >> 1) & 1)) ^ swz) << 4);
  }
  const float sl = p.scale_log2;
  // The reference point of the exponentials only follows the running maximum when that has grown by more
  // than 8 in log2 units (a factor 256 in the weights, harmless in fp32 and fp16): the rescale of the
  // accumulators, which otherwise runs whenever any of the wave's 32 columns sees a new maximum, becomes
  // rare.  Without ALiBi the maximum is tracked on the raw dot products (the scale is positive) and the
  // scale is applied inside the exponent's fused multiply-add.
  const float lazy = ALIBI ? 8.f : 8.f / sl;

  auto stage = [&](auto bufc, auto widec, int kb) {
    constexpr int buf = decltype(bufc)::value;
    constexpr bool WIDE = decltype(widec)::value;
    gload();  // always issued: past the last stage it re-reads the last row and nobody uses it
    const char *st = smem + buf * kStageBytes;
    const int t0 = kb * kKeyBlock;
    if (t0 < wave_end) {  // wave-uniform: else nothing this wave's columns may see
      u32x4 ka[2][kKS];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c = 0; c < kKS; ++c)
          ka[t][c] = *reinterpret_cast<const u32x4 *>(st + t * kTile * kRowBytes + ka_off[c]);
      const bool masked = t0 + kKeyBlock > wave_first_limit;  // wave-uniform: the stage reaches some column's limit
      // all S MFMAs first, then per column block its softmax followed by its P.V MFMAs, so that the matrix
      // pipe works on one block's P.V while the vector unit does the next block's softmax
      f32x4 sacc[kNB][2];
      // The S MFMAs of a stage head a chain everything else of the stage hangs on: they are issued at raised
      // priority, ahead of the other wave of the SIMD, which is mostly in its softmax (2 to 3 % per launch; the
      // other way round, softmax and P.V raised, changes nothing).
      __builtin_amdgcn_s_setprio(3);
#pragma unroll
      for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          sacc[nb][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < kKS; ++ks)
            sacc[nb][t] = mfma_16x16x32<F16>(ka[t][ks], qop[nb][ks], sacc[nb][t]);
        }
      // reduction slot (g, j) of the K=32 P.V MFMA stands for row 4g+j of the first tile (j < 4) and row
      // 4g+j-4 of the second (j >= 4), so a lane's A operand is its transposed quad of the first tile
      // followed by that of the second; read once for both column blocks
      __builtin_amdgcn_s_setprio(0);
      u32x4 vop[kDB];
#pragma unroll
      for (int db = 0; db < kDB; ++db) {
        const u32x2 qa = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                                       (__attribute__((address_space(3))) s16x4 *)(st + vq_off[db])));
        const u32x2 qb = __builtin_bit_cast(
            u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                       (__attribute__((address_space(3))) s16x4 *)(st + kTile * kRowBytes + vq_off[db])));
        vop[db] = (u32x4){qa[0], qa[1], qb[0], qb[1]};
      }
#pragma unroll
      for (int nb = 0; nb < kNB; ++nb) {
        // x[4t + r] belongs to row t0 + 16t + 4g + r of the lane's column: with ALiBi the logit in log2
        // units, else the raw dot product
        float x[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if (ALIBI)
              x[4 * t + r] = __builtin_fmaf(sacc[nb][t][r], sl,
                                            slope_log2[nb] * (float)(t0 + 16 * t + 4 * g + r - limit[nb] + 1));
            else
              x[4 * t + r] = sacc[nb][t][r];
          }
        if (masked) {
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (t0 + 16 * t + 4 * g + r >= limit[nb]) x[4 * t + r] = -INFINITY;
        }
        // the lane's own maximum; the maximum of the column (its four row groups) is only needed when some lane
        // sees a value above the reference point's margin, which is exactly when the column's maximum is above it
        const float lmax = fmax2(fmax3(x[0], x[1], x[2]), fmax3(fmax3(x[3], x[4], x[5]), x[6], x[7]));
        if (__builtin_amdgcn_ballot_w64(lmax > m_run[nb] + lazy) != 0) {  // rare: some column moves its reference point
          const float tmax = wave_max_over_row_groups(lmax);
          const bool grow = tmax > m_run[nb] + lazy;
          const float m_new = grow ? tmax : m_run[nb];
          // (a column that has seen only masked rows keeps -inf and rescales its zeros by 1)
          const float alpha = grow ? __builtin_amdgcn_exp2f(ALIBI ? m_run[nb] - m_new : (m_run[nb] - m_new) * sl) : 1.f;
          m_run[nb] = m_new;
          // (a column can have everything so far masked; the reference point 0 keeps exp2(-inf - ref) = 0)
          const float m_ref = m_new == -INFINITY ? 0.f : m_new;
          m_off[nb] = ALIBI ? -m_ref : -m_ref * sl;
          acc_l[nb] *= alpha;
#pragma unroll
          for (int d = 0; d < kDB; ++d) acc[nb][d] *= alpha;
        }
        float pr[8];
        if (ALIBI) {
#pragma unroll
          for (int r = 0; r < 8; ++r) pr[r] = __builtin_amdgcn_exp2f(x[r] + m_off[nb]);
        } else {
#pragma unroll
          for (int r = 0; r < 8; ++r) pr[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[r], sl, m_off[nb]));
        }
        // P^T as fp16 (11 significant bits: the rounding stays below 2^-12 relative, which a bf16 P would
        // miss by a factor 16); the normaliser sums the same rounded weights
        if constexpr (WIDE) {
          u32x4 ph, pt;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            ph[r] = pack_bf16x2(pr[2 * r], pr[2 * r + 1]);
            pt[r] = pack_bf16x2(pr[2 * r] - __builtin_bit_cast(float, ph[r] << 16),
                                pr[2 * r + 1] - __builtin_bit_cast(float, ph[r] & 0xffff0000u));
          }
          {  // the normaliser: head and tail of the weights against ones (1.0 in bf16)
            const bf16x8 ones = __builtin_bit_cast(bf16x8, (u32x4){0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
            acc_l[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, __builtin_bit_cast(bf16x8, ph), acc_l[nb], 0, 0, 0);
            acc_l[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, __builtin_bit_cast(bf16x8, pt), acc_l[nb], 0, 0, 0);
          }
#pragma unroll
          for (int db = 0; db < kDB; ++db) {
            acc[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vop[db]),
                                                                  __builtin_bit_cast(bf16x8, ph), acc[nb][db], 0, 0, 0);
            acc[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vop[db]),
                                                                  __builtin_bit_cast(bf16x8, pt), acc[nb][db], 0, 0, 0);
          }
        } else {
          u32x4 pb;
#pragma unroll
          for (int r = 0; r < 4; ++r) pb[r] = pack_f16x2(pr[2 * r], pr[2 * r + 1]);
          const f16x8 pop = __builtin_bit_cast(f16x8, pb);
          {  // the normaliser sums the same rounded weights (1.0 in fp16)
            const f16x8 ones = __builtin_bit_cast(f16x8, (u32x4){0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u});
            acc_l[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pop, acc_l[nb], 0, 0, 0);
          }
#pragma unroll
          for (int db = 0; db < kDB; ++db)
            acc[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, vop[db]), pop, acc[nb][db], 0,
                                                                 0, 0);
        }
      }
    }
    // the other stage: its readers finished before the last barrier
    lstore(std::integral_constant<int, buf ^ 1>{}, widec);
    __syncthreads();
  };

  auto run = [&](auto widec) {
    gload();
    lstore(std::integral_constant<int, 0>{}, widec);
    __syncthreads();
#ifdef VTKV_PREFILL_TRACE
    trace_t1 = wall_clock64();
#endif
    for (int kb = 0; kb < nblocks; kb += 2) {
      stage(std::integral_constant<int, 0>{}, widec, kb);
      if (kb + 1 < nblocks) stage(std::integral_constant<int, 1>{}, widec, kb + 1);
    }
  };
  run(std::false_type{});
#ifdef VTKV_PREFILL_TRACE
  const unsigned long long trace_t2 = wall_clock64();
#endif
  if constexpr (!FP8 && !F16) {
    // A V value beyond the fp16 range went into LDS as infinity and has made some accumulator of the workgroup
    // infinite or NaN (a weight of exactly zero gives NaN).  Then the whole unit is computed again with V in
    // bf16; e4m3fn codes always fit fp16.  Inputs that are themselves non-finite take the second pass too and
    // come out non-finite again.
    unsigned expo = 0;
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
      for (int db = 0; db < kDB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) expo = max(expo, __builtin_bit_cast(unsigned, acc[nb][db][i]) & 0x7f800000u);
    // (one flag at the start of the stage memory, which nobody reads any more: every wave has passed the last
    // stage's barrier; the second pass may only overwrite it once all have read it)
    int *flag = reinterpret_cast<int *>(smem);
    if (threadIdx.x == 0) *flag = 0;
    __syncthreads();
    if (__builtin_amdgcn_ballot_w64(expo == 0x7f800000u) != 0 && lane == 0) *flag = 1;
    __syncthreads();
    const bool again = uniform(*flag) != 0;
    __syncthreads();
    if (again) {
      reset();
      rewind();
      run(std::true_type{});
    }
  }

  // ---- normalise and store: lane (n, g) holds O[column n][d = 16*db + 4g + i]
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    const float l = acc_l[nb][0];  // (already the sum over all rows: see acc_l)
    if (col_tok[nb] < 0) continue;
    const float inv = p.v_scale / l;
    const int64_t o0 = ((int64_t)(u_row0 + col_tok[nb]) * p.num_heads + head0 + col_head[nb]) * kD + 4 * g;
#pragma unroll
    for (int db = 0; db < kDB; ++db) {
      const f32x4 r = acc[nb][db] * inv;
      if (p.out_f32) {
        *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.out) + o0 + db * 16) = r;
      } else {
        u32x2 w = {pack_16x2<F16>(r[0], r[1]), pack_16x2<F16>(r[2], r[3])};
        *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(p.out) + o0 + db * 16) = w;
      }
    }
  }
#ifdef VTKV_PREFILL_TRACE
  if (threadIdx.x == 0 && blockIdx.x < 4096) {
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    g_prefill_trace[blockIdx.x][0] = xcc & 0xf;
    g_prefill_trace[blockIdx.x][1] = trace_t0;
    g_prefill_trace[blockIdx.x][2] = trace_t1;
    g_prefill_trace[blockIdx.x][3] = trace_t2;
    g_prefill_trace[blockIdx.x][4] = wall_clock64();
    g_prefill_trace[blockIdx.x][5] = (unsigned long long)nblocks;
  }
#endif
}

// 64, 80, 96, 112, 128, 256 (vllm/attention/ops/paged_attn.py:33-34) -> 0..5, anything else -> -1
int size_index(int head_size) {
  switch (head_size) {
    case 64: return 0;
    case 80: return 1;
    case 96: return 2;
    case 112: return 3;
    case 128: return 4;
    case 256: return 5;
    default: return -1;
  }
}

}  // namespace

extern "C" {

int vtkv_prefill_unit_tokens_for(int num_heads, int num_kv_heads, int head_size, int kv_dtype) {
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0) return 0;
  const int group_real = num_heads / num_kv_heads, split = vtkv_kv_split(group_real);
  if (size_index(head_size) < 0) return 0;
  (void)kv_dtype;  // the same kernels serve both cache types
  return cols_per_group(head_size) / ((group_real + split - 1) / split);
}

int vtkv_prefill_unit_tokens(int num_heads, int num_kv_heads, int kv_dtype) {
  return vtkv_prefill_unit_tokens_for(num_heads, num_kv_heads, 128, kv_dtype);
}

int vtkv_prefill_attention(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                           const int64_t *slot_ids, const int32_t *units, int num_units, int num_heads,
                           int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                           const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                           float v_scale, void *stream) {
  VTKV_REQUIRE(out && q && k_ptrs && v_ptrs && slot_ids && units, "null argument");
  VTKV_REQUIRE(num_units >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0,
               "num_heads %d must be a positive multiple of num_kv_heads %d", num_heads, num_kv_heads);
  const int d_index = size_index(head_size);
  VTKV_REQUIRE(d_index >= 0, "head_size %d is not supported (64, 80, 96, 112, 128, 256)", head_size);
  if (q_dtype == VTKV_F32) {
    // float32 models: every prompt token streams its own rows through the float32 decode kernel
    VTKV_REQUIRE(kv_dtype == VTKV_F32 && out_dtype == VTKV_F32, "float32 queries take a float32 cache and a float32 result");
    VTKV_REQUIRE(scale > 0.f && scale < INFINITY, "scale must be positive and finite");
    const int per_unit = vtkv_prefill_unit_tokens_for(num_heads, num_kv_heads, head_size, kv_dtype);
    VTKV_REQUIRE(per_unit > 0, "unsupported head counts");
    return vtkv::attention_f32((float *)out, (const float *)q, k_ptrs, v_ptrs, slot_ids, nullptr, units, per_unit,
                               num_units * per_unit, num_heads, num_kv_heads, head_size, q_stride, scale, max_seq_len,
                               alibi_slopes, nullptr, nullptr, nullptr, 0, nullptr, 0, stream);
  }
  VTKV_REQUIRE(q_dtype == VTKV_BF16 || q_dtype == VTKV_F16, "q_dtype must be BF16, F16 or F32");
  VTKV_REQUIRE(out_dtype == q_dtype || out_dtype == VTKV_F32, "out_dtype must be q_dtype or F32");
  VTKV_REQUIRE(scale > 0.f && scale < INFINITY, "scale must be positive and finite");
  VTKV_REQUIRE(kv_dtype == q_dtype || kv_dtype == VTKV_FP8_E4M3, "kv_dtype must be q_dtype or FP8_E4M3");
  const bool fp8 = kv_dtype == VTKV_FP8_E4M3;
  if (fp8) VTKV_REQUIRE(k_scale > 0.f && v_scale > 0.f, "fp8 scales must be positive");
  // more than 16 query heads per kv head: several virtual kv heads over the same rows (see first_head_of)
  const int group_real = num_heads / num_kv_heads, split = vtkv_kv_split(group_real);
  const int group = (group_real + split - 1) / split, kv_virtual = num_kv_heads * split;
  VTKV_REQUIRE(q_stride >= (int64_t)num_heads * head_size && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
                   (uintptr_t)out % 16 == 0,
               "q rows must be 16-byte aligned and at least num_heads*head_size apart");
  // (the kernel addresses a sequence's rows with 32-bit byte offsets)
  VTKV_REQUIRE(max_seq_len > 0 && ((int64_t)max_seq_len + 64) * num_kv_heads * head_size * 2 < (1ll << 31),
               "max_seq_len %d: a sequence's K or V range must stay below 2 GiB", max_seq_len);
  VTKV_REQUIRE((int64_t)num_units * kv_virtual < (1ll << 31), "too many units");
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
  p.num_kv_heads = kv_virtual;
  p.group = group;
  p.kv_split = split;
  p.group_real = group_real;
  p.scale_log2 = scale * kLog2e * (fp8 ? k_scale : 1.f);
  p.v_scale = fp8 ? v_scale : 1.f;
  const dim3 grid((unsigned)((int64_t)num_units * kv_virtual)), block(kThreads);
  hipStream_t st = (hipStream_t)stream;
  // head size 128: one kernel per (type, cache type, ALiBi); the other sizes decide ALiBi at run time
  static void (*const kKernels[8])(PrefillParams) = {
      prefill_attn_kernel<false, false, false>, prefill_attn_kernel<true, false, false>,
      prefill_attn_kernel<false, true, false>,  prefill_attn_kernel<true, true, false>,
      prefill_attn_kernel<false, false, true>,  prefill_attn_kernel<true, false, true>,
      prefill_attn_kernel<false, true, true>,   prefill_attn_kernel<true, true, true>,
  };
#define VTKV_PREFILL_SIZE(HS)                                                                        \
  prefill_attn_kernel<true, false, false, HS>, prefill_attn_kernel<true, true, false, HS>,           \
      prefill_attn_kernel<true, false, true, HS>, prefill_attn_kernel<true, true, true, HS>
  static void (*const kOthers[6][4])(PrefillParams) = {
      {VTKV_PREFILL_SIZE(64)}, {VTKV_PREFILL_SIZE(80)},  {VTKV_PREFILL_SIZE(96)},
      {VTKV_PREFILL_SIZE(112)}, {VTKV_PREFILL_SIZE(128)}, {VTKV_PREFILL_SIZE(256)},
  };
#undef VTKV_PREFILL_SIZE
  const bool f16 = q_dtype == VTKV_F16;
  void (*kernel)(PrefillParams) = head_size == 128 ? kKernels[(f16 ? 4 : 0) + (fp8 ? 2 : 0) + (alibi_slopes ? 1 : 0)]
                                                   : kOthers[d_index][(f16 ? 2 : 0) + (fp8 ? 1 : 0)];
  hipLaunchKernelGGL(kernel, grid, block, 0, st, p);
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

#ifdef VTKV_PREFILL_TRACE
__attribute__((visibility("default"))) int vtkv_debug_prefill_trace(unsigned long long *out, int n) {
  VTKV_HIP(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_prefill_trace), (size_t)n * 6 * sizeof(unsigned long long)));
  return VTKV_OK;
}
#endif

}  // extern "C"
