// Decode attention over per-sequence contiguous KV ranges ("vTensor" layout) for gfx950.
//
// One query token per sequence attends to the first seq_len rows of that sequence's K and V
// ranges, both token-major [T, Hkv, D].  The work is bound by HBM reads of K and V
// (2*Hkv*D*e bytes per token, 2*G/e flop per byte with G = Hq/Hkv), so the design goal is to read
// every K/V byte exactly once, keep many 16-byte loads in flight on every CU for the whole launch,
// and spend as little time as possible outside the streaming loop:
//
//  * work is counted in tiles of 16 rows of one kv head.  All tiles of the batch form one sequence
//    ordered (sequence, kv head, tile), or (kv head, sequence, tile) where that lines the kv heads up with
//    the XCDs; it is cut into gridDim.x equal contiguous spans, one per
//    workgroup, whatever the sequence lengths are ("stream-K" split).  Every CU therefore gets the
//    same number of bytes, a workgroup streams a long contiguous run of rows, and the fixed cost of
//    starting and finishing a (sequence, kv head) segment is paid once or twice per workgroup instead
//    of once per 512 rows.  The grid is the number of workgroups the device holds at once.
//  * ALL G query heads of a kv head's group share the pass over its rows (the reference launches one
//    block per query head and re-reads KV G times, csrc/attention/attention_kernels.cu:625).
//  * inside a workgroup the tiles of a segment are dealt round-robin to four wave64.  A wave loads a
//    K or V tile as whole rows: 16 consecutive lanes take the 256 bytes of one head row, so every
//    request covers full cache lines, and all of them carry the non-temporal hint: each byte is used
//    once, and on this part streaming loads that do not displace cache lines run about 8% faster than
//    plain ones.  (Loading K in its MFMA layout straight from global memory touches only 64 bytes of
//    a row per request; that is fine for plain loads, which merge in L2, and slow for streaming ones.)
//  * S^T = K_tile . Q^T runs on v_mfma_f32_16x16x32_bf16 with the G query heads padded to the 16
//    columns: K rows are the A operand.  A wave passes its K tile through a private swizzled LDS tile
//    to get from the row-per-16-lanes load layout to the row-per-lane operand layout.
//  * softmax statistics stay in registers: in the MFMA C layout a lane owns one head column and four
//    rows, so a head's max/sum over the tile is an in-lane reduction plus two cross-row-group
//    exchanges; an online (running-max) rescale keeps one pass.
//  * O^T += V_tile^T . P^T runs on v_mfma_f32_16x16x32_bf16.  P^T is the C layout of S^T as is.  V is
//    row-major but the A operand needs four rows per lane, so V tiles go through a wave-private,
//    XOR-swizzled LDS tile and come back with ds_read_b64_tr_b16 (the transposing LDS read).
//  * each wave keeps (m, l, O) for its rows; at the end of a segment the four waves merge through LDS
//    and the workgroup writes one normalised partial (max, sum, O/sum) per head into slot
//    (workgroup + segment id), which is unique because both only ever increase along the tile order.
//    A second small kernel merges the few partials of each (sequence, head) with the log-sum-exp rule
//    of the reference's split kernel (csrc/attention/attention_kernels.cu:486-583; CPU twin
//    csrc/cpu/attention.cpp:583-644).
//
// Numerics: bf16 q.k products accumulated in fp32 and softmax in fp32 as in the reference
// (csrc/attention/attention_kernels.cu:226-283).  The reference CUDA kernel rounds P to bf16
// before P.V (:326-327) while its CPU twin keeps P in fp32 (csrc/cpu/attention.cpp:197-211); here P
// enters the MFMA as a bf16 head plus a bf16 tail, which is as good as fp32 P for the tolerance in
// force.  fp32 accumulation, output rounded to bf16 once.  No epsilon is added to the softmax
// denominator (the CPU twin has none, csrc/cpu/attention.cpp:43-67).
#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <vector>

#include <hip/hip_ext.h>

#include "vtkv_common.h"
#ifndef VTKV_ATTN_STAGES
// Register tiles per wave of the bf16 variants.  One (the next tile's K loads are issued as soon as the K
// registers are free, its V loads likewise) against two: config 2 and 3 the same within 0.3 %, config 5
// 1 to 1.5 % faster per step (0.2083 against 0.2115 ms); three are 0.5 % slower than two.  More loads in
// flight do not help a kernel that already saturates the memory system.
#define VTKV_ATTN_STAGES 1
#endif
#ifndef VTKV_ATTN_BF16_WAVES
#define VTKV_ATTN_BF16_WAVES 2  // waves per SIMD of the bf16 variants (3 spills)
#endif
static_assert(VTKV_ATTN_STAGES >= 1 && VTKV_ATTN_STAGES <= 4, "1 to 4 register tiles per wave");
#include "vtkv_attn_common.h"
#include "vtkv_fp8.h"

#ifdef VTKV_ATTN_TRACE
// Tuning builds only: per workgroup of the last launch {XCC id, start, first segment's loads issued, end of the
// streaming loop, end} on the 100 MHz wall clock.
__device__ unsigned long long g_attn_trace[4096][6];
#endif

namespace {

using namespace vtkv_attn;


constexpr int kWaves = 4;          // waves per workgroup
constexpr int kThreads = kWaves * 64;
#ifndef VTKV_ATTN_FP8_STAGES
#define VTKV_ATTN_FP8_STAGES 1
#endif
constexpr int kStagesFp8 = VTKV_ATTN_FP8_STAGES;  // likewise for the fp8 variant (see the kernel)
#ifndef VTKV_ATTN_FP8_PAIR
#define VTKV_ATTN_FP8_PAIR 1  // fp8 rows: a workgroup streams two adjacent kv heads (see the kernel)
#endif
#ifndef VTKV_ATTN_FP8_WAVES
#define VTKV_ATTN_FP8_WAVES 3  // waves per SIMD of the fp8 variants
#endif
#ifndef VTKV_ATTN_SMALL_WAVES
#define VTKV_ATTN_SMALL_WAVES 2      // waves per SIMD of the 16-bit variants with head sizes below 128
#endif
#ifndef VTKV_ATTN_SMALL_FP8_WAVES
#define VTKV_ATTN_SMALL_FP8_WAVES 3  // likewise with fp8 rows
#endif
constexpr int kStagesBf16 = VTKV_ATTN_STAGES;  // register tiles per wave (prefetch distance kStages-1)
constexpr int kMaxSeqs = 1024;     // sequences per call (prefix sums of tile counts live in LDS)
constexpr int kMinSpan = 4;        // a workgroup takes at least one tile per wave
constexpr int kDefaultMaxGrid = 4096;  // upper bound of the resident-workgroup grid, sizes the scratch
constexpr int kMaxKvHeads = 64;        // kv heads per call (sizes the arrival counters)
constexpr int kInlineLens = 512;       // sequence lengths that fit the kernel argument block

struct AttnParams {
  const uint16_t *q;
  const int64_t *k_ptrs, *v_ptrs, *slot_ids;
  const int32_t *seq_lens;
  const float *alibi_slopes;
  // scratch: partial results per slot, and the prefix sums of per-sequence tile counts
  float *part_out;  // [slots][G][D]
  float *part_max;  // [slots][G]   (log2 units)
  float *part_sum;  // [slots][G]
  int32_t *cum_tiles;  // [num_seqs + 1]
  // [num_seqs * num_kv_heads] arrivals per (sequence, kv head) when the merge is done in the streaming
  // kernel (fused_merge); zero between launches: the workgroup that arrives last resets its counter
  uint32_t *seg_count;
  int fused_merge;
  int heads_per_seg;  // kv heads that share a segment of the tile order: 1, or 2 for the PAIR variants
  int reduce_sets;    // workgroups of the merge kernel that share the heads of a (kv head, sequence)
  void *out;           // [B,Hq,D] bf16, or fp32 when out_f32
  int out_f32;
  int64_t q_stride;
  int num_seqs, num_heads, num_kv_heads, group;  // B, Hq, Hkv, G (kv heads and heads of each as the kernels see them)
  int kv_split, group_real;  // see first_head_of: > 1 when a kv head has more than 16 query heads
  int head_size;    // D as the caller's tensors have it (the kernels hold it padded to their tile sizes)
  int out_f16;      // 16-bit outputs are fp16 (else bf16)
  int span_tiles;   // tiles per workgroup; 0 = all tiles / gridDim.x
  int grid;         // workgroups of the streaming kernel
  int xcd_spans;    // > 0: workgroup i takes span (i % 8) * xcd_spans + i / 8 (see the kernel)
  int head_major;   // the tile order is (kv head, sequence, tile) instead of (sequence, kv head, tile)
  float scale_log2;  // scale * log2(e) [* k_scale for fp8 K]
  float v_scale;
  // fused append: the step's new K/V rows, one per sequence, row b at new_k + b * new_k_stride (bytes)
  const char *new_k, *new_v;
  int64_t new_k_stride, new_v_stride;
  float k_quant, v_quant;  // fp8 cache: the new rows are stored as e4m3fn(x / k_quant), e4m3fn(x / v_quant)
  int inline_lens;  // sequence lengths come with the kernel arguments instead of from seq_lens
  // Partitions aligned with the sequences, the reference's split (csrc/attention/attention_kernels.cu:451-482):
  // > 0: workgroup ((sequence * segments per sequence + segment) * aligned_parts + j) takes rows
  // [j * 16 * span_tiles, (j + 1) * 16 * span_tiles) of that sequence, and besides its partial result in the
  // scratch it writes the caller's exp_sums / max_logits [B, Hq, aligned_parts] and tmp_out
  // [B, Hq, aligned_parts, D] (bf16), which the reference's interface hands in.
  int aligned_parts;
  float *v2_exp_sums, *v2_max_logits;
  uint16_t *v2_tmp_out;
};

// Sequence lengths passed by value (no upload, no dependent global load at the start of the kernel).
struct InlineLens {
  int32_t v[kInlineLens];
};


// Tiles per workgroup span, the same rule in both kernels.
__device__ __forceinline__ int span_of(const AttnParams &p, int total_tiles) {
  if (p.span_tiles > 0) return p.span_tiles;
  return max((total_tiles + p.grid - 1) / p.grid, kMinSpan);
}

// FP8: K and V rows hold one e4m3fn code per element (128 bytes per head row).  They are widened to
// bf16 in registers (K) or on the way into the LDS tile (V); the per-tensor scales are folded into the
// logit scale (K) and into the final normalisation (V), so dequantisation costs no multiply per element.
//
// HPS (kv heads per segment) = 2: a pair of adjacent kv heads is the unit of the tile order: a segment is
// (sequence, head pair), waves 0 and 2 take the even head of the pair and waves 1 and 3 the odd one, over the
// same rows at about the same time.  Everything a wave does is unchanged; only two waves instead of four
// share a head's tiles and its end-of-segment merge.  Two uses.  An fp8 head row is 128 bytes, and a stream
// of isolated 128-byte pieces (one per token, the kv heads of a token being 128 bytes apart) reaches about
// 6.1 TB/s on this part where 256-byte pieces reach 6.9 to 7.1, whichever workgroup fetches the
// neighbouring piece: with pairs the two 128-byte halves of a 256-byte piece are requested together from
// one CU.  And a batch of very many short sequences pays the start and the merge of a segment half as
// often.
//
// APPEND: seq_lens count the step's new token, whose K/V row is not in the cache yet but in new_k /
// new_v.  The rows before it are read from the cache as usual; the new row forms one more tile of its
// own at the end of the sequence's tile list, loaded from new_k / new_v, and the wave that handles it
// also stores the row into the cache.  One launch then does reshape_and_cache and attention, and each
// byte of the new rows is read once.
//
// D, F16: the head size (64, 80, 96, 112, 128 or 256) and whether q / K / V / out are fp16 instead of bf16.  The
// kernel was shaped for D = 128 and bf16, where every constant below takes the value it always had; the other
// sizes run the same code with fewer or more 16-byte pieces per row, MFMA steps and accumulator blocks.  A head
// size that is no multiple of the MFMA depth is held padded (80 as 96, 112 as 128; with fp8 rows, whose pieces
// carry 16 elements, 80, 96 and 112 as 128): the padding of the K and V tiles in LDS is cleared once and q is
// zero there, so padded columns add nothing to the logits and yield output columns that are never stored.
//
// SPLIT: some kv head has more than 16 query heads and is served in parts (see first_head_of); the variants
// without it index heads as kv head * group and carry none of that arithmetic.
//
// GW > 1 (kv heads per wave tile): GW adjacent kv heads whose query heads fit the 16 MFMA columns together are
// one kv head to everything outside the tile loop (the host hands over num_kv_heads / GW heads of group * GW
// query heads): column n belongs to sub-head n / (group / GW).  A wave's tile is 16 tokens of all GW sub-heads,
// GW * D * e contiguous bytes per token, a whole number of 128-byte lines, and it is loaded line by line: one
// load instruction takes one line of eight tokens, so that every line is asked for once.  A head row of 160,
// 192 or 224 bytes asked for by itself occupies two or three line requests of the CU's limited number in
// flight for 1.25 to 1.75 lines of data (head size 80: 0.62 of the peak, what 160 / 256 of the streaming rate
// gives).  The sub-heads then pass through the wave's K and V tiles one after the other: the lanes that hold
// pieces of a sub-head store them, all 16 columns get logits against its K rows, and the columns of other
// sub-heads are given weight zero before P.V, which adds nothing to their accumulators.  Per byte this is the
// arithmetic of the one-head tiles (whose unused columns compute throw-away values just the same).
template <bool ALIBI, bool FP8, bool APPEND, int HPS, int D = 128, bool F16 = false, bool SPLIT = false, int GW = 1>
__global__ void __launch_bounds__(kThreads)
    __attribute__((amdgpu_waves_per_eu(D > 128   ? 1
                                       : GW > 1 && D == 112 ? 1  // (four head rows of 224 bytes: 28 registers of 16 bytes per tile)
                                       : GW > 1  ? (FP8 && D <= 64 ? 3 : 2)  // (a tile of several kv heads is held in registers)
                                       : D < 128 ? (FP8 ? VTKV_ATTN_SMALL_FP8_WAVES : VTKV_ATTN_SMALL_WAVES)
                                                 : (FP8 ? VTKV_ATTN_FP8_WAVES : VTKV_ATTN_BF16_WAVES))))
    decode_attn_stream_kernel(AttnParams p, InlineLens il) {
  static_assert(D % 16 == 0 && D >= 64 && D <= 256, "head sizes are multiples of 16 from 64 to 256");
  static_assert(!APPEND || D == 128 || !FP8, "the fused append quantises new rows for head size 128 only");
  static_assert(!SPLIT || HPS == 1, "a segment of several kv heads is never one of split kv heads");
  static_assert(GW == 1 || (HPS == 1 && !SPLIT), "sub-heads per wave tile: one segment per kv head group");
  static_assert(GW == 1 || (GW * (FP8 ? D : 2 * D)) % 128 == 0, "the sub-heads of a token must fill whole cache lines");
  constexpr int kHD = FP8 ? (D + 63) / 64 * 64 : (D + 31) / 32 * 32;  // head size as held in LDS and registers
  constexpr int kKSteps = kHD / 32;                                  // MFMA steps of S^T = K.Q^T
  constexpr int kDBlocks = kHD / 16;                                 // 16-row blocks of O^T
  constexpr int kPitch = kHD * 2 < 256 ? 256 : kHD * 2;              // bytes of a tile row in LDS (16-bit elements)
  constexpr int kPitch8 = kHD < 128 ? 128 : kHD;                     // likewise for a K tile of fp8 codes
  constexpr int kTileBytes = kTile * kPitch;
  // An fp8 tile is half the bytes of a bf16 tile for the same chain of dependent steps, so that variant
  // is bound by latency, not by HBM: it runs three waves per SIMD (it fits 168 registers with one
  // register tile per wave, refilled as soon as its contents have gone to LDS) instead of two.
  constexpr int kStages = FP8 ? kStagesFp8 : kStagesBf16;
  // wave-private V tiles (4 KiB each); reused at the end of a segment for the cross-wave merge
  // then the merge statistics (1 KiB) and the wave-private K tiles
  __shared__ __attribute__((aligned(16))) char smem[2 * kWaves * kTileBytes + 1024];
  __shared__ int s_cum[kMaxSeqs + 1];  // s_cum[b] = tiles (of one kv head) of sequences before b
  __shared__ int s_wave_tot[kWaves];
  // pieces of shared (sequence, kv head) segments this workgroup has written: segment, first and last
  // workgroup of the segment, and whether this workgroup delivered the last piece
  __shared__ int s_pend[8][5];
  __shared__ int s_npend;

  const int lane = threadIdx.x & 63;
  // everything that decides control flow and base addresses is kept wave-uniform (scalar registers)
  const int wave = uniform(threadIdx.x >> 6);
  const int g = lane >> 4;   // row group of the MFMA layouts
  const int n = lane & 15;   // column: query head inside the group (S^T, O^T), or row of the tile (A operand)
  const int G = p.group;
  const int Hkv = p.num_kv_heads;
  const int B = p.num_seqs;
  static_assert(HPS == 1 || HPS == 2 || HPS == 4, "1, 2 or 4 kv heads per segment");  // (4 measured: no better than 2)
  constexpr int kHps = HPS;                    // kv heads per segment
  constexpr bool PAIR = HPS > 1;
  constexpr int kWph = kWaves / kHps;          // waves that share a head's tiles
  const int side = wave % kHps;                // this wave's head inside the segment
  const int ws = wave / kHps;                  // its place among the waves of that head
  const int Hseg = Hkv / kHps;                 // segments per sequence
  auto len_of = [&](int idx) { return p.inline_lens ? il.v[idx] : p.seq_lens[idx]; };
  // tiles of one kv head of a sequence: its cached rows in 16s, plus the new row's own tile
  auto tiles_of = [](int len) {
    if (len <= 0) return 0;
    return APPEND ? (len - 1 + kTile - 1) / kTile + 1 : (len + kTile - 1) / kTile;
  };

#ifdef VTKV_ATTN_TRACE
  const unsigned long long trace_t0 = wall_clock64();
#endif
  if (threadIdx.x == 0) s_npend = 0;
  // ---- exclusive prefix sums of the per-sequence tile counts (every workgroup computes its own copy)
  {
    constexpr int kPer = kMaxSeqs / kThreads;
    int local[kPer], sum = 0;
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      const int idx = threadIdx.x * kPer + k;
      const int len = idx < B ? len_of(idx) : 0;
      local[k] = sum;
      sum += tiles_of(len);
    }
    int incl = sum;  // inclusive scan over the wave
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int t = __shfl_up(incl, d);
      if (lane >= d) incl += t;
    }
    if (lane == 63) s_wave_tot[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += s_wave_tot[w];
    const int excl = base + incl - sum;
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      const int idx = threadIdx.x * kPer + k;
      if (idx <= B) s_cum[idx] = excl + local[k];
    }
    if (threadIdx.x == 0) s_cum[B] = s_wave_tot[0] + s_wave_tot[1] + s_wave_tot[2] + s_wave_tot[3];
    __syncthreads();
  }
  const int seq_tiles_total = uniform(s_cum[B]);
  const int total_tiles = seq_tiles_total * Hseg;
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i <= B; i += kThreads) p.cum_tiles[i] = s_cum[i];

  // ---- this workgroup's span [g_cur, g_end) of the global tile order
  const int span = span_of(p, total_tiles);
  // Which span a workgroup takes.  The hardware deals workgroups to the eight XCDs in turn (workgroup i runs
  // on XCD i % 8); with p.xcd_spans = gridDim.x / 8 every XCD gets one contiguous eighth of the tile order
  // instead of every eighth span.  Long sequences stream 5 % faster that way (config 3: 152 -> 144 us, and
  // the gain grows with the run of consecutive spans per XCD: 16, 32, 64 spans give 150, 146, 144 us;
  // config 2: 111.4 -> 110.1 us; each XCD has its own L2 and address translation, which of the two it is
  // has not been established); many short sequences with the merge inside this kernel lose 1.7 %
  // (config 5) unless the tile order is head-major as well (below), so the host asks for it together with the
  // separate merge kernel or with that order.
  const int wg = p.xcd_spans > 0 ? (int)(blockIdx.x % 8) * p.xcd_spans + (int)(blockIdx.x / 8) : (int)blockIdx.x;
  const int aligned = uniform(p.aligned_parts);
  int g_cur = wg * span;
  if (!aligned && g_cur >= total_tiles) return;
  int g_end = min(total_tiles, g_cur + span);

  // Two tile orders.  (sequence, kv head, tile): tile g of the order is Hseg*cum[b] + kvg*nt_b + tile.
  // (kv head, sequence, tile), p.head_major: g = kvg*cum[B] + cum[b] + tile; with eight kv heads and one
  // contiguous eighth of the order per XCD every XCD then streams one kv head of all sequences, i.e. pieces
  // whose address bits 8..10 are the same: the streaming micro-benchmark reads 1.5 to 2 % faster when each
  // XCD keeps to one such residue than when all XCDs read all of them (6 960 against 6 850 GB/s).
  const bool head_major = uniform(p.head_major) != 0;
  // first sequence of the span: the last b whose first tile is <= g_cur (sequences without rows own no tile)
  int b = 0, kvg = 0, tile0 = 0;
  if (!aligned) {
    const int hm_kvg = head_major ? g_cur / seq_tiles_total : 0;
    const int key = head_major ? g_cur - hm_kvg * seq_tiles_total : g_cur;  // compared with cum[b] * mul
    const int mul = head_major ? 1 : Hseg;
    int lo = 0, hi = B;  // invariant: mul*cum[lo] <= key < mul*cum[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (uniform(s_cum[mid]) * mul <= key) lo = mid; else hi = mid;
    }
    b = lo;
    const int nt = uniform(s_cum[b + 1]) - uniform(s_cum[b]);
    const int rest = key - uniform(s_cum[b]) * mul;
    kvg = head_major ? hm_kvg : rest / nt;  // segment of the sequence: kv head, or pair of kv heads
    tile0 = head_major ? rest : rest - kvg * nt;
  }
  int nt_b = uniform(s_cum[b + 1]) - uniform(s_cum[b]);
  int v2_part = 0;
  if (aligned) {
    // one segment, named by the workgroup's index; [g_cur, g_end) only counts its tiles
    v2_part = wg % aligned;
    const int sk = wg / aligned;
    kvg = sk % Hseg;
    b = sk / Hseg;
    nt_b = uniform(s_cum[b + 1]) - uniform(s_cum[b]);
    tile0 = v2_part * span;
    if (tile0 >= nt_b) return;
    g_cur = 0;
    g_end = min(span, nt_b - tile0);
  }

  typedef const __attribute__((address_space(1))) char *gptr;
  typedef const __attribute__((address_space(1))) u32x4 *gvec;
  constexpr int kKvRowBytes = FP8 ? D : 2 * D;       // bytes of one head row in global memory
  constexpr int kPieces = kKvRowBytes / 16;          // 16-byte pieces of a head row
  constexpr int kTilePieces = kTile * kPieces;       // ... of a 16-row tile, dealt to the lanes in order:
  // GW > 1: load j takes line j / 2 of tokens 8 (j % 2) .. + 8 of the tile, lane l the piece l % 8 of token l / 8
  constexpr int kLines = GW * kKvRowBytes / 128;     // (GW > 1) cache lines of a token's sub-heads
  constexpr int kLoads = GW > 1 ? 2 * kLines : (kTilePieces + 63) / 64;  // GW == 1: load j of lane l takes piece 64 j + l, i.e. row (64 j + l) / kPieces
  constexpr bool kEvenLoads = GW > 1 || kTilePieces % 64 == 0;  // every load of every lane carries a piece of the tile
  constexpr int kKa = FP8 ? kHD / 64 : kKSteps;      // 16-byte A-operand pieces a lane reads back per K tile
  const uint32_t row_stride = (uint32_t)(SPLIT ? Hkv / p.kv_split : Hkv) * (kKvRowBytes * GW);  // bytes between consecutive tokens
  char *v_tile = smem + wave * kTileBytes;
  char *k_tile = smem + kWaves * kTileBytes + 1024 + wave * kTileBytes;
  // tile layouts in LDS (see vtkv_attn_common.h for the swizzles), with this head size's row pitch
  auto v_off = [](int row, int piece16) { return row * kPitch + ((piece16 ^ ((row & 7) << 1)) << 4); };
  auto k_off = [](int row, int piece16) {
    return FP8 ? row * kPitch8 + ((piece16 ^ ((row >> 1) & 7)) << 4) : row * kPitch + ((piece16 ^ (row & 15)) << 4);
  };
  // where this lane's j-th load of a tile goes: (row, piece) of the tile, or nothing
  auto load_row = [&](int j) { return GW > 1 ? 8 * (j & 1) + (lane >> 3) : (64 * j + lane) / kPieces; };
  // (GW > 1: the piece's place in the token's region of GW head rows; sub-head and piece inside it follow from it)
  auto load_piece = [&](int j) { return GW > 1 ? 8 * (j >> 1) + (lane & 7) : (64 * j + lane) % kPieces; };
  auto load_live = [&](int j) { return kEvenLoads || 64 * j + lane < kTilePieces; };
  if constexpr ((FP8 ? kHD / 16 : kHD / 8) != kPieces) {
    // padded head size: the pad pieces of both tiles are cleared once; no load ever writes them
    constexpr int kPadK = (FP8 ? kHD / 16 : kHD / 8) - kPieces, kPadV = kHD / 8 - D / 8;
    for (int i = lane; i < kTile * kPadK; i += 64)
      *reinterpret_cast<u32x4 *>(k_tile + k_off(i / kPadK, kPieces + i % kPadK)) = (u32x4){0, 0, 0, 0};
    for (int i = lane; i < kTile * kPadV; i += 64)
      *reinterpret_cast<u32x4 *>(v_tile + v_off(i / kPadV, D / 8 + i % kPadV)) = (u32x4){0, 0, 0, 0};
  }

  // ---- one segment = the part of the span that lies in one (sequence, kv head or pair of kv heads)
  while (g_cur < g_end) {
    const int kvh = kvg * kHps + side;  // this wave's kv head
    const int seg_tiles = min(g_end - g_cur, nt_b - tile0);
    const int seq_len = uniform(len_of(b));
    const int ctx_len = APPEND ? seq_len - 1 : seq_len;                // rows read from the cache
    const bool has_new = APPEND && tile0 + seg_tiles == nt_b;          // the segment ends with the new row's tile
    const int seg_start = tile0 * kTile;                               // first row of the segment
    const int seg_end = min(ctx_len, (tile0 + seg_tiles) * kTile);     // one past its last cached row

    // the tables hold plain integers: say explicitly that they are global-memory addresses, otherwise
    // the loads become flat loads that also count on the LDS wait counter and defeat the prefetch
    const int64_t slot = p.slot_ids[b];
    // (virtual kv heads of one kv head read the same rows; with the fused append each of them stores the new
    // row, the same bytes at the same place)
    // this wave's kv head in memory and its query heads [head0, head0 + n_heads)
    int kv_real = kvh, head0 = kvh * G, n_heads = G;
    if constexpr (SPLIT) {
      kv_real = kvh / p.kv_split;
      const int part = kvh - kv_real * p.kv_split;
      head0 = kv_real * p.group_real + part * G;
      n_heads = min(G, p.group_real - part * G);
    }
    gptr k_base = (gptr)(uintptr_t)p.k_ptrs[slot] + kv_real * (kKvRowBytes * GW);
    gptr v_base = (gptr)(uintptr_t)p.v_ptrs[slot] + kv_real * (kKvRowBytes * GW);
    gptr nk_base = k_base, nv_base = v_base;
    if (APPEND) {
      nk_base = (gptr)(uintptr_t)p.new_k + (int64_t)b * p.new_k_stride + kv_real * (2 * D * GW);
      nv_base = (gptr)(uintptr_t)p.new_v + (int64_t)b * p.new_v_stride + kv_real * (2 * D * GW);
    }

    // B operand of S^T = K.Q^T: for MFMA step ks lane (n, g) holds the eight q[head n][d] whose K
    // elements the lane's 16-byte K operand pieces hold: d = 32*ks + 8*g + j for bf16 rows; for fp8 rows one
    // load carries 16 elements, so steps 2c and 2c+1 take d = 64*c + 16*g + j and + 8.  Zero for
    // padded heads.
    u32x4 qop[kKSteps];
    {
      const uint16_t *qrow = p.q + (int64_t)b * p.q_stride + (int64_t)(head0 + (n < n_heads ? n : 0)) * D;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        const int d0 = FP8 ? (ks >> 1) * 64 + g * 16 + (ks & 1) * 8 : ks * 32 + g * 8;
        u32x4 raw = (u32x4){0, 0, 0, 0};
        if (kHD == D || d0 < D) raw = *reinterpret_cast<const u32x4 *>(qrow + d0);  // (pieces are all in or all out)
        if (n >= n_heads) raw = (u32x4){0, 0, 0, 0};
        qop[ks] = raw;
      }
    }
    const int my_sub = GW > 1 ? n / (G / GW) : 0;  // sub-head of this lane's column
    float slope_log2 = 0.f;
    if (ALIBI) slope_log2 = (n < n_heads && p.alibi_slopes) ? p.alibi_slopes[head0 + n] * kLog2e : 0.f;

    f32x4 acc[kDBlocks];
#pragma unroll
    for (int i = 0; i < kDBlocks; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;  // running max of scaled logits (log2 units) of head n
    float l_run = 0.f;        // this lane's share of the running sum

    // The segment's tiles are dealt round-robin to the waves of a head: this wave owns tiles ws, ws+kWph, ...
    // Only the last tile of a sequence can be ragged; its missing rows are redirected to the last valid
    // row (their logits are masked) so no lane reads past the mapped part of a range.
    const int n_tiles = seg_tiles - (has_new ? 1 : 0);  // tiles of cached rows; the new row's tile comes last
    const int my_tiles = (seg_tiles - ws + kWph - 1) / kWph;
    // rows in the last tile of cached rows, 1..16
    const int valid_last = n_tiles > 0 ? seg_end - (seg_start + (n_tiles - 1) * kTile) : kTile;
    // per-lane byte offsets inside a K or V tile: load j of a lane takes row 4j+g, piece n, i.e. four
    // whole rows per load (fp8 rows are 128 bytes: a load then covers eight rows, lane l takes row
    // 8j + l/8, piece l%8).
    // (GW > 1: two offsets, one per half of the tile's tokens; load j adds its line, 128 (j / 2), as a constant)
    constexpr int kOffs = GW > 1 ? 2 : kLoads;
    uint32_t t_off[kOffs], t_off_last[kOffs];
    // The new row's tile.  16-bit cache: every row slot holds the one new row, a lane's load j the piece it
    // takes of any row (GW > 1: piece lane % 8 of line j / 2, the line added as a constant like above).
    // fp8 cache: the new row arrives as bf16 and is quantised in consume(): a lane's two loads fetch the
    // two bf16 pieces that become its 16 codes, pieces 2*(lane%8) and 2*(lane%8)+1 of the 256-byte row.
    uint32_t t_off_new[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; ++j)
      t_off_new[j] = FP8 ? ((lane & 7) * 2 + j) * 16 : GW > 1 ? (lane & 7) * 16 : load_live(j) ? load_piece(j) * 16 : 0;
#pragma unroll
    for (int j = 0; j < kOffs; ++j) {
      // (lanes past the end of the tile, where the head size leaves some, fetch its last row's first piece)
      const int row = load_live(j) ? load_row(j) : kTile - 1;
      const int col = load_live(j) ? load_piece(j) * 16 : 0;
      t_off[j] = (uint32_t)row * row_stride + col;
      t_off_last[j] = (uint32_t)min(row, valid_last - 1) * row_stride + col;
    }
    auto off_of = [&](int j, bool last) {
      if constexpr (GW > 1) return (last ? t_off_last[j & 1] : t_off[j & 1]) + (uint32_t)(j >> 1) * 128u;
      else return last ? t_off_last[j] : t_off[j];
    };

    // Loads of the i-th tile of this wave.  Always issued, never predicated, so the wait counters the
    // compiler derives are exact; past the wave's last tile every lane loads the segment's first 16
    // bytes instead (one cache line per load, not consumed).
    // `want(j)` (compile-time after unrolling) picks the loads to issue now: all of them, or with GW > 1 those of
    // the lines whose last sub-head has just gone to LDS, so that a tile's loads are spread over the previous one
    auto load_tile = [&](gptr base, gptr new_base, int i, u32x4 *regs, auto want) {
      const bool live = i < my_tiles;
      const int tile = ws + kWph * i;
      const bool last = tile == n_tiles - 1;
      const bool is_new = APPEND && has_new && live && tile == seg_tiles - 1;
      // (masks, not selects: selects here end up as branches around separate copies of the loads)
      const uint32_t mask = uniform(live && !is_new ? ~0u : 0u);
      const uint32_t mask_new = uniform(is_new ? ~0u : 0u);
      const int64_t row0 = (int64_t)((uint32_t)(seg_start + tile * kTile) & mask) * row_stride;
      gptr src = base;
      if (APPEND) src = (gptr)((uintptr_t)base + (((uintptr_t)new_base - (uintptr_t)base) & (uintptr_t)(int64_t)(int32_t)mask_new));  // base or new_base
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        if (!want(j)) continue;
        if constexpr (GW > 1) {
          // (the line's constant stays outside the mask: past the wave's last tile load j reads line j / 2 of the
          // segment's first token, which is mapped)
          uint32_t off = (last ? t_off_last[j & 1] : t_off[j & 1]) & mask;
          if (APPEND) off |= t_off_new[j] & mask_new;
          regs[j] = __builtin_nontemporal_load((gvec)(src + row0 + off + (j >> 1) * 128));
        } else {
          uint32_t off = off_of(j, last) & mask;
          if (APPEND) off |= t_off_new[j] & mask_new;
          // A head row that is no whole number of lines shares its first and last line with its neighbours,
          // which other waves of the workgroup ask for at about the same time: plain loads find them in L2
          // (HBM reads of head size 80: 1.27 x the rows with the streaming hint, 1.02 x without).
          if constexpr (kKvRowBytes % 128 != 0)
            regs[j] = *(gvec)(src + row0 + off);
          else
            regs[j] = __builtin_nontemporal_load((gvec)(src + row0 + off));
        }
      }
    };
    auto every = [](int) { return true; };
    auto load_k = [&](int i, u32x4 *kr) { load_tile(k_base, nk_base, i, kr, every); };
    auto load_v = [&](int i, u32x4 *vr) { load_tile(v_base, nv_base, i, vr, every); };

    // one 16-row tile: logits, online softmax update, P.V
    auto consume = [&](int i, u32x4 *kreg, u32x4 *vreg) {
      const int tile = ws + kWph * i;
      const bool is_new = APPEND && has_new && tile == seg_tiles - 1;
      const int t0 = is_new ? seq_len - 1 : seg_start + tile * kTile;                  // position of the tile's row 0
      const int valid = is_new ? 1 : (tile == n_tiles - 1 ? valid_last : kTile);       // rows that count
      if constexpr (APPEND && FP8) {
        if (is_new) {
          // the lane's sixteen new bf16 values of K and of V become e4m3fn codes, as scatter_rows_fp8_kernel
          // makes them (IEEE division by the scale, round to nearest even, saturate); the codes take the place
          // of a loaded tile whose rows all hold the new row, and lanes 0..7 append them to the cache
          auto quantise = [](const u32x4 &a, const u32x4 &b, float sc) {
            u32x4 c;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              const u32x4 &src = w < 2 ? a : b;
              uint32_t word = 0;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const uint32_t pair = src[(2 * w + e / 2) & 3];
                const float x = unpack_16<F16>(pair, e & 1);
                word |= (uint32_t)vtkv::fp8_e4m3fn_encode(x / sc) << (8 * e);
              }
              c[w] = word;
            }
            return c;
          };
          kreg[0] = kreg[1] = quantise(kreg[0], kreg[1], p.k_quant);
          vreg[0] = vreg[1] = quantise(vreg[0], vreg[1], p.v_quant);
          if (lane < 8) {
            typedef __attribute__((address_space(1))) u32x4 *gvec_rw;
            const int64_t dst = (int64_t)(seq_len - 1) * row_stride + lane * 16;
            *(gvec_rw)((uintptr_t)k_base + dst) = kreg[0];
            *(gvec_rw)((uintptr_t)v_base + dst) = vreg[0];
          }
        }
      } else if (APPEND && is_new) {
        // the lanes that hold row 0 of the tile hold the 16-byte pieces of the new K and V rows: append them to
        // the cache (one head row: lanes 0 .. kPieces - 1 of load 0; GW > 1: lanes 0..7 of each line's first load)
        typedef __attribute__((address_space(1))) u32x4 *gvec_rw;
        const int64_t dst = (int64_t)(seq_len - 1) * row_stride + lane * 16;
        if constexpr (GW > 1) {
          if (lane < 8) {
#pragma unroll
            for (int line = 0; line < kLines; ++line) {
              *(gvec_rw)((uintptr_t)k_base + dst + line * 128) = kreg[2 * line];
              *(gvec_rw)((uintptr_t)v_base + dst + line * 128) = vreg[2 * line];
            }
          }
        } else if (lane < kPieces) {
          *(gvec_rw)((uintptr_t)k_base + dst) = kreg[0];
          *(gvec_rw)((uintptr_t)v_base + dst) = vreg[0];
        }
      }
      // GW > 1: the tile's sub-heads one after the other through the same K and V tiles (once for GW == 1).
      // Load j of a lane holds a piece of sub-head hh iff its place in the token's region lies in that head's
      // pieces; which loads can hold any is known at compile time (line j / 2 against the head's byte range).
#pragma unroll
      for (int hh = 0; hh < GW; ++hh) {
      auto sub_live = [&](int j) {
        if constexpr (GW == 1) return load_live(j);
        else return load_piece(j) >= hh * kPieces && load_piece(j) < (hh + 1) * kPieces;
      };
      auto sub_line = [&](int j) {  // compile-time part of sub_live
        return GW == 1 || (8 * (j >> 1) < (hh + 1) * kPieces && 8 * (j >> 1) + 8 > hh * kPieces);
      };
      auto sub_piece = [&](int j) { return GW == 1 ? load_piece(j) : load_piece(j) - hh * kPieces; };
      const bool mine = GW == 1 || my_sub == hh;  // this lane's column belongs to the sub-head
      // S^T[row, head] = sum_d K[row, d] q[head, d]
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
      // K tile through LDS: in as loaded, out as A operand (lane (n, g): row n, bytes [16g, +16) of
      // each 64-byte quarter)
      u32x4 ka[kKa];
#pragma unroll
      for (int j = 0; j < kLoads; ++j)
        if (sub_line(j) && sub_live(j)) *reinterpret_cast<u32x4 *>(k_tile + k_off(load_row(j), sub_piece(j))) = kreg[j];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
      for (int c = 0; c < kKa; ++c) ka[c] = *reinterpret_cast<const u32x4 *>(k_tile + k_off(n, 4 * c + g));
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      // the K registers are free again: refill them (GW > 1: those of the lines that end in this sub-head)
      auto done_with = [&](int j) { return GW == 1 || min(GW - 1, (8 * (j >> 1) + 7) / kPieces) == hh; };
      if (kStages == 1) load_tile(k_base, nk_base, i + 1, kreg, done_with);
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        const u32x4 kop =
            FP8 ? fp8x8_widen<F16>(ka[ks >> 1][2 * (ks & 1)], ka[ks >> 1][2 * (ks & 1) + 1]) : ka[ks];
        s = mfma_16x16x32<F16>(kop, qop[ks], s);
      }

      // stage V (as 16-bit values) for the transposing read
      if constexpr (FP8) {
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
          if (!sub_line(j) || !sub_live(j)) continue;
          const int row = load_row(j), piece = 2 * sub_piece(j);
          *reinterpret_cast<u32x4 *>(v_tile + v_off(row, piece)) = fp8x8_widen<F16>(vreg[j][0], vreg[j][1]);
          *reinterpret_cast<u32x4 *>(v_tile + v_off(row, piece + 1)) = fp8x8_widen<F16>(vreg[j][2], vreg[j][3]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < kLoads; ++j)
          if (sub_line(j) && sub_live(j)) *reinterpret_cast<u32x4 *>(v_tile + v_off(load_row(j), sub_piece(j))) = vreg[j];
      }
      if (kStages == 1) load_tile(v_base, nv_base, i + 1, vreg, done_with);  // likewise the V registers once they are in LDS

      // logits in log2 units; lane owns rows t0 + 4*g + r of head n
      float x[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        x[r] = s[r] * p.scale_log2;
        if (ALIBI) x[r] += slope_log2 * (float)(t0 + 4 * g + r - seq_len + 1);
      }
      if (valid < kTile) {  // wave-uniform: only a sequence's ragged last tile, or the new row's tile
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (4 * g + r >= valid) x[r] = -INFINITY;
      }
      const float tmax = max_over_row_groups(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])));
      // (a column of another sub-head: maximum and accumulators stay as they are, its weights are zero; the selects
      // also discard whatever the arithmetic makes of a maximum that is still -inf)
      const float m_new = mine ? fmaxf(m_run, tmax) : m_run;
      const float alpha_raw = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first tile (m_run = -inf)
      const float alpha = mine ? alpha_raw : 1.f;
      m_run = m_new;
      float pr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = __builtin_amdgcn_exp2f(x[r] - m_new);
        pr[r] = mine ? e : 0.f;
      }
      l_run = l_run * alpha + ((pr[0] + pr[1]) + (pr[2] + pr[3]));
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
        for (int d = 0; d < kDBlocks; ++d) acc[d] *= alpha;
      }
      // P^T as B operand, split into a bf16 head and a bf16 tail so that P.V keeps ~16 mantissa bits of
      // P (the result then tracks an fp32-P reference, not just a bf16-P one).  Head and tail share one
      // K=32 MFMA: reduction slot (g, j) of v_mfma_f32_16x16x32_bf16 stands for row 4g+j with the head of
      // P for j < 4 and for row 4g+j-4 with the tail for j >= 4, so the B operand is [head(4), tail(4)]
      // straight from this lane's four logits and the A operand is the lane's V^T quad twice.
      // (fp16 rows: head and tail are fp16, 22 bits of P between them; a tail below 2^-24 is lost, which is
      // an absolute error of that size in a weight that is at most 1)
      float plo[4];
      u32x4 pb;
      pb[0] = pack_16x2<F16>(pr[0], pr[1]);
      pb[1] = pack_16x2<F16>(pr[2], pr[3]);
#pragma unroll
      for (int r = 0; r < 4; ++r) plo[r] = pr[r] - unpack_16<F16>(pb[r >> 1], r & 1);
      pb[2] = pack_16x2<F16>(plo[0], plo[1]);
      pb[3] = pack_16x2<F16>(plo[2], plo[3]);
      const u32x4 pop = pb;

      // O^T[d, head] += sum_row V[row, d] P[row, head], 16 d per MFMA.  LDS operations of one wave
      // execute in order, so the fences only pin the compiler's ordering of tile writes and reads.
      // The reads are issued four at a time ahead of the MFMAs that use them.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      {
        const int row = 4 * g + (n >> 2);
        const int base = row * kPitch + ((n & 1) << 3);
        const int swz = (row & 7) << 1;
#pragma unroll
        for (int d0 = 0; d0 < kDBlocks; d0 += 4) {
          constexpr int kGroup = 4;  // blocks whose reads are issued together (the last group may be shorter)
          u32x4 vop[kGroup];
#pragma unroll
          for (int d4 = 0; d4 < kGroup; ++d4) {
            const int db = d0 + d4;
            if (db >= kDBlocks) break;
            const int off = base + (((2 * db + ((n >> 1) & 1)) ^ swz) << 4);
            const s16x4 quad =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(v_tile + off));
            const u32x2 qd = __builtin_bit_cast(u32x2, quad);
            vop[d4] = (u32x4){qd[0], qd[1], qd[0], qd[1]};
          }
#pragma unroll
          for (int d4 = 0; d4 < kGroup; ++d4) {
            if (d0 + d4 >= kDBlocks) break;
            acc[d0 + d4] = mfma_16x16x32<F16>(vop[d4], pop, acc[d0 + d4]);
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }  // sub-heads
    };

    // A ring of kStages register tiles per wave: while one tile is consumed the loads of the wave's next
    // kStages-1 tiles are in flight.  The steady-state path has no join after a load, only exits.
    if (my_tiles > 0) {
      u32x4 kbuf[kStages][kLoads], vbuf[kStages][kLoads];
      if constexpr (kStages == 1) {
        // one register tile per wave, refilled inside consume() as soon as its contents have been used:
        // the loads of tile i+1 fly during the softmax and P.V of tile i at no extra register cost
        load_k(0, kbuf[0]);
        load_v(0, vbuf[0]);
        for (int i = 0; i < my_tiles; ++i) consume(i, kbuf[0], vbuf[0]);
      } else {
#pragma unroll
        for (int st = 0; st < kStages - 1; ++st) {
          load_k(st, kbuf[st]);
          load_v(st, vbuf[st]);
        }
        int i = 0;
#define VTKV_STAGE(ST)                                                           \
  {                                                                              \
    load_k(i + kStages - 1, kbuf[((ST) + kStages - 1) % kStages]);               \
    load_v(i + kStages - 1, vbuf[((ST) + kStages - 1) % kStages]);               \
    consume(i, kbuf[(ST)], vbuf[(ST)]);                                          \
    if (++i >= my_tiles) break;                                                  \
  }
        for (;;) {
          VTKV_STAGE(0)
          if constexpr (kStages > 1) VTKV_STAGE(1)
          if constexpr (kStages > 2) VTKV_STAGE(2)
          if constexpr (kStages > 3) VTKV_STAGE(3)
        }
#undef VTKV_STAGE
      }
    }

    // ---- merge the waves of each head.  l_run is still split over the four row groups of a lane column.
    l_run = sum_over_row_groups(l_run);
    __syncthreads();  // every wave is done with its V tile: smem is free for the merge
    float *sm_m = reinterpret_cast<float *>(smem + kWaves * kTileBytes);  // [4][16]
    float *sm_l = sm_m + kWaves * 16;                                        // [4][16]
    float *sm_o = reinterpret_cast<float *>(smem);                           // [4][8][kHD]: at most the V tiles' size
    if (g == 0) {
      sm_m[wave * 16 + n] = m_run;
      sm_l[wave * 16 + n] = l_run;
    }
    __syncthreads();
    // the waves of head `sd` of the segment are sd, sd + kHps, ...
    auto head_max = [&](int sd, int head) {
      float m = sm_m[sd * 16 + head];
#pragma unroll
      for (int j = 1; j < kWph; ++j) m = fmaxf(m, sm_m[(sd + kHps * j) * 16 + head]);
      return m;
    };
    const float f = __builtin_amdgcn_exp2f(m_run - head_max(side, n));  // 0 for a wave that saw no row
    // Slot of this (workgroup, segment, head): kHps * workgroup + (sequence * Hkv + kv head).  Along the tile
    // order neither the workgroup nor the segment ever decreases, and a later workgroup's kv head is at most
    // kHps - 1 lower than an earlier one's (inside a shared pair), so the sum is unique.
    // Workgroups w0..w1 hold the pieces of this segment: its tiles are [first, first + nt_b) of the
    // global order.
    const int first_tile = head_major ? kvg * seq_tiles_total + uniform(s_cum[b]) : uniform(s_cum[b]) * Hseg + kvg * nt_b;
    const int w0 = first_tile / span, w1 = (first_tile + nt_b - 1) / span;
    const bool whole = p.fused_merge && w0 == w1;  // no other workgroup: the result is final
    auto store_out = [&](int kv_head, int head, int d, float r) {
      const int64_t oi = ((int64_t)b * p.num_heads + (SPLIT ? head0 : kv_head * G) + head) * D + d;
      if (p.out_f32)
        reinterpret_cast<float *>(p.out)[oi] = r;
      else
        reinterpret_cast<uint16_t *>(p.out)[oi] = f32_to_16<F16>(r);
    };
    // G <= 8 fits the 16 KiB; for larger groups the merge runs in two halves of 8 heads
    for (int h0 = 0; h0 < G; h0 += 8) {
      if (h0 > 0) __syncthreads();
      if (n >= h0 && n < min(G, h0 + 8)) {
#pragma unroll
        for (int db = 0; db < kDBlocks; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            sm_o[(wave * 8 + (n - h0)) * kHD + db * 16 + 4 * g + i] = acc[db][i] * f;
      }
      __syncthreads();
      const int nh = min(G, h0 + 8) - h0;
      for (int idx = threadIdx.x; idx < kHps * nh * kHD; idx += kThreads) {
        const int sd = PAIR ? idx / (nh * kHD) : 0;
        const int rem = idx - sd * (nh * kHD);
        const int hh = rem / kHD, d = rem % kHD;
        if (kHD != D && d >= D) continue;  // a padded column
        const int head = h0 + hh;
        const int kv_head = kvg * kHps + sd;
        const bool real_head = !SPLIT || head < n_heads;  // (the last part of a split kv head may have fewer)
        const float mw = head_max(sd, head);
        float lsum = 0.f, o = 0.f;
#pragma unroll
        for (int j = 0; j < kWph; ++j) {
          const int w = sd + kHps * j;
          lsum += sm_l[w * 16 + head] * __builtin_amdgcn_exp2f(sm_m[w * 16 + head] - mw);
          o += sm_o[(w * 8 + hh) * kHD + d];
        }
        const float o_norm = o / lsum;
        if (aligned && p.v2_tmp_out && real_head) {
          // the reference's per-partition outputs: max logit in natural units, sum of exponentials, and the
          // partition's normalised result in the model's dtype (csrc/attention/attention_kernels.cu:404-419)
          const int64_t vi = ((int64_t)b * p.num_heads + (SPLIT ? head0 : kv_head * G) + head) * aligned + v2_part;
          p.v2_tmp_out[vi * D + d] = f32_to_16<F16>(o_norm * p.v_scale);
          if (d == 0) {
            p.v2_max_logits[vi] = mw * 0.6931471805599453f;
            p.v2_exp_sums[vi] = lsum;
          }
        }
        if (whole) {
          if (real_head) store_out(kv_head, head, d, o_norm * p.v_scale);
          continue;
        }
        // (head-major order: (segment's kv heads, sequence, head inside the segment) is what grows along it)
        const int64_t seg_rank = head_major ? ((int64_t)kvg * B + b) * kHps + sd : (int64_t)b * Hkv + kv_head;
        const int64_t pidx = ((int64_t)kHps * wg + seg_rank) * G + head;
        if (p.fused_merge) {
          store_device_coherent(&p.part_out[pidx * kHD + d], o_norm);
          if (d == 0) {
            store_device_coherent(&p.part_max[pidx], mw);
            store_device_coherent(&p.part_sum[pidx], lsum);
          }
        } else {
          p.part_out[pidx * kHD + d] = o_norm;
          if (d == 0) {
            p.part_max[pidx] = mw;  // log2 units
            p.part_sum[pidx] = lsum;
          }
        }
      }
    }
    if (p.fused_merge && !whole && threadIdx.x == 0) {
      // Pieces of (sequence, kv head) segments that other workgroups share.  Their arrival is counted at the
      // end of this workgroup's span, not here, so that the streaming goes on without waiting for the
      // stores.  Only the first and the last segment of a span can be such pieces.
      int k = s_npend;
      for (int sd = 0; sd < kHps; ++sd, ++k) {
        s_pend[k][0] = b * Hkv + kvg * kHps + sd;
        s_pend[k][4] = head_major ? (kvg * B + b) * kHps + sd : s_pend[k][0];  // its place among the partial slots
        s_pend[k][1] = w0;
        s_pend[k][2] = w1;
      }
      s_npend = k;
    }

    // ---- next segment of the span
    g_cur += seg_tiles;
    tile0 += seg_tiles;
    if (g_cur < g_end) {
      if (tile0 == nt_b) {
        tile0 = 0;
        if (head_major) {
          do {
            if (++b == B) {
              b = 0;
              ++kvg;
            }
            nt_b = uniform(s_cum[b + 1]) - uniform(s_cum[b]);
          } while (nt_b == 0);  // g_cur < total_tiles guarantees a later segment with rows
        } else if (++kvg == Hseg) {
          kvg = 0;
          do {
            ++b;
            nt_b = uniform(s_cum[b + 1]) - uniform(s_cum[b]);
          } while (nt_b == 0);  // g_cur < total_tiles guarantees a later sequence with rows
        }
      }
      __syncthreads();  // the merge area is the next segment's V tiles
    }
  }

#ifdef VTKV_ATTN_TRACE
  if (threadIdx.x == 0 && blockIdx.x < 4096) {
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    g_attn_trace[blockIdx.x][0] = xcc & 0xf;
    g_attn_trace[blockIdx.x][1] = trace_t0;
    g_attn_trace[blockIdx.x][2] = (unsigned long long)wg;
    g_attn_trace[blockIdx.x][3] = wall_clock64();
    g_attn_trace[blockIdx.x][4] = (unsigned long long)(g_end - wg * span);
  }
#endif
  // ---- arrivals and merges of the shared segments (the rule of decode_attn_reduce_kernel below).
  // Pieces come from other CUs and other L2s: they were written with device-coherent stores, every wave
  // waits until its stores have completed before the arrivals are counted, and the pieces are read with
  // device-coherent loads.  Why relaxed atomics are enough here: ordering is not left to the memory model
  // but made by completion.  An agent-scope atomic store on this part is a write-through store (sc1) that is
  // acknowledged only once it is visible device-wide; s_waitcnt vmcnt(0) holds each wave until all of its
  // stores are acknowledged, the barrier collects the waves, and only then does one lane count the arrival,
  // so a workgroup that reads the full count can only run after every piece is visible, and it reads the
  // pieces with loads that bypass its own L2.  A release/acquire pair at agent scope would be correct too
  // but is implemented as a write-back and invalidate of the whole L2 on either side, which tripled the
  // kernel's time when it was tried.  The workgroup that delivers the last piece of a segment merges it and leaves
  // the counter at zero for the next launch.
  if (p.fused_merge) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int np = uniform(s_npend);
    if (np == 0) return;
    for (int k = wave; k < np && lane == 0; k += kWaves) {
      const int seg = s_pend[k][0];
      const unsigned pieces = (unsigned)(s_pend[k][2] - s_pend[k][1] + 1);
      const unsigned old = __hip_atomic_fetch_add(&p.seg_count[seg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last_piece = old + 1 == pieces;
      if (last_piece) __hip_atomic_store(&p.seg_count[seg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_pend[k][3] = last_piece;
    }
    __syncthreads();
    const int per_seg = G * kHD;
    for (int idx = threadIdx.x; idx < np * per_seg; idx += kThreads) {
      const int j = idx / per_seg;
      if (!s_pend[j][3]) continue;
      const int head = (idx - j * per_seg) / kHD, d = idx % kHD;
      if (kHD != D && d >= D) continue;
      const int64_t seg = s_pend[j][0], seg_rank = s_pend[j][4];
      const int w0 = s_pend[j][1], w1 = s_pend[j][2];
      // four pieces at a time, all their loads in flight together; running (max, sum, out) across batches
      float m = -INFINITY, wsum = 0.f, o = 0.f;
      for (int wb = w0; wb <= w1; wb += 4) {
        float pm[4], ps[4], po[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int64_t pidx = ((int64_t)kHps * min(wb + jj, w1) + seg_rank) * G + head;
          pm[jj] = load_device_coherent(&p.part_max[pidx]);
          ps[jj] = load_device_coherent(&p.part_sum[pidx]);
          po[jj] = load_device_coherent(&p.part_out[pidx * kHD + d]);
        }
        float bm = pm[0];
#pragma unroll
        for (int jj = 1; jj < 4; ++jj) bm = fmaxf(bm, pm[jj]);
        const float m_new = fmaxf(m, bm);
        const float keep = __builtin_amdgcn_exp2f(m - m_new);  // 0 for the first batch
        wsum *= keep;
        o *= keep;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const float wt = wb + jj <= w1 ? ps[jj] * __builtin_amdgcn_exp2f(pm[jj] - m_new) : 0.f;
          wsum += wt;
          o += po[jj] * wt;
        }
        m = m_new;
      }
      const float r = o / wsum * p.v_scale;
      // segment = sequence * Hkv + kv head, so (segment * G + head) is (sequence * Hq + query head)
      int64_t oi = (seg * G + head) * D + d;
      if constexpr (SPLIT) {
        const int bb = (int)seg / Hkv, kv_head = (int)seg - bb * Hkv;
        if (head >= heads_of(p, kv_head)) continue;
        oi = ((int64_t)bb * p.num_heads + first_head_of(p, kv_head) + head) * D + d;
      }
      if (p.out_f32)
        reinterpret_cast<float *>(p.out)[oi] = r;
      else
        reinterpret_cast<uint16_t *>(p.out)[oi] = f32_to_16<F16>(r);
    }
  }
}

// Merge the partials of one (sequence, head): out = sum_j o_j w_j / sum_j w_j with
// w_j = l_j * 2^(m_j - max m)  (csrc/attention/attention_kernels.cu:515-582).  The segment's tiles
// [first, first + nt) of the global order were handled by workgroups first/span .. (first+nt-1)/span.
// One workgroup per (kv head, sequence), thread d; the group's heads are taken four at a time and the
// pieces four at a time, so that up to 48 loads of a thread are in flight together: the kernel is a chain
// of three or four memory round trips (tile counts, then statistics and partial outputs of a batch), and
// with one small workgroup per query head it was that chain times many more workgroups.
// GROUPS > 1 (segments of many pieces: a few long sequences): GROUPS sets of kD threads take every GROUPS-th
// batch of four pieces and their running (max, sum, out) are combined through LDS at the end, so the chain
// of dependent round trips is GROUPS times shorter (config 3: 37 pieces per segment).
// HSETS > 1 (only with GROUPS == 1, which has no barrier): HSETS sets of kD threads take the group's heads
// four at a time in turn, so a group of eight heads is merged in one pass instead of two.
// HD: the head size as the stream kernel pads it (the row length of a partial result); thread d handles
// column d and stores it if it is a real one (d < p.head_size).
template <int GROUPS, int HSETS, int HD = 128, bool SPLIT = false>
__global__ void __launch_bounds__(HD * GROUPS * HSETS) decode_attn_reduce_kernel(AttnParams p) {
  static_assert(GROUPS == 1 || HSETS == 1, "head sets only without piece groups");
  constexpr int kD = HD;  // (shadows the library-wide 128 inside this kernel)
  // (groups above 8: the heads of a kv head are dealt to p.reduce_sets workgroups, four heads at a time in turn)
  const int sets = p.reduce_sets, kvh = blockIdx.x / sets, bset = blockIdx.x % sets;
  const int b = blockIdx.y, d = threadIdx.x % kD;
  const int grp = GROUPS > 1 ? threadIdx.x / kD : 0, hset = HSETS > 1 ? threadIdx.x / kD : 0;
  __shared__ float sm_red[GROUPS > 1 ? 3 * GROUPS * 4 * kD : 1];
  const int G = p.group, Hkv = p.num_kv_heads;
  const int cum_b = p.cum_tiles[b];
  const int nt = p.cum_tiles[b + 1] - cum_b;
  if (nt <= 0) return;
  const int hps = p.heads_per_seg, Hseg = Hkv / hps;
  const int total_tiles = p.cum_tiles[p.num_seqs] * Hseg;
  const int span = span_of(p, total_tiles);
  const int first = p.head_major ? (kvh / hps) * p.cum_tiles[p.num_seqs] + cum_b : cum_b * Hseg + (kvh / hps) * nt;
  int w0 = first / span, w1 = (first + nt - 1) / span;
  if (p.aligned_parts > 0) {
    w0 = (b * Hseg + kvh / hps) * p.aligned_parts;
    w1 = w0 + (nt + span - 1) / span - 1;
  }
  const int64_t seg = p.head_major ? ((int64_t)(kvh / hps) * p.num_seqs + b) * hps + kvh % hps : (int64_t)b * Hkv + kvh;
  bool first_pass = true;
  for (int h0 = 4 * (hset + HSETS * bset); h0 < G; h0 += 4 * HSETS * sets) {
    float m[4], wsum[4], o[4];
#pragma unroll
    for (int hh = 0; hh < 4; ++hh) m[hh] = -INFINITY, wsum[hh] = 0.f, o[hh] = 0.f;
    for (int wb = w0 + 4 * grp; wb <= w1; wb += 4 * GROUPS) {
      float pm[4][4], ps[4][4], po[4][4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
#pragma unroll
        for (int hh = 0; hh < 4; ++hh) {
          // (pieces and heads past the end repeat the last one; their weights are set to zero below)
          const int64_t pidx = ((int64_t)hps * min(wb + jj, w1) + seg) * G + min(h0 + hh, G - 1);
          pm[jj][hh] = p.part_max[pidx];
          ps[jj][hh] = p.part_sum[pidx];
          po[jj][hh] = p.part_out[pidx * kD + d];
        }
#pragma unroll
      for (int hh = 0; hh < 4; ++hh) {
        float bm = pm[0][hh];
#pragma unroll
        for (int jj = 1; jj < 4; ++jj) bm = fmaxf(bm, pm[jj][hh]);
        const float m_new = fmaxf(m[hh], bm);
        const float keep = __builtin_amdgcn_exp2f(m[hh] - m_new);  // 0 for the first batch
        wsum[hh] *= keep;
        o[hh] *= keep;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const float wt = wb + jj <= w1 ? ps[jj][hh] * __builtin_amdgcn_exp2f(pm[jj][hh] - m_new) : 0.f;
          wsum[hh] += wt;
          o[hh] += po[jj][hh] * wt;
        }
        m[hh] = m_new;
      }
    }
    if constexpr (GROUPS > 1) {
      if (!first_pass) __syncthreads();  // the previous heads' values have been read
      first_pass = false;
#pragma unroll
      for (int hh = 0; hh < 4; ++hh) {
        float *at = sm_red + ((grp * 4 + hh) * kD + d) * 3;
        at[0] = m[hh], at[1] = wsum[hh], at[2] = o[hh];
      }
      __syncthreads();
      if (grp == 0) {
#pragma unroll
        for (int hh = 0; hh < 4; ++hh) {
          float mm = m[hh];  // finite: group 0 always has the segment's first piece
          for (int gg = 1; gg < GROUPS; ++gg) mm = fmaxf(mm, sm_red[((gg * 4 + hh) * kD + d) * 3]);
          float ws = 0.f, oo = 0.f;
          for (int gg = 0; gg < GROUPS; ++gg) {
            const float *at = sm_red + ((gg * 4 + hh) * kD + d) * 3;
            const float f = __builtin_amdgcn_exp2f(at[0] - mm);  // 0 for a group that saw no piece
            ws += at[1] * f;
            oo += at[2] * f;
          }
          wsum[hh] = ws, o[hh] = oo;
        }
      }
    }
    if (grp != 0) continue;
#pragma unroll
    for (int hh = 0; hh < 4; ++hh) {
      if (h0 + hh >= (SPLIT ? heads_of(p, kvh) : G)) break;
      if (d >= p.head_size) break;  // a padded column
      const float r = o[hh] / wsum[hh] * p.v_scale;
      const int64_t oi = ((int64_t)b * p.num_heads + (SPLIT ? first_head_of(p, kvh) : kvh * G) + h0 + hh) * p.head_size + d;
      if (p.out_f32)
        reinterpret_cast<float *>(p.out)[oi] = r;
      else
        reinterpret_cast<uint16_t *>(p.out)[oi] = p.out_f16 ? f32_to_16<true>(r) : f32_to_16<false>(r);
    }
  }
}

__global__ void clear_counters_kernel(uint32_t *counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0u;
}

// Scratch of vtkv_decode_attention_noalloc: partial results, prefix sums and arrival counters of one call, in
// device memory that belongs to the loaded library itself, so that the entry point has nothing to allocate.
// Every device the library runs on holds its own copy of the array at its own address until the process ends.
// In host code `g_static_scratch` only names the symbol; the address kernels can use comes from
// hipGetSymbolAddress, once per device (static_scratch_ptr below).
constexpr int64_t kStaticScratchBytes = 32ll << 20;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
struct StaticScratch {
  std::mutex mu;
  void *ptr[kMaxDevices] = {};
};
StaticScratch g_scratch_ptrs;

// Device address of the current device's copy of g_static_scratch; nullptr (and the error set) on failure.
void *static_scratch_ptr() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    vtkv::fail(VTKV_EHIP, "hipGetDevice failed or device %d is beyond %d: %s", dev, kMaxDevices, hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_scratch_ptrs.mu);
  if (!g_scratch_ptrs.ptr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess || !ptr) {
      vtkv::fail(VTKV_EHIP, "hipGetSymbolAddress of the static scratch failed: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptrs.ptr[dev] = ptr;
  }
  return g_scratch_ptrs.ptr[dev];
}

// Optional per-kernel timing for benchmarks: when switched on, every vtkv_decode_attention call
// launches its kernels with a start and a stop event each (hipExtLaunchKernelGGL: the events take the
// begin and the end of that kernel's own dispatch on the caller's stream, which is what a kernel trace
// reports; events recorded before and after a launch also contain the dispatch of the kernel and the
// completion of the event markers, 5 to 6 us here).  Nothing waits for them, so the calls stay queued
// back to back as they are in production.  Up to kTimedCalls calls are kept.
constexpr int kTimedCalls = 1024;
struct KernelTimer {
  std::atomic<bool> on{false};
  std::mutex mu;               // held by a timed call from its first event to its last, and by the readers
  std::vector<hipEvent_t> ev;  // four per call (start and stop of either kernel), created on first use
  std::vector<char> merged;    // per call: the merge ran inside the streaming kernel (no second kernel)
  int calls = 0;
};
KernelTimer g_timer;

// Workgroups of the streaming kernel that the current device holds at once (per kernel variant).
constexpr int kVariants = 16 + 24 + 2 + 18 + 28 + 6 + 18 + 10 + 4;  // instantiations of the streaming kernel: 16 of the tuned shape, 24
                                                       // others, the fused append for fp16 at head size 128 (fp16 rows,
                                                       // fp8 rows), 18 that stream several kv heads per segment at other
                                                       // shapes, 28 for kv heads of more than 16 query heads (SPLIT), 6
                                                       // whose wave tiles hold several kv heads (GW), 18 with the fused
                                                       // append for 16-bit rows of the other head sizes, 10 more of
                                                       // those for kv heads of more than 16 query heads, 4 for wave
                                                       // tiles of four kv heads at head size 112

// 64, 80, 96, 112, 128, 256 (vllm/attention/ops/paged_attn.py:33-34) -> 0..5, anything else -> -1
int head_size_index(int head_size) {
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
struct Residency {
  std::mutex mu;
  int device = -1;
  int grid[kVariants] = {};
};
Residency g_res;

template <typename K>
int resident_grid(K kernel, int variant) {
  std::lock_guard<std::mutex> lk(g_res.mu);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (g_res.device != dev) {
    g_res.device = dev;
    for (int &v : g_res.grid) v = 0;
  }
  if (g_res.grid[variant] == 0) {
    int per_cu = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, 0) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    g_res.grid[variant] = std::min(std::max(per_cu, 1) * cus, kDefaultMaxGrid);
  }
  return g_res.grid[variant];
}

// Upper bound of the number of partial slots: one per workgroup plus one per (sequence, kv head);
// each slot holds `group` heads, and num_seqs*num_kv_heads*group = num_seqs*num_heads.
int64_t scratch_floats(int64_t grid, int num_seqs, int num_heads, int head_size) {
  return (grid * 16 + (int64_t)num_seqs * num_heads) * (head_size + 2);
}

// Arrival counters, one per (sequence, kv head); sized for the largest batch so that their place in
// the workspace is fixed (num_kv_heads <= num_heads).
int64_t counter_bytes(int /*num_seqs*/, int /*num_heads*/) { return (int64_t)kMaxSeqs * kMaxKvHeads * 4; }

// Process-wide tuning knobs, settable from any thread: every call reads each of them once, at its start.
std::atomic<int> g_fused_merge{-1};  // -1: decide per call, 0: never, 1: always
std::atomic<int> g_head_major{-1};   // likewise for the head-major tile order

int64_t fixed_span_grid(int num_seqs, int num_kv_heads_bound, int max_seq_len, int partition_tokens) {
  const int64_t tiles = (int64_t)num_seqs * num_kv_heads_bound * ((max_seq_len + kTile - 1) / kTile);
  const int64_t span = partition_tokens / kTile;
  return (tiles + span - 1) / span;
}

// The caller's per-partition buffers of the reference's split-K interface (paged_attention_v2).
struct V2Side {
  float *exp_sums, *max_logits;  // [num_seqs, num_heads, max_parts]
  void *tmp_out;                 // [num_seqs, num_heads, max_parts, head_size], q's dtype
  int max_parts;
};
constexpr int kV2Partition = 512;  // rows per partition (vllm/attention/ops/paged_attn.py:10)

// One batch of at most kMaxSeqs sequences (kInlineLens with host lengths).  new_key == nullptr: attention only.
// v2 != nullptr: partitions of 512 rows aligned with the sequences, the caller's side buffers filled.
int attention_batch(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs, const int64_t *slot_ids,
                   const int32_t *seq_lens, const int32_t *host_seq_lens, int num_seqs, int num_heads,
                   int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                   const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale, float v_scale,
                   void *workspace, int64_t workspace_bytes, int partition_tokens, void *stream, const void *new_key,
                   const void *new_value, int64_t key_stride, int64_t value_stride, const V2Side *v2,
                   bool static_scratch) {
  const bool append = new_key != nullptr;
  if (v2) {
    partition_tokens = kV2Partition;
    VTKV_REQUIRE(!append, "the split-K interface has no fused append");
    VTKV_REQUIRE(v2->exp_sums && v2->max_logits && v2->tmp_out, "null argument");
    VTKV_REQUIRE(max_seq_len > 0 && v2->max_parts >= (max_seq_len + kV2Partition - 1) / kV2Partition,
                 "%d partitions do not hold %d rows", v2->max_parts, max_seq_len);
  }
  VTKV_REQUIRE(out && q && k_ptrs && v_ptrs && slot_ids, "null argument");
  VTKV_REQUIRE((seq_lens != nullptr) != (host_seq_lens != nullptr), "pass either device or host sequence lengths");
  VTKV_REQUIRE(num_seqs >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0,
               "num_heads %d must be a positive multiple of num_kv_heads %d", num_heads, num_kv_heads);
  VTKV_REQUIRE(num_seqs <= kMaxSeqs, "at most %d sequences per call, got %d", kMaxSeqs, num_seqs);
  VTKV_REQUIRE(!host_seq_lens || num_seqs <= kInlineLens, "at most %d sequence lengths can be passed from the host, got %d",
               kInlineLens, num_seqs);
  const int d_index = head_size_index(head_size);
  VTKV_REQUIRE(d_index >= 0, "head_size %d is not supported (64, 80, 96, 112, 128, 256)", head_size);
  VTKV_REQUIRE(q_dtype == VTKV_BF16 || q_dtype == VTKV_F16, "q_dtype must be BF16 or F16");
  VTKV_REQUIRE(out_dtype == q_dtype || out_dtype == VTKV_F32, "out_dtype must be q_dtype or F32");
  VTKV_REQUIRE(kv_dtype == q_dtype || kv_dtype == VTKV_FP8_E4M3, "kv_dtype must be q_dtype or FP8_E4M3");
  const bool f16 = q_dtype == VTKV_F16;
  const bool tuned = head_size == 128 && !f16;  // the shape the kernel was built around, with all its variants
  if (kv_dtype == VTKV_FP8_E4M3) VTKV_REQUIRE(k_scale > 0.f && v_scale > 0.f, "fp8 scales must be positive");
  // More than 16 query heads per kv head: the kernels see every kv head as kv_split virtual ones over the same
  // rows, each with at most 16 of its query heads (see first_head_of).  From here on num_kv_heads and group are
  // what the kernels see; kv_heads_real is what the rows in memory hold.
  const int kv_heads_real = num_kv_heads, group_real = num_heads / num_kv_heads;
  const int kv_split = vtkv_kv_split(group_real);
  int group = (group_real + kv_split - 1) / kv_split;
  num_kv_heads = kv_heads_real * kv_split;
  VTKV_REQUIRE(num_kv_heads <= kMaxKvHeads, "%d kv heads (as %d of at most 16 query heads each) exceed %d", kv_heads_real,
               num_kv_heads, kMaxKvHeads);
  VTKV_REQUIRE(q_stride >= (int64_t)num_heads * head_size && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0,
               "q rows must be 16-byte aligned and at least num_heads*head_size apart");
  VTKV_REQUIRE(max_seq_len > 0, "max_seq_len must be > 0");
  // the kernel addresses rows of a range with 32-bit byte offsets
  VTKV_REQUIRE((int64_t)max_seq_len * kv_heads_real * head_size * vtkv::elem_bytes(kv_dtype) < (1ll << 31),
               "a sequence range of %d rows exceeds 2 GiB", max_seq_len);
  VTKV_REQUIRE(partition_tokens == 0 || (partition_tokens >= kWaves * kTile && partition_tokens % kTile == 0),
               "partition_tokens must be 0 or a multiple of %d that is at least %d", kTile, kWaves * kTile);
  if (append) {
    VTKV_REQUIRE(new_value != nullptr, "null argument");
    VTKV_REQUIRE(head_size == 128 || kv_dtype == q_dtype, "the fused append at head sizes other than 128 needs 16-bit rows");
    const int64_t row = (int64_t)kv_heads_real * head_size;
    VTKV_REQUIRE(key_stride >= row && value_stride >= row && key_stride % 8 == 0 && value_stride % 8 == 0 &&
                     (uintptr_t)new_key % 16 == 0 && (uintptr_t)new_value % 16 == 0,
                 "key/value rows must be 16-byte aligned and at least num_kv_heads*head_size apart");
  }
  if (num_seqs == 0) return VTKV_OK;

  const bool fp8 = kv_dtype == VTKV_FP8_E4M3;
  const bool alibi = alibi_slopes != nullptr;
  // kv heads per segment (see the kernel): two for fp8 rows, and for bf16 rows when the batch is made of very
  // many short segments (16 or more per CU of this part), where halving the number of segment starts and
  // merges per workgroup is worth 3 to 7 % (1 024 sequences of 64..512 rows: 250 -> 235 us; 512 sequences
  // of 128..1 024 rows: 219 -> 211 us) while batches of fewer, longer sequences gain nothing or lose (the
  // merge kernel sees twice the pieces per head: config 3 152 -> 158 us).  Slots: seg_heads * grid +
  // num_seqs * num_kv_heads of `group` heads each, which the workspace (16 heads per workgroup) holds for
  // groups up to 8.
  const bool many_short = (int64_t)num_seqs * num_kv_heads >= 4096;
  const bool pair = tuned && kv_split == 1 && (fp8 ? VTKV_ATTN_FP8_PAIR != 0 : many_short) && num_kv_heads % 2 == 0 &&
                    group <= 8;
  int seg_heads = pair ? 2 : 1;
  // kernel variant of the tuned shape: bit 0 alibi, bit 1 fused append, bit 2 paired kv heads, bit 3 fp8; the
  // other head sizes and fp16 have one variant per (head size, type, cache type), ALiBi decided at run time
  int variant = tuned    ? (fp8 ? 8 : 0) + (pair ? 4 : 0) + (append ? 2 : 0) + (alibi ? 1 : 0)
                : append ? 40 + (fp8 ? 1 : 0)
                         : 16 + (d_index * 2 + (f16 ? 1 : 0)) * 2 + (fp8 ? 1 : 0);
  const bool append_other = append && head_size != 128;  // (16-bit rows: checked above)
  if (append_other) variant = 94 + (d_index < 4 ? d_index : 4) * 2 + (f16 ? 1 : 0);
  if (!tuned) {
    // A head row that is no whole number of 128-byte lines (160, 192, 224 bytes; 64 to 112 bytes of fp8 codes)
    // drags its neighbours' bytes along with every fetch, and a lone line streams slower than a pair (see the
    // kernel): where the head counts allow it, a segment then holds 2 or 4 adjacent kv heads, so that a workgroup
    // reads 256 to 896 contiguous bytes per token.  64 sequences of 512..4096 rows, 8 kv heads, share of the
    // HBM peak with one head per segment: head size 80 0.51, 96 0.60, 112 0.53, 64 0.72; fp8 rows 0.29 to 0.40.
    static const int kHeads16[6] = {2, 4, 2, 4, 1, 1}, kHeads8[6] = {4, 4, 4, 4, 2, 1};
    const int want = fp8 ? kHeads8[d_index] : kHeads16[d_index];
    if (want > 1 && kv_split == 1 && num_kv_heads % want == 0 && group * want <= 16 && (!append_other || d_index == 3)) {
      seg_heads = want;
      variant = head_size == 128 ? 58 + (append ? 1 : 0)
                : append_other   ? 110 + (f16 ? 1 : 0)
                                 : 42 + d_index * 4 + (f16 ? 2 : 0) + (fp8 ? 1 : 0);
    }
  }
  // Several kv heads per wave tile (GW, see the kernel) for 16-bit rows of head sizes 64 (2 kv heads: 256 bytes per
  // token), 80 (4: 640 bytes) and 96 (2: 384 bytes), where the heads that make whole lines have room in the 16
  // columns together.  To everything below, the GW heads are one kv head of group * GW query heads.  64 sequences
  // of 512..4096 rows, 8 kv heads of 4 query heads, stream kernel, share of the HBM peak, against one wave per head
  // with plain loads: 80: 0.675 against 0.62, 96: 0.766 against 0.67, 64: 0.73 either way; 112 (4 heads: 896 bytes
  // per token, 28 registers of 16 bytes to hold a K or V tile) spills at two waves per SIMD (0.57 against 0.66) and
  // runs one wave per SIMD instead, like head size 256: 0.715 against 0.675.  Measured and left out: fp8 rows of 64
  // and 96 with 4 (0.48 and 0.49 against 0.56 and 0.61).
  if (!tuned && !fp8 && kv_split == 1 && d_index < 4) {
    static const int kGw16[4] = {2, 4, 2, 4};
    const int gw = kGw16[d_index];
    if (num_kv_heads % gw == 0 && group * gw <= 16) {
      seg_heads = 1;
      variant = d_index < 3 ? (append ? 104 : 88) + d_index * 2 + (f16 ? 1 : 0) : (append ? 124 : 122) + (f16 ? 1 : 0);
      num_kv_heads /= gw;
      group *= gw;
    }
  }
  // kv heads of more than 16 query heads: one variant per (head size, type, cache type), the fused append at 128
  if (kv_split > 1)
    variant = append_other ? 112 + (d_index < 4 ? d_index : 4) * 2 + (f16 ? 1 : 0)
              : append     ? 84 + (f16 ? 2 : 0) + (fp8 ? 1 : 0)
                           : 60 + (d_index * 2 + (f16 ? 1 : 0)) * 2 + (fp8 ? 1 : 0);
#define VTKV_ROW(F8, H)                                                                                      \
  decode_attn_stream_kernel<false, F8, false, H>, decode_attn_stream_kernel<true, F8, false, H>,             \
      decode_attn_stream_kernel<false, F8, true, H>, decode_attn_stream_kernel<true, F8, true, H>
#define VTKV_SIZE(DD)                                                                                         \
  decode_attn_stream_kernel<true, false, false, 1, DD, false>, decode_attn_stream_kernel<true, true, false, 1, DD, false>, \
      decode_attn_stream_kernel<true, false, false, 1, DD, true>, decode_attn_stream_kernel<true, true, false, 1, DD, true>
  static void (*const kKernels[kVariants])(AttnParams, InlineLens) = {
      VTKV_ROW(false, 1), VTKV_ROW(false, 2), VTKV_ROW(true, 1), VTKV_ROW(true, 2),
      VTKV_SIZE(64), VTKV_SIZE(80), VTKV_SIZE(96), VTKV_SIZE(112), VTKV_SIZE(128), VTKV_SIZE(256),
      decode_attn_stream_kernel<true, false, true, 1, 128, true>, decode_attn_stream_kernel<true, true, true, 1, 128, true>,
#define VTKV_GROUPED(DD, H16, H8)                                                                                  \
  decode_attn_stream_kernel<true, false, false, H16, DD, false>, decode_attn_stream_kernel<true, true, false, H8, DD, false>, \
      decode_attn_stream_kernel<true, false, false, H16, DD, true>, decode_attn_stream_kernel<true, true, false, H8, DD, true>
      VTKV_GROUPED(64, 2, 4), VTKV_GROUPED(80, 4, 4), VTKV_GROUPED(96, 2, 4), VTKV_GROUPED(112, 4, 4),
#undef VTKV_GROUPED
      decode_attn_stream_kernel<true, true, false, 2, 128, true>, decode_attn_stream_kernel<true, true, true, 2, 128, true>,
#define VTKV_SPLIT(DD, APP)                                                                                               \
  decode_attn_stream_kernel<true, false, APP, 1, DD, false, true>, decode_attn_stream_kernel<true, true, APP, 1, DD, false, true>, \
      decode_attn_stream_kernel<true, false, APP, 1, DD, true, true>, decode_attn_stream_kernel<true, true, APP, 1, DD, true, true>
      VTKV_SPLIT(64, false), VTKV_SPLIT(80, false), VTKV_SPLIT(96, false), VTKV_SPLIT(112, false), VTKV_SPLIT(128, false),
      VTKV_SPLIT(256, false), VTKV_SPLIT(128, true),
#undef VTKV_SPLIT
#define VTKV_GW(DD, F8, W)                                                                                     \
  decode_attn_stream_kernel<true, F8, false, 1, DD, false, false, W>, decode_attn_stream_kernel<true, F8, false, 1, DD, true, false, W>
      VTKV_GW(64, false, 2), VTKV_GW(80, false, 4), VTKV_GW(96, false, 2),
#undef VTKV_GW
#define VTKV_APPEND16(DD, H, W)                                                                                 \
  decode_attn_stream_kernel<true, false, true, H, DD, false, false, W>, decode_attn_stream_kernel<true, false, true, H, DD, true, false, W>
      VTKV_APPEND16(64, 1, 1), VTKV_APPEND16(80, 1, 1), VTKV_APPEND16(96, 1, 1), VTKV_APPEND16(112, 1, 1), VTKV_APPEND16(256, 1, 1),
      VTKV_APPEND16(64, 1, 2), VTKV_APPEND16(80, 1, 4), VTKV_APPEND16(96, 1, 2), VTKV_APPEND16(112, 4, 1),
#undef VTKV_APPEND16
#define VTKV_SPLIT_APPEND16(DD)                                                                                 \
  decode_attn_stream_kernel<true, false, true, 1, DD, false, true>, decode_attn_stream_kernel<true, false, true, 1, DD, true, true>
      VTKV_SPLIT_APPEND16(64), VTKV_SPLIT_APPEND16(80), VTKV_SPLIT_APPEND16(96), VTKV_SPLIT_APPEND16(112),
      VTKV_SPLIT_APPEND16(256),
#undef VTKV_SPLIT_APPEND16
      decode_attn_stream_kernel<true, false, false, 1, 112, false, false, 4>, decode_attn_stream_kernel<true, false, false, 1, 112, true, false, 4>,
      decode_attn_stream_kernel<true, false, true, 1, 112, false, false, 4>, decode_attn_stream_kernel<true, false, true, 1, 112, true, false, 4>,
  };
#undef VTKV_ROW
#undef VTKV_SIZE
  void (*kernel)(AttnParams, InlineLens) = kKernels[variant];
  // the head size as the kernels hold it: padded to the MFMA depth (to 64 elements for fp8 rows)
  const int hd = fp8 ? (head_size + 63) / 64 * 64 : (head_size + 31) / 32 * 32;
  int64_t grid;
  if (v2) {
    grid = (int64_t)num_seqs * (num_kv_heads / seg_heads) * v2->max_parts;
    VTKV_REQUIRE(grid <= (1ll << 24), "%d partitions per sequence give %lld workgroups", v2->max_parts, (long long)grid);
  } else if (partition_tokens > 0) {
    // (the fused append adds one tile per sequence and kv head)
    grid = fixed_span_grid(num_seqs, num_kv_heads / seg_heads, max_seq_len + (append ? kTile : 0), partition_tokens);
    VTKV_REQUIRE(grid <= (1ll << 24), "partition_tokens %d gives %lld workgroups", partition_tokens, (long long)grid);
  } else {
    const int g = resident_grid(kernel, variant);
    if (g <= 0) return vtkv::fail(VTKV_EHIP, "cannot query the kernel's occupancy");
    grid = g;
  }
  const int64_t n_float = scratch_floats(grid, num_seqs, num_kv_heads * group, hd);
  const int64_t count_bytes = counter_bytes(num_seqs, num_heads);
  const int64_t cum_bytes = ((int64_t)(num_seqs + 1) * 4 + 15) / 16 * 16;
  const int64_t need = n_float * (int64_t)sizeof(float) + cum_bytes + count_bytes;
  if (static_scratch && workspace_bytes < need)
    return vtkv::fail(VTKV_EINVAL, "%d sequences of %d heads need %lld bytes of scratch, the library's static scratch "
                      "holds %lld: use vtkv_decode_attention with a workspace of the caller's", num_seqs, num_heads,
                      (long long)need, (long long)workspace_bytes);
  if (!workspace || workspace_bytes < need)
    return vtkv::fail(VTKV_ENOMEM, "workspace of %lld bytes is smaller than the %lld needed",
                      (long long)workspace_bytes, (long long)need);
  VTKV_REQUIRE((uintptr_t)workspace % 16 == 0, "workspace must be 16-byte aligned");

  AttnParams p;
  p.q = (const uint16_t *)q;
  p.k_ptrs = k_ptrs;
  p.v_ptrs = v_ptrs;
  p.slot_ids = slot_ids;
  p.seq_lens = seq_lens;
  p.alibi_slopes = alibi_slopes;
  const int64_t n_stat = grid * 16 + (int64_t)num_seqs * num_kv_heads * group;  // (slot, head) pairs
  // the counters come first, at a place that does not depend on the sizes of a call
  p.seg_count = (uint32_t *)workspace;
  // Merging inside the streaming kernel saves the second launch, but the workgroup that arrives last
  // does it at the very end of the kernel with device-coherent round trips (about 6 us), and every shared
  // segment costs its workgroups coherent stores and an arrival.  That pays when most (sequence, kv head)
  // segments lie inside one workgroup and need no merge at all.  Measured on 512 workgroups with ragged
  // lengths, stream kernel + merge, inside against separate (the separate form also lets every XCD take a
  // contiguous part of the tile order): 1024 segments 188 against 180 us (group 4) and 196 against 192 us
  // (group 8); 1280 segments 212 / 209 and 219 / 221; 1536 segments 206 / 205 and 217 / 222; 2048 segments
  // 201.5 / 212 and 216 / 231.  Hence inside from two and a half segments per workgroup on.
  // Where the head-major tile order applies (below) the merge inside gains more from it than the separate
  // form (torch allocations, 300 000 rows over 64..1024 ragged sequences, group 4 / group 8, inside against
  // separate, both head-major: 1 segment per workgroup 173 / 174 and 179 / 178 us; 2 segments 190 / 194 and
  // 201 / 203; 4 segments 197 / 205 and 210 / 219; 16 segments 223 / 243 and 247 / 271): inside from two
  // segments per workgroup on.
  const int knob_merge = g_fused_merge.load(std::memory_order_relaxed);
  const int knob_hm = g_head_major.load(std::memory_order_relaxed);
  const int segs_per_seq = num_kv_heads / seg_heads;
  const int64_t segs = (int64_t)num_seqs * segs_per_seq;
  // (the parts of a split kv head read the same rows: head-major only if every XCD then holds whole kv heads, else
  // each part would fetch the rows into another L2; one kv head of 64 query heads, 64 sequences: 58 us against 67)
  const bool hm_fits = partition_tokens == 0 && grid % 8 == 0 && (segs_per_seq % 8 == 0 || 8 % segs_per_seq == 0) &&
                       (kv_split == 1 || (segs_per_seq % 8 == 0 && (segs_per_seq / 8) % kv_split == 0));
  const bool hm_auto = knob_hm != 0 && hm_fits;  // the head-major order is open to this call
  p.fused_merge = !v2 && (knob_merge == 1 || (knob_merge < 0 && (hm_auto ? segs >= 2 * grid : 2 * segs >= 5 * grid)));
  p.heads_per_seg = seg_heads;
  p.reduce_sets = 1;
  p.cum_tiles = (int32_t *)((char *)workspace + count_bytes);
  p.part_out = (float *)((char *)workspace + count_bytes + cum_bytes);
  p.part_max = p.part_out + n_stat * hd;
  p.part_sum = p.part_max + n_stat;
  p.out = out;
  p.out_f32 = out_dtype == VTKV_F32;
  p.out_f16 = f16;
  p.head_size = head_size;
  p.q_stride = q_stride;
  p.num_seqs = num_seqs;
  p.num_heads = num_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = group;
  p.kv_split = kv_split;
  p.group_real = group_real;
  p.span_tiles = partition_tokens > 0 ? partition_tokens / kTile : 0;
  p.grid = (int)grid;
  // Head-major tile order (see the kernel) where it lines the kv heads up with the XCDs: a contiguous eighth
  // of the order per XCD, and eight XCDs per whole number of segments of a sequence or the other way round
  // (8 kv heads: one per XCD; 4 pairs of kv heads: a pair per two XCDs).  Without it the per-XCD span order
  // only pays with the separate merge kernel (config 5 with the merge inside lost 1.7 %).
  p.xcd_spans = partition_tokens == 0 && grid % 8 == 0 && (!p.fused_merge || hm_auto || knob_hm == 1)
                    ? (int)(grid / 8) : 0;
  p.head_major = partition_tokens == 0 && (knob_hm == 1 ? (!p.fused_merge || p.xcd_spans > 0)
                                                              : (hm_auto && p.xcd_spans > 0));
  // x = code * scale: the K scale multiplies every logit, the V scale the whole output
  p.scale_log2 = scale * kLog2e * (fp8 ? k_scale : 1.f);
  p.v_scale = fp8 ? v_scale : 1.f;
  p.new_k = (const char *)new_key;
  p.new_v = (const char *)new_value;
  p.new_k_stride = key_stride * 2;
  p.new_v_stride = value_stride * 2;
  p.k_quant = k_scale;
  p.v_quant = v_scale;
  p.inline_lens = host_seq_lens != nullptr;
  p.aligned_parts = v2 ? v2->max_parts : 0;
  p.v2_exp_sums = v2 ? v2->exp_sums : nullptr;
  p.v2_max_logits = v2 ? v2->max_logits : nullptr;
  p.v2_tmp_out = v2 ? (uint16_t *)v2->tmp_out : nullptr;
  InlineLens il;
  if (host_seq_lens) memcpy(il.v, host_seq_lens, (size_t)num_seqs * sizeof(int32_t));

  hipStream_t st = (hipStream_t)stream;
  if (static_scratch && p.fused_merge) {
    // The static scratch is shared by every call on this device and keeps what the last one left: the arrival
    // counters of this call's (sequence, kv head) pairs are cleared first (by a kernel, not a memset, so that
    // the call can be recorded into a HIP graph).
    const int n_count = num_seqs * num_kv_heads;
    hipLaunchKernelGGL(clear_counters_kernel, dim3((n_count + 255) / 256), dim3(256), 0, st, p.seg_count, n_count);
  }
  std::unique_lock<std::mutex> timer_lock(g_timer.mu, std::defer_lock);
  // timed calls take turns; the entry point that must not allocate is never timed (events are created on demand)
  if (!static_scratch && g_timer.on.load(std::memory_order_relaxed)) timer_lock.lock();
  const bool timed = timer_lock.owns_lock() && g_timer.on.load(std::memory_order_relaxed) && g_timer.calls < kTimedCalls;
  hipEvent_t *ev = nullptr;
  if (timed) {
    if ((int)g_timer.ev.size() < 4 * (g_timer.calls + 1)) {
      hipEvent_t e4[4];
      for (auto &e : e4) VTKV_HIP(hipEventCreate(&e));
      g_timer.ev.insert(g_timer.ev.end(), e4, e4 + 4);
    }
    ev = &g_timer.ev[4 * g_timer.calls];
    hipExtLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kThreads), 0, st, ev[0], ev[1], 0, p, il);
  } else {
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kThreads), 0, st, p, il);
  }
  if (!p.fused_merge) {
    // segments of at least four pieces on average: four sets of threads share a segment's pieces
    // (several workgroups per (kv head, sequence) where its heads would take more than one pass: four heads per pass
    // when the pieces of a segment are shared out over four sets of threads, else eight)
    p.reduce_sets = 4 * segs <= grid ? (group + 3) / 4 : (group + 7) / 8;
    const dim3 rgrid(num_kv_heads * p.reduce_sets, num_seqs);
#define VTKV_REDUCE_LAUNCH_(G, S, HD, SP)                                                                     \
  do {                                                                                                        \
    if (timed)                                                                                                \
      hipExtLaunchKernelGGL((decode_attn_reduce_kernel<G, S, HD, SP>), rgrid, dim3(G * S * HD), 0, st, ev[2], \
                            ev[3], 0, p);                                                                     \
    else                                                                                                      \
      hipLaunchKernelGGL((decode_attn_reduce_kernel<G, S, HD, SP>), rgrid, dim3(G * S * HD), 0, st, p);       \
  } while (0)
#define VTKV_REDUCE_LAUNCH(G, S, HD)                                                                          \
  do {                                                                                                        \
    if (kv_split > 1)                                                                                         \
      VTKV_REDUCE_LAUNCH_(G, S, HD, true);                                                                    \
    else                                                                                                      \
      VTKV_REDUCE_LAUNCH_(G, S, HD, false);                                                                   \
  } while (0)
#define VTKV_REDUCE(HD)                                                                                       \
  do {                                                                                                        \
    if (4 * segs <= grid)                                                                                     \
      VTKV_REDUCE_LAUNCH(4, 1, HD);                                                                           \
    else if (group > 4)                                                                                       \
      VTKV_REDUCE_LAUNCH(1, 2, HD);                                                                           \
    else                                                                                                      \
      VTKV_REDUCE_LAUNCH(1, 1, HD);                                                                           \
  } while (0)
    switch (hd) {
      case 64: VTKV_REDUCE(64); break;
      case 96: VTKV_REDUCE(96); break;
      case 256: VTKV_REDUCE(256); break;
      default: VTKV_REDUCE(128); break;
    }
#undef VTKV_REDUCE
#undef VTKV_REDUCE_LAUNCH
#undef VTKV_REDUCE_LAUNCH_
  }
  if (timed) {
    g_timer.merged.resize(g_timer.calls + 1);
    g_timer.merged[g_timer.calls] = p.fused_merge != 0;
    ++g_timer.calls;
  }
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

// Shared by the entry points: larger batches run as consecutive batches of kMaxSeqs sequences (kInlineLens
// when the lengths come from the host) on the caller's stream; rows of different sequences are independent and
// the scratch of a batch is free again when the next one starts on the same stream.
int attention_impl(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs, const int64_t *slot_ids,
                   const int32_t *seq_lens, const int32_t *host_seq_lens, int num_seqs, int num_heads,
                   int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                   const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale, float v_scale,
                   void *workspace, int64_t workspace_bytes, int partition_tokens, void *stream, const void *new_key,
                   const void *new_value, int64_t key_stride, int64_t value_stride, const V2Side *v2 = nullptr,
                   bool static_scratch = false) {
  if (q_dtype == VTKV_F32) {
    // float32 models: a kernel of their own over float32 rows (csrc/vtkv_attention_f32.hip)
    VTKV_REQUIRE(kv_dtype == VTKV_F32 && out_dtype == VTKV_F32, "float32 queries take a float32 cache and a float32 result");
    VTKV_REQUIRE(!new_key && !host_seq_lens, "the fused append is built for 16-bit models");
    VTKV_REQUIRE(seq_lens, "null argument");
    if (v2) VTKV_REQUIRE(v2->exp_sums && v2->max_logits && v2->tmp_out, "null argument");
    // (the start of a workspace holds the arrival counters of the 16-bit kernels, which they expect to find at
    // zero: the partial results of this path go behind them)
    const int64_t skip = counter_bytes(0, 0);
    const bool usable = workspace && workspace_bytes > skip;
    return vtkv::attention_f32((float *)out, (const float *)q, k_ptrs, v_ptrs, slot_ids, seq_lens, nullptr, 0, num_seqs,
                               num_heads, num_kv_heads, head_size, q_stride, scale, max_seq_len, alibi_slopes,
                               v2 ? v2->exp_sums : nullptr, v2 ? v2->max_logits : nullptr,
                               v2 ? (float *)v2->tmp_out : nullptr, v2 ? v2->max_parts : 0,
                               usable ? (char *)workspace + skip : nullptr, usable ? workspace_bytes - skip : 0, stream);
  }
  const int per_call = host_seq_lens ? kInlineLens : kMaxSeqs;
  if (num_seqs <= per_call || !out || !q || !slot_ids || num_heads <= 0 || head_size <= 0)
    return attention_batch(out, q, k_ptrs, v_ptrs, slot_ids, seq_lens, host_seq_lens, num_seqs, num_heads, num_kv_heads,
                           head_size, q_stride, scale, max_seq_len, alibi_slopes, q_dtype, out_dtype, kv_dtype, k_scale,
                           v_scale, workspace, workspace_bytes, partition_tokens, stream, new_key, new_value, key_stride,
                           value_stride, v2, static_scratch);
  const int64_t out_row = (int64_t)num_heads * head_size * (out_dtype == VTKV_F32 ? 4 : 2);
  for (int at = 0; at < num_seqs; at += per_call) {
    const int n = std::min(per_call, num_seqs - at);
    V2Side side;
    if (v2) {
      const int64_t rows = (int64_t)at * num_heads * v2->max_parts;
      side = *v2;
      if (side.exp_sums) side.exp_sums += rows;
      if (side.max_logits) side.max_logits += rows;
      if (side.tmp_out) side.tmp_out = (char *)side.tmp_out + rows * head_size * 2;
    }
    int rc = attention_batch((char *)out + at * out_row, (const char *)q + (int64_t)at * q_stride * 2, k_ptrs, v_ptrs,
                             slot_ids + at, seq_lens ? seq_lens + at : nullptr,
                             host_seq_lens ? host_seq_lens + at : nullptr, n, num_heads, num_kv_heads, head_size,
                             q_stride, scale, max_seq_len, alibi_slopes, q_dtype, out_dtype, kv_dtype, k_scale, v_scale,
                             workspace, workspace_bytes, partition_tokens, stream,
                             new_key ? (const char *)new_key + (int64_t)at * key_stride * 2 : nullptr,
                             new_value ? (const char *)new_value + (int64_t)at * value_stride * 2 : nullptr, key_stride,
                             value_stride, v2 ? &side : nullptr, static_scratch);
    if (rc < 0) return rc;
  }
  return VTKV_OK;
}

}  // namespace

extern "C" {

int64_t vtkv_decode_attention_workspace_bytes(int num_seqs, int num_heads, int head_size, int max_seq_len,
                                              int partition_tokens) {
  if (num_seqs <= 0 || num_heads <= 0 || head_size <= 0 || max_seq_len <= 0) return 0;
  const int64_t grid = partition_tokens >= kTile
                           ? fixed_span_grid(num_seqs, num_heads, max_seq_len + kTile, partition_tokens)
                           : kDefaultMaxGrid;
  const int64_t cum_bytes = ((int64_t)(num_seqs + 1) * 4 + 15) / 16 * 16;
  // (the kernels hold a head size padded to 32 elements, to 64 for fp8 rows: sized for the larger)
  // (kv heads with more than 16 query heads are served in parts that may leave some of their 16 places empty:
  // at most one sixteenth more places than heads)
  return scratch_floats(grid, num_seqs, num_heads + num_heads / 16, (head_size + 63) / 64 * 64) * (int64_t)sizeof(float) +
         cum_bytes + counter_bytes(num_seqs, num_heads);
}

int vtkv_decode_attention(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                          const int64_t *slot_ids, const int32_t *seq_lens, int num_seqs, int num_heads,
                          int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                          const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                          float v_scale, void *workspace, int64_t workspace_bytes, int partition_tokens,
                          void *stream) {
  VTKV_REQUIRE(seq_lens, "null argument");
  return attention_impl(out, q, k_ptrs, v_ptrs, slot_ids, seq_lens, nullptr, num_seqs, num_heads, num_kv_heads,
                        head_size, q_stride, scale, max_seq_len, alibi_slopes, q_dtype, out_dtype, kv_dtype, k_scale,
                        v_scale, workspace, workspace_bytes, partition_tokens, stream, nullptr, nullptr, 0, 0);
}

int64_t vtkv_decode_attention_v2_workspace_bytes(int num_seqs, int num_heads, int head_size, int max_num_partitions) {
  if (num_seqs <= 0 || num_heads <= 0 || head_size <= 0 || max_num_partitions <= 0) return 0;
  const int64_t grid = (int64_t)num_seqs * num_heads * max_num_partitions;  // at most one workgroup per head
  const int64_t cum_bytes = ((int64_t)(num_seqs + 1) * 4 + 15) / 16 * 16;
  // (the kernels hold a head size padded to 32 elements, to 64 for fp8 rows: sized for the larger)
  return scratch_floats(grid, num_seqs, num_heads + num_heads / 16, (head_size + 63) / 64 * 64) * (int64_t)sizeof(float) +
         cum_bytes + counter_bytes(num_seqs, num_heads);
}

int vtkv_decode_attention_v2(void *out, float *exp_sums, float *max_logits, void *tmp_out, const void *q,
                             const int64_t *k_ptrs, const int64_t *v_ptrs, const int64_t *slot_ids,
                             const int32_t *seq_lens, int num_seqs, int num_heads, int num_kv_heads, int head_size,
                             int64_t q_stride, float scale, int max_seq_len, int max_num_partitions,
                             const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                             float v_scale, void *workspace, int64_t workspace_bytes, void *stream) {
  VTKV_REQUIRE(seq_lens, "null argument");
  const V2Side side = {exp_sums, max_logits, tmp_out, max_num_partitions};
  return attention_impl(out, q, k_ptrs, v_ptrs, slot_ids, seq_lens, nullptr, num_seqs, num_heads, num_kv_heads,
                        head_size, q_stride, scale, max_seq_len, alibi_slopes, q_dtype, out_dtype, kv_dtype, k_scale,
                        v_scale, workspace, workspace_bytes, kV2Partition, stream, nullptr, nullptr, 0, 0, &side);
}

int64_t vtkv_decode_attention_noalloc_max_bytes(void) { return kStaticScratchBytes; }

int vtkv_decode_attention_noalloc(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                                  const int64_t *slot_ids, const int32_t *seq_lens, int num_seqs, int num_heads,
                                  int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                                  const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                                  float v_scale, void *stream) {
  VTKV_REQUIRE(seq_lens, "null argument");
  void *scratch = static_scratch_ptr();
  if (!scratch) return VTKV_EHIP;
  return attention_impl(out, q, k_ptrs, v_ptrs, slot_ids, seq_lens, nullptr, num_seqs, num_heads, num_kv_heads,
                        head_size, q_stride, scale, max_seq_len, alibi_slopes, q_dtype, out_dtype, kv_dtype, k_scale,
                        v_scale, scratch, kStaticScratchBytes, 0, stream, nullptr, nullptr, 0, 0, nullptr, true);
}

int vtkv_decode_append_attention(void *out, const void *q, const void *key, const void *value, int64_t key_stride,
                                 int64_t value_stride, const int64_t *k_ptrs, const int64_t *v_ptrs,
                                 const int64_t *slot_ids, const int32_t *seq_lens, const int32_t *host_seq_lens,
                                 int num_seqs, int num_heads, int num_kv_heads, int head_size, int64_t q_stride,
                                 float scale, int max_seq_len, const float *alibi_slopes, int q_dtype, int out_dtype,
                                 int kv_dtype, float k_scale, float v_scale, void *workspace, int64_t workspace_bytes,
                                 int partition_tokens, void *stream) {
  VTKV_REQUIRE(key && value, "null argument");
  return attention_impl(out, q, k_ptrs, v_ptrs, slot_ids, seq_lens, host_seq_lens, num_seqs, num_heads, num_kv_heads,
                        head_size, q_stride, scale, max_seq_len, alibi_slopes, q_dtype, out_dtype, kv_dtype, k_scale,
                        v_scale, workspace, workspace_bytes, partition_tokens, stream, key, value, key_stride,
                        value_stride);
}

#ifdef VTKV_ATTN_TRACE
__attribute__((visibility("default"))) int vtkv_debug_attn_trace(unsigned long long *out, int n) {
  VTKV_HIP(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_attn_trace), (size_t)n * 6 * sizeof(unsigned long long)));
  return VTKV_OK;
}
#endif

int vtkv_set_head_major(int on) {
  g_head_major.store(on < 0 ? -1 : (on != 0), std::memory_order_relaxed);
  return VTKV_OK;
}

int vtkv_set_fused_merge(int on) {
  g_fused_merge.store(on < 0 ? -1 : (on != 0), std::memory_order_relaxed);
  return VTKV_OK;
}

int vtkv_set_kernel_timing(int on) {
  std::lock_guard<std::mutex> lk(g_timer.mu);
  g_timer.on.store(on != 0, std::memory_order_relaxed);
  if (on) g_timer.calls = 0;
  return VTKV_OK;
}

int vtkv_attention_kernel_times(float *stream_ms, float *reduce_ms, int capacity) {
  VTKV_REQUIRE(stream_ms && reduce_ms && capacity >= 0, "null argument");
  std::lock_guard<std::mutex> lk(g_timer.mu);
  const int n = std::min(capacity, g_timer.calls);
  for (int i = 0; i < n; ++i) {
    hipEvent_t *ev = &g_timer.ev[4 * i];
    VTKV_HIP(hipEventSynchronize(ev[1]));
    VTKV_HIP(hipEventElapsedTime(&stream_ms[i], ev[0], ev[1]));
    reduce_ms[i] = 0.f;
    if (!g_timer.merged[i]) {
      VTKV_HIP(hipEventSynchronize(ev[3]));
      VTKV_HIP(hipEventElapsedTime(&reduce_ms[i], ev[2], ev[3]));
    }
  }
  return n;
}

}  // extern "C"
