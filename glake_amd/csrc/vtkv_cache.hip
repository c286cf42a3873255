// Cache ops of the vTensor KV path for gfx950: scatter of new K/V rows into each sequence's
// contiguous range (with optional fp8 e4m3fn quantisation), the upstream paged scatter, block
// copies, fp8 conversion and the host<->device swap paths.
//
// All kernels move bytes: they are bound by HBM bandwidth or, at decode-step sizes, by launch
// latency, so they use 16-byte loads and stores and nothing else.
#include <algorithm>
#include <mutex>
#include <vector>

#include "vtkv_common.h"
#include "vtkv_fp8.h"

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------------------------
// vTensor scatter (replaces vllm::reshape_and_cache_kernel, csrc/cache_kernels.cu:153-200).
// grid (batch, max_seq_len); one workgroup copies the K row and the V row of one token.
// A row is row_bytes = Hkv*D*elem contiguous bytes on both sides, so lanes move 16 bytes each;
// the first half of the workgroup's lanes takes K, the second half V.
template <bool ALIGNED16>
__global__ void __launch_bounds__(256) scatter_rows_kernel(const char *__restrict__ key,
                                                           const char *__restrict__ value,
                                                           const int64_t *__restrict__ k_ptrs,
                                                           const int64_t *__restrict__ v_ptrs,
                                                           const int64_t *__restrict__ slot_m,
                                                           const int64_t *__restrict__ slot_ids,
                                                           const int32_t *__restrict__ seq_lens,
                                                           const int32_t *__restrict__ cache_seq_lens,
                                                           int max_seq_len, int row_bytes, int64_t key_stride_bytes,
                                                           int64_t value_stride_bytes) {
  const int b = blockIdx.x, t = blockIdx.y;
  if (max_seq_len != 1 && t >= seq_lens[b]) return;
  const int64_t off = slot_m[b];
  if (off < 0) return;
  const int64_t slot = slot_ids[b];
  const int64_t src_row = max_seq_len == 1 ? (int64_t)b : (int64_t)cache_seq_lens[b] + t;
  const int half = blockDim.x >> 1;
  const bool is_v = threadIdx.x >= half;
  const int lane = is_v ? threadIdx.x - half : threadIdx.x;
  const char *src = is_v ? value + src_row * value_stride_bytes : key + src_row * key_stride_bytes;
  char *dst = reinterpret_cast<char *>(is_v ? v_ptrs[slot] : k_ptrs[slot]) + off + (int64_t)t * row_bytes;
  if (ALIGNED16) {
    for (int i = lane * 16; i < row_bytes; i += half * 16)
      *reinterpret_cast<u32x4 *>(dst + i) = *reinterpret_cast<const u32x4 *>(src + i);
  } else {
    for (int i = lane * 2; i < row_bytes; i += half * 2)
      *reinterpret_cast<uint16_t *>(dst + i) = *reinterpret_cast<const uint16_t *>(src + i);
  }
}

// Same scatter with quantisation to fp8 e4m3fn: code = encode(x / scale).  Each lane converts
// 8 source elements (16 bytes of bf16) into 8 code bytes.
template <int SRC_DTYPE>
__device__ __forceinline__ float load_as_f32(const char *p, int i) {
  if (SRC_DTYPE == VTKV_F32) return reinterpret_cast<const float *>(p)[i];
  if (SRC_DTYPE == VTKV_BF16) return vtkv::bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p)[i]);
  return (float)reinterpret_cast<const _Float16 *>(p)[i];
}

template <int SRC_DTYPE>
__global__ void __launch_bounds__(256) scatter_rows_fp8_kernel(const char *__restrict__ key,
                                                               const char *__restrict__ value,
                                                               const int64_t *__restrict__ k_ptrs,
                                                               const int64_t *__restrict__ v_ptrs,
                                                               const int64_t *__restrict__ slot_m,
                                                               const int64_t *__restrict__ slot_ids,
                                                               const int32_t *__restrict__ seq_lens,
                                                               const int32_t *__restrict__ cache_seq_lens,
                                                               int max_seq_len, int row_elems,
                                                               int64_t key_stride_bytes, int64_t value_stride_bytes,
                                                               float k_scale, float v_scale) {
  const int b = blockIdx.x, t = blockIdx.y;
  if (max_seq_len != 1 && t >= seq_lens[b]) return;
  const int64_t off = slot_m[b];
  if (off < 0) return;
  const int64_t slot = slot_ids[b];
  const int64_t src_row = max_seq_len == 1 ? (int64_t)b : (int64_t)cache_seq_lens[b] + t;
  const int half = blockDim.x >> 1;
  const bool is_v = threadIdx.x >= half;
  const int lane = is_v ? threadIdx.x - half : threadIdx.x;
  const char *src = is_v ? value + src_row * value_stride_bytes : key + src_row * key_stride_bytes;
  const float scale = is_v ? v_scale : k_scale;
  uint8_t *dst = reinterpret_cast<uint8_t *>(is_v ? v_ptrs[slot] : k_ptrs[slot]) + off + (int64_t)t * row_elems;
  for (int i = lane * 8; i < row_elems; i += half * 8) {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo |= (uint32_t)vtkv::fp8_e4m3fn_encode(load_as_f32<SRC_DTYPE>(src, i + j) / scale) << (8 * j);
      hi |= (uint32_t)vtkv::fp8_e4m3fn_encode(load_as_f32<SRC_DTYPE>(src, i + 4 + j) / scale) << (8 * j);
    }
    u32x2 v = {lo, hi};
    *reinterpret_cast<u32x2 *>(dst + i) = v;
  }
}

// ---------------------------------------------------------------------------------------------
// Upstream paged scatter (csrc/cpu/cache.cpp:34-81): K [nb,H,D/x,bs,x] gets x-element (16-byte)
// groups, V [nb,H,D,bs] single elements.  grid (num_tokens), one lane per 16-byte K group.
template <int EB>
__global__ void __launch_bounds__(256) scatter_paged_kernel(const char *__restrict__ key,
                                                            const char *__restrict__ value,
                                                            char *__restrict__ key_cache,
                                                            char *__restrict__ value_cache,
                                                            const int64_t *__restrict__ slot_mapping, int num_heads,
                                                            int head_size, int block_size,
                                                            int64_t key_stride_bytes, int64_t value_stride_bytes) {
  constexpr int X = 16 / EB;
  const int64_t tok = blockIdx.x;
  const int64_t slot = slot_mapping[tok];
  if (slot < 0) return;
  const int64_t blk = slot / block_size, off = slot % block_size;
  const int n = num_heads * head_size;
  const int64_t block_elems = (int64_t)n * block_size;
  for (int i = threadIdx.x * X; i < n; i += blockDim.x * X) {
    const int h = i / head_size, d = i % head_size;
    const int64_t head_base = block_elems * blk + (int64_t)h * block_size * head_size;
    const u32x4 kv = *reinterpret_cast<const u32x4 *>(key + tok * key_stride_bytes + (int64_t)i * EB);
    *reinterpret_cast<u32x4 *>(key_cache + (head_base + (int64_t)d * block_size + off * X) * EB) = kv;
    const char *vs = value + tok * value_stride_bytes + (int64_t)i * EB;
#pragma unroll
    for (int j = 0; j < X; ++j) {
      char *vd = value_cache + (head_base + (int64_t)(d + j) * block_size + off) * EB;
      if (EB == 2)
        *reinterpret_cast<uint16_t *>(vd) = *reinterpret_cast<const uint16_t *>(vs + j * EB);
      else if (EB == 4)
        *reinterpret_cast<uint32_t *>(vd) = *reinterpret_cast<const uint32_t *>(vs + j * EB);
      else
        *vd = vs[j];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Scatter into the flash-attention cache layout (replaces vllm::reshape_and_cache_flash_kernel,
// csrc/cache_kernels.cu:202-236): K and V caches are both [num_blocks, block_size, H, D], so a token's row is
// H*D contiguous elements on both sides.  grid (num_tokens); half of the lanes take K, half V, 16 bytes each.
template <bool ALIGNED16>
__global__ void __launch_bounds__(256) scatter_flash_kernel(const char *__restrict__ key, const char *__restrict__ value,
                                                            char *__restrict__ k_cache, char *__restrict__ v_cache,
                                                            const int64_t *__restrict__ slot_mapping, int block_size,
                                                            int row_bytes, int64_t block_stride_bytes,
                                                            int64_t key_stride_bytes, int64_t value_stride_bytes) {
  const int64_t tok = blockIdx.x;
  const int64_t slot = slot_mapping[tok];
  if (slot < 0) return;  // a padded token
  const int64_t blk = slot / block_size, off = slot % block_size;
  const int half = blockDim.x >> 1;
  const bool is_v = threadIdx.x >= half;
  const int lane = is_v ? threadIdx.x - half : threadIdx.x;
  const char *src = is_v ? value + tok * value_stride_bytes : key + tok * key_stride_bytes;
  char *dst = (is_v ? v_cache : k_cache) + blk * block_stride_bytes + off * (int64_t)row_bytes;
  if (ALIGNED16) {
    for (int i = lane * 16; i < row_bytes; i += half * 16)
      *reinterpret_cast<u32x4 *>(dst + i) = *reinterpret_cast<const u32x4 *>(src + i);
  } else {
    for (int i = lane * 2; i < row_bytes; i += half * 2)
      *reinterpret_cast<uint16_t *>(dst + i) = *reinterpret_cast<const uint16_t *>(src + i);
  }
}

// ---------------------------------------------------------------------------------------------
// Block copies across layers (replaces vllm::copy_blocks_kernel, csrc/cache_kernels.cu:74-100).
// grid (layers of this launch, num_pairs).  The layers' base addresses travel in the kernel-argument block,
// up to kCopyLayers per launch: nothing to allocate, upload or wait for on the host (the reference builds two
// device tensors of pointers per call, csrc/cache_kernels.cu:117-132).
constexpr int kCopyLayers = 128;
struct LayerTable {
  uint64_t key[kCopyLayers], value[kCopyLayers];
};
__global__ void __launch_bounds__(256) copy_blocks_kernel(LayerTable layers, const int64_t *__restrict__ mapping,
                                                          int64_t block_bytes) {
  const int layer = blockIdx.x, pair = blockIdx.y;
  const int64_t src = mapping[2 * pair] * block_bytes, dst = mapping[2 * pair + 1] * block_bytes;
  char *kc = reinterpret_cast<char *>(layers.key[layer]);
  char *vc = reinterpret_cast<char *>(layers.value[layer]);
  for (int64_t i = (int64_t)threadIdx.x * 16; i < block_bytes; i += (int64_t)blockDim.x * 16) {
    *reinterpret_cast<u32x4 *>(kc + dst + i) = *reinterpret_cast<const u32x4 *>(kc + src + i);
    *reinterpret_cast<u32x4 *>(vc + dst + i) = *reinterpret_cast<const u32x4 *>(vc + src + i);
  }
}

// ---------------------------------------------------------------------------------------------
// Elementwise fp8 conversion (replaces vllm::convert_fp8_kernel, csrc/cache_kernels.cu:346-357).
template <int WIDE>
__global__ void __launch_bounds__(256) to_fp8_kernel(uint8_t *__restrict__ dst, const char *__restrict__ src,
                                                     int64_t n, float scale) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float x;
    if (WIDE == VTKV_F32) x = reinterpret_cast<const float *>(src)[i];
    else if (WIDE == VTKV_BF16) x = vtkv::bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(src)[i]);
    else x = (float)reinterpret_cast<const _Float16 *>(src)[i];
    dst[i] = vtkv::fp8_e4m3fn_encode(x / scale);
  }
}

template <int WIDE>
__global__ void __launch_bounds__(256) from_fp8_kernel(char *__restrict__ dst, const uint8_t *__restrict__ src,
                                                       int64_t n, float scale) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float x = vtkv::fp8_e4m3fn_decode(src[i]) * scale;
    if (WIDE == VTKV_F32) reinterpret_cast<float *>(dst)[i] = x;
    else if (WIDE == VTKV_BF16) reinterpret_cast<uint16_t *>(dst)[i] = vtkv::f32_to_bf16_bits_rne(x);
    else reinterpret_cast<_Float16 *>(dst)[i] = (_Float16)x;
  }
}

hipMemcpyKind copy_kind(int direction) {
  return direction == VTKV_D2H ? hipMemcpyDeviceToHost
                               : direction == VTKV_H2D ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
}

// Internal copy streams and events of vtkv_swap_ranges, created on first use per device.
struct SwapCtx {
  std::mutex mu;
  int device = -1;
  hipStream_t streams[8] = {};
  hipEvent_t fork = nullptr;
  hipEvent_t join[8] = {};
  int n_streams = 0;
};
SwapCtx g_swap;

}  // namespace

extern "C" {

int vtkv_reshape_and_cache(const void *key, const void *value, const int64_t *k_ptrs, const int64_t *v_ptrs,
                           const int64_t *slot_m, const int64_t *slot_ids, const int32_t *seq_lens,
                           const int32_t *cache_seq_lens, int batch, int max_seq_len, int num_heads, int head_size,
                           int64_t key_stride, int64_t value_stride, int src_dtype, int kv_dtype, float k_scale,
                           float v_scale, void *stream) {
  VTKV_REQUIRE(key && value && k_ptrs && v_ptrs && slot_m && slot_ids, "null argument");
  VTKV_REQUIRE(batch >= 0 && max_seq_len >= 1 && num_heads > 0 && head_size > 0, "bad sizes");
  VTKV_REQUIRE(max_seq_len == 1 || (seq_lens && cache_seq_lens), "seq_lens and cache_seq_lens are needed when max_seq_len > 1");
  VTKV_REQUIRE(max_seq_len <= 65535, "max_seq_len %d exceeds the grid limit 65535", max_seq_len);
  const int eb = vtkv::elem_bytes(src_dtype);
  VTKV_REQUIRE(eb == 2 || eb == 4, "src_dtype must be F32, BF16 or F16");
  const int row_elems = num_heads * head_size;
  VTKV_REQUIRE(key_stride >= row_elems && value_stride >= row_elems, "row stride smaller than a row");
  if (batch == 0) return VTKV_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(batch, max_seq_len);
  const char *k = (const char *)key, *v = (const char *)value;
  if (kv_dtype == src_dtype) {
    const int row_bytes = row_elems * eb;
    const bool aligned = row_bytes % 16 == 0 && (key_stride * eb) % 16 == 0 && (value_stride * eb) % 16 == 0 &&
                         ((uintptr_t)key % 16 == 0) && ((uintptr_t)value % 16 == 0);
    VTKV_REQUIRE(row_bytes % 2 == 0, "row bytes must be even");
    // 2 x (row_bytes/16) lanes cover K and V in one pass when the row is 2 KiB (Hkv=8, D=128, bf16)
    int threads = aligned ? std::min(256, std::max(64, 2 * ((row_bytes / 16 + 31) / 32 * 32))) : 256;
    if (aligned)
      hipLaunchKernelGGL(scatter_rows_kernel<true>, grid, dim3(threads), 0, st, k, v, k_ptrs, v_ptrs, slot_m,
                         slot_ids, seq_lens, cache_seq_lens, max_seq_len, row_bytes, key_stride * eb,
                         value_stride * eb);
    else
      hipLaunchKernelGGL(scatter_rows_kernel<false>, grid, dim3(threads), 0, st, k, v, k_ptrs, v_ptrs, slot_m,
                         slot_ids, seq_lens, cache_seq_lens, max_seq_len, row_bytes, key_stride * eb,
                         value_stride * eb);
  } else if (kv_dtype == VTKV_FP8_E4M3) {
    VTKV_REQUIRE(row_elems % 8 == 0, "fp8 scatter needs num_heads*head_size to be a multiple of 8");
    VTKV_REQUIRE(k_scale > 0.f && v_scale > 0.f, "fp8 scales must be positive");
    const int threads = 256;
#define LAUNCH_FP8(DT)                                                                                            \
  hipLaunchKernelGGL(scatter_rows_fp8_kernel<DT>, grid, dim3(threads), 0, st, k, v, k_ptrs, v_ptrs, slot_m,       \
                     slot_ids, seq_lens, cache_seq_lens, max_seq_len, row_elems, key_stride * eb, value_stride * eb, \
                     k_scale, v_scale)
    if (src_dtype == VTKV_F32) LAUNCH_FP8(VTKV_F32);
    else if (src_dtype == VTKV_BF16) LAUNCH_FP8(VTKV_BF16);
    else LAUNCH_FP8(VTKV_F16);
#undef LAUNCH_FP8
  } else {
    return vtkv::fail(VTKV_EINVAL, "kv_dtype %d must equal src_dtype %d or be FP8_E4M3", kv_dtype, src_dtype);
  }
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

int vtkv_reshape_and_cache_paged(const void *key, const void *value, void *key_cache, void *value_cache,
                                 const int64_t *slot_mapping, int num_tokens, int num_heads, int head_size,
                                 int block_size, int64_t key_stride, int64_t value_stride, int elem_bytes,
                                 void *stream) {
  VTKV_REQUIRE(key && value && key_cache && value_cache && slot_mapping, "null argument");
  VTKV_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, "elem_bytes must be 1, 2 or 4");
  const int x = 16 / elem_bytes;
  VTKV_REQUIRE(num_heads > 0 && head_size > 0 && head_size % x == 0 && block_size > 0, "bad sizes");
  VTKV_REQUIRE((key_stride * elem_bytes) % 16 == 0 && (value_stride * elem_bytes) % 16 == 0 &&
                   (uintptr_t)key % 16 == 0 && (uintptr_t)key_cache % 16 == 0,
               "key rows and the key cache must be 16-byte aligned");
  if (num_tokens <= 0) return VTKV_OK;
  hipStream_t st = (hipStream_t)stream;
  const int threads = std::min(256, std::max(64, (num_heads * head_size / x + 63) / 64 * 64));
#define LAUNCH_PAGED(EB)                                                                                          \
  hipLaunchKernelGGL(scatter_paged_kernel<EB>, dim3(num_tokens), dim3(threads), 0, st, (const char *)key,         \
                     (const char *)value, (char *)key_cache, (char *)value_cache, slot_mapping, num_heads,        \
                     head_size, block_size, key_stride * EB, value_stride * EB)
  if (elem_bytes == 4) LAUNCH_PAGED(4);
  else if (elem_bytes == 2) LAUNCH_PAGED(2);
  else LAUNCH_PAGED(1);
#undef LAUNCH_PAGED
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

int vtkv_swap_blocks(const void *src, void *dst, int64_t block_bytes, const int64_t *mapping, int num_pairs,
                     int direction, void *stream) {
  VTKV_REQUIRE(src && dst && block_bytes > 0 && num_pairs >= 0 && (num_pairs == 0 || mapping), "bad argument");
  VTKV_REQUIRE(direction >= VTKV_D2H && direction <= VTKV_D2D, "bad direction");
  const hipMemcpyKind kind = copy_kind(direction);
  hipStream_t st = (hipStream_t)stream;
  int i = 0;
  while (i < num_pairs) {
    // merge runs where both source and destination blocks are consecutive into one copy
    int j = i + 1;
    while (j < num_pairs && mapping[2 * j] == mapping[2 * (j - 1)] + 1 &&
           mapping[2 * j + 1] == mapping[2 * (j - 1) + 1] + 1)
      ++j;
    VTKV_REQUIRE(mapping[2 * i] >= 0 && mapping[2 * i + 1] >= 0, "negative block number");
    VTKV_HIP(hipMemcpyAsync((char *)dst + mapping[2 * i + 1] * block_bytes,
                            (const char *)src + mapping[2 * i] * block_bytes, (size_t)(j - i) * block_bytes, kind,
                            st));
    i = j;
  }
  return VTKV_OK;
}

int vtkv_swap_ranges(const uint64_t *src, const uint64_t *dst, const int64_t *bytes, int n, int direction,
                     int64_t piece_bytes, int num_streams, void *stream) {
  VTKV_REQUIRE(n >= 0 && (n == 0 || (src && dst && bytes)), "null argument");
  VTKV_REQUIRE(direction >= VTKV_D2H && direction <= VTKV_D2D, "bad direction");
  if (piece_bytes <= 0) piece_bytes = 16ll << 20;
  if (num_streams <= 0) num_streams = 2;
  VTKV_REQUIRE(num_streams <= 8, "at most 8 copy streams");
  if (n == 0) return VTKV_OK;
  const hipMemcpyKind kind = copy_kind(direction);
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lk(g_swap.mu);
  int dev = 0;
  VTKV_HIP(hipGetDevice(&dev));
  if (g_swap.device != dev) {
    VTKV_REQUIRE(g_swap.device < 0, "swap streams already belong to device %d", g_swap.device);
    g_swap.device = dev;
    VTKV_HIP(hipEventCreateWithFlags(&g_swap.fork, hipEventDisableTiming));
  }
  while (g_swap.n_streams < num_streams) {
    // default priority on purpose: streams of mixed priority are not used anywhere in this library
    VTKV_HIP(hipStreamCreateWithFlags(&g_swap.streams[g_swap.n_streams], hipStreamNonBlocking));
    VTKV_HIP(hipEventCreateWithFlags(&g_swap.join[g_swap.n_streams], hipEventDisableTiming));
    ++g_swap.n_streams;
  }
  // fork: the copy streams start after what the caller already queued
  VTKV_HIP(hipEventRecord(g_swap.fork, st));
  for (int s = 0; s < num_streams; ++s) VTKV_HIP(hipStreamWaitEvent(g_swap.streams[s], g_swap.fork, 0));
  int rr = 0;
  for (int i = 0; i < n; ++i) {
    VTKV_REQUIRE(bytes[i] >= 0, "negative size");
    for (int64_t off = 0; off < bytes[i]; off += piece_bytes) {
      const int64_t len = std::min(piece_bytes, bytes[i] - off);
      VTKV_HIP(hipMemcpyAsync((void *)(uintptr_t)(dst[i] + off), (const void *)(uintptr_t)(src[i] + off),
                              (size_t)len, kind, g_swap.streams[rr]));
      rr = (rr + 1) % num_streams;
    }
  }
  // join: the caller's stream continues once every copy stream is done
  for (int s = 0; s < num_streams; ++s) {
    VTKV_HIP(hipEventRecord(g_swap.join[s], g_swap.streams[s]));
    VTKV_HIP(hipStreamWaitEvent(st, g_swap.join[s], 0));
  }
  return VTKV_OK;
}

int vtkv_copy_blocks(const uint64_t *key_caches, const uint64_t *value_caches, int num_layers,
                     const int64_t *mapping, int num_pairs, int64_t block_bytes, void *stream) {
  VTKV_REQUIRE(num_layers >= 0 && num_pairs >= 0, "bad counts");
  if (num_layers == 0 || num_pairs == 0) return VTKV_OK;
  VTKV_REQUIRE(key_caches && value_caches && mapping, "null argument");
  VTKV_REQUIRE(block_bytes > 0 && block_bytes % 16 == 0, "block_bytes must be a positive multiple of 16");
  VTKV_REQUIRE(num_pairs <= 65535, "more than 65535 pairs in one call");
  hipStream_t st = (hipStream_t)stream;
  for (int at = 0; at < num_layers; at += kCopyLayers) {
    const int n = std::min(kCopyLayers, num_layers - at);
    LayerTable layers = {};
    for (int l = 0; l < n; ++l) {
      VTKV_REQUIRE(key_caches[at + l] % 16 == 0 && value_caches[at + l] % 16 == 0, "caches must be 16-byte aligned");
      layers.key[l] = key_caches[at + l];
      layers.value[l] = value_caches[at + l];
    }
    hipLaunchKernelGGL(copy_blocks_kernel, dim3(n, num_pairs), dim3(256), 0, st, layers, mapping, block_bytes);
  }
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

int vtkv_reshape_and_cache_flash(const void *key, const void *value, void *k_cache, void *v_cache,
                                 const int64_t *slot_mapping, int num_tokens, int num_heads, int head_size,
                                 int block_size, int64_t block_stride, int64_t key_stride, int64_t value_stride,
                                 int elem_bytes, void *stream) {
  VTKV_REQUIRE(key && value && k_cache && v_cache && slot_mapping, "null argument");
  VTKV_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "elem_bytes must be 2 or 4");
  VTKV_REQUIRE(num_heads > 0 && head_size > 0 && block_size > 0, "bad sizes");
  const int64_t row_elems = (int64_t)num_heads * head_size;
  VTKV_REQUIRE(key_stride >= row_elems && value_stride >= row_elems && block_stride >= row_elems * block_size,
               "a stride is smaller than what it steps over");
  if (num_tokens <= 0) return VTKV_OK;
  const int row_bytes = (int)(row_elems * elem_bytes);
  const bool aligned = row_bytes % 16 == 0 && (key_stride * elem_bytes) % 16 == 0 && (value_stride * elem_bytes) % 16 == 0 &&
                       (block_stride * elem_bytes) % 16 == 0 && (uintptr_t)key % 16 == 0 && (uintptr_t)value % 16 == 0 &&
                       (uintptr_t)k_cache % 16 == 0 && (uintptr_t)v_cache % 16 == 0;
  const int threads = aligned ? std::min(256, std::max(64, 2 * ((row_bytes / 16 + 31) / 32 * 32))) : 256;
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH_FLASH(A)                                                                                          \
  hipLaunchKernelGGL(scatter_flash_kernel<A>, dim3(num_tokens), dim3(threads), 0, st, (const char *)key,         \
                     (const char *)value, (char *)k_cache, (char *)v_cache, slot_mapping, block_size, row_bytes, \
                     block_stride * elem_bytes, key_stride * elem_bytes, value_stride * elem_bytes)
  if (aligned) LAUNCH_FLASH(true); else LAUNCH_FLASH(false);
#undef LAUNCH_FLASH
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

int vtkv_convert_fp8(void *dst, const void *src, int64_t n, float scale, int to_fp8, int wide_dtype, void *stream) {
  VTKV_REQUIRE(n >= 0 && (n == 0 || (dst && src)), "null argument");
  VTKV_REQUIRE(scale > 0.f, "scale must be positive");
  VTKV_REQUIRE(wide_dtype == VTKV_F32 || wide_dtype == VTKV_BF16 || wide_dtype == VTKV_F16, "bad wide dtype");
  if (n == 0) return VTKV_OK;
  hipStream_t st = (hipStream_t)stream;
  const int blocks = (int)std::min<int64_t>((n + 255) / 256, 256 * 32);
#define LAUNCH_CVT(W)                                                                                             \
  if (to_fp8)                                                                                                     \
    hipLaunchKernelGGL(to_fp8_kernel<W>, dim3(blocks), dim3(256), 0, st, (uint8_t *)dst, (const char *)src, n, scale); \
  else                                                                                                            \
    hipLaunchKernelGGL(from_fp8_kernel<W>, dim3(blocks), dim3(256), 0, st, (char *)dst, (const uint8_t *)src, n, scale)
  if (wide_dtype == VTKV_F32) { LAUNCH_CVT(VTKV_F32); }
  else if (wide_dtype == VTKV_BF16) { LAUNCH_CVT(VTKV_BF16); }
  else { LAUNCH_CVT(VTKV_F16); }
#undef LAUNCH_CVT
  VTKV_HIP(hipGetLastError());
  return VTKV_OK;
}

}  // extern "C"
