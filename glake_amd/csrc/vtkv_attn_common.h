// Device helpers shared by the attention kernels of this library: the MFMA operand types, the swizzled
// LDS tile layouts for K and V, row-group reductions with the gfx950 lane-swap instructions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vtkv_fp8.h"

namespace vtkv_attn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int kD = 128;            // head size
constexpr int kTile = 16;          // rows per MFMA tile
constexpr int kRowBytes = kD * 2;  // bf16 row of one head
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) {
  // round to nearest even, as the reference's from_float(bf16) does
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  bf16x2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(unsigned, v);
}

// LDS tile of 16 V rows x 256 bytes.  The 16-byte piece p of row r lives at piece slot
// p ^ (2*(r & 7)): a transposing read then touches all 64 banks evenly (rows of one read differ
// in r, pieces in one read are the pair {2*dblk, 2*dblk+1}).
__device__ __forceinline__ int v_lds_offset(int row, int piece16) {
  return row * kRowBytes + ((piece16 ^ ((row & 7) << 1)) << 4);
}

// LDS tile of 16 K rows as loaded (256 bytes of bf16, or 128 bytes of fp8 codes).  It is written a
// row quarter per 16 lanes and read back one piece per row by 16 lanes; the swizzles keep both
// conflict-free.
__device__ __forceinline__ int k_lds_offset(int row, int piece16) {
  return row * kRowBytes + ((piece16 ^ (row & 15)) << 4);
}
__device__ __forceinline__ int k8_lds_offset(int row, int piece16) {
  return row * kD + ((piece16 ^ ((row >> 1) & 7)) << 4);
}

// max / sum over the four row groups (lanes l, l^16, l^32, l^48) with the gfx950 lane-swap
// instructions: v_permlane16_swap exchanges odd 16-lane rows of its first operand with even rows of its
// second, v_permlane32_swap does the same for 32-lane halves, so swapping a value with itself and
// combining the two results folds rows pairwise.
// (the two results are copied to scalars before the bit cast: a bit cast applied directly to an
// element of the returned vector reads element 0 both times with this compiler)
__device__ __forceinline__ void swap_rows16(float x, float &a, float &b) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  a = __builtin_bit_cast(float, r0);
  b = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ void swap_rows32(float x, float &a, float &b) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  a = __builtin_bit_cast(float, r0);
  b = __builtin_bit_cast(float, r1);
}

__device__ __forceinline__ float max_over_row_groups(float x) {
  float a, b;
  swap_rows16(x, a, b);
  swap_rows32(fmaxf(a, b), a, b);
  return fmaxf(a, b);
}

__device__ __forceinline__ float sum_over_row_groups(float x) {
  float a, b;
  swap_rows16(x, a, b);
  swap_rows32(a + b, a, b);
  return a + b;
}

// eight e4m3fn codes (two dwords) -> eight bf16 values; exact, every e4m3fn value is a bf16 value
__device__ __forceinline__ u32x4 fp8x8_to_bf16x8(unsigned lo, unsigned hi) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  u32x4 r;
  r[0] = __builtin_bit_cast(unsigned, (bf16x2)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false));
  r[1] = __builtin_bit_cast(unsigned, (bf16x2)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true));
  r[2] = __builtin_bit_cast(unsigned, (bf16x2)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false));
  r[3] = __builtin_bit_cast(unsigned, (bf16x2)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true));
  return r;
}

// The same helpers for either 16-bit type of the model (F16 = false: bf16, true: fp16).
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <bool F16>
__device__ __forceinline__ f32x4 mfma_16x16x32(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// two floats -> two 16-bit values in one dword (a in the low half), round to nearest even
template <bool F16>
__device__ __forceinline__ unsigned pack_16x2(float a, float b) {
  if constexpr (F16) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f16x2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(unsigned, v);
  } else {
    return pack_bf16x2(a, b);
  }
}

// the low (which = 0) or high half of such a dword as a float
template <bool F16>
__device__ __forceinline__ float unpack_16(unsigned pair, int which) {
  if constexpr (F16) {
    const unsigned short h = (unsigned short)(which ? pair >> 16 : pair & 0xffffu);
    return (float)__builtin_bit_cast(_Float16, h);
  } else {
    return __builtin_bit_cast(float, which ? (pair & 0xffff0000u) : (pair << 16));
  }
}

template <bool F16>
__device__ __forceinline__ uint16_t f32_to_16(float r) {
  if constexpr (F16)
    return __builtin_bit_cast(unsigned short, (_Float16)r);  // v_cvt_f16_f32: round to nearest even
  else
    return vtkv::f32_to_bf16_bits_rne(r);
}

// eight e4m3fn codes -> eight fp16 values; exact (e4m3fn has 3 mantissa bits and exponents -9..8)
__device__ __forceinline__ u32x4 fp8x8_to_f16x8(unsigned lo, unsigned hi) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  u32x4 r;
  r[0] = __builtin_bit_cast(unsigned, (f16x2)__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false));
  r[1] = __builtin_bit_cast(unsigned, (f16x2)__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true));
  r[2] = __builtin_bit_cast(unsigned, (f16x2)__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false));
  r[3] = __builtin_bit_cast(unsigned, (f16x2)__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true));
  return r;
}

template <bool F16>
__device__ __forceinline__ u32x4 fp8x8_widen(unsigned lo, unsigned hi) {
  if constexpr (F16) return fp8x8_to_f16x8(lo, hi); else return fp8x8_to_bf16x8(lo, hi);
}

// Loads and stores that are coherent across the whole device (they go past the per-XCD L2), for the
// few values that workgroups hand to each other inside one launch.  A device-scope fence would also
// do, but it writes back and invalidates a whole L2 each time, which costs far more than these.
__device__ __forceinline__ void store_device_coherent(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_device_coherent(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// More than 16 query heads per kv head (multi-query models).  The MFMA layouts hold a group's heads in 16
// columns, so such a kv head is served as kv_split virtual kv heads that read the same K and V rows: the
// kernels' num_kv_heads counts the virtual heads and `group` is the heads of each, virtual head v stands for
// kv head v / kv_split and for the query heads [first_head_of(v), + heads_of(v)); the last virtual head of a
// kv head has fewer heads than `group` when group_real is no multiple of it.  kv_split == 1: nothing changes.
template <class Params>
__device__ __forceinline__ int first_head_of(const Params &p, int kvh) {
  if (p.kv_split == 1) return kvh * p.group;
  return (kvh / p.kv_split) * p.group_real + (kvh % p.kv_split) * p.group;
}
template <class Params>
__device__ __forceinline__ int real_kv_head(const Params &p, int kvh) {
  return p.kv_split == 1 ? kvh : kvh / p.kv_split;
}
template <class Params>
__device__ __forceinline__ int heads_of(const Params &p, int kvh) {
  if (p.kv_split == 1) return p.group;
  return min(p.group, p.group_real - (kvh % p.kv_split) * p.group);
}

}  // namespace vtkv_attn

// Host side of the same rule: how many virtual kv heads a kv head with `group_real` query heads becomes.
inline int vtkv_kv_split(int group_real) { return (group_real + 15) / 16; }
