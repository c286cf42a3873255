// OCP fp8 e4m3fn (bias 7, no infinities, NaN = S.1111.111, largest finite 448) <-> fp32,
// written with integer arithmetic so the same source gives identical bits on the host (where it
// is checked exhaustively against a library cast) and on the device.
//
// Encoding follows the reference's NVIDIA KV-cache path, cvt_float_to_fp8(x, SATFINITE, E4M3)
// (csrc/quantization/fp8/nvidia/quant_utils.cuh:481-490): round to nearest even, finite overflow
// and infinities clamp to +-448, NaN stays NaN.
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define VTKV_HD __host__ __device__ __forceinline__
#else
#define VTKV_HD inline
#endif

namespace vtkv {

VTKV_HD uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
VTKV_HD float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

VTKV_HD uint8_t fp8_e4m3fn_encode(float x) {
  const uint32_t u = f32_bits(x);
  const uint32_t sign = (u >> 24) & 0x80u;
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);  // NaN
  if (a >= 0x43e80000u) return (uint8_t)(sign | 0x7eu); // |x| >= 464 rounds past 448: saturate
  if (a < 0x3c800000u) {
    // below 2^-6 the grid is m * 2^-9, m = 0..8.  Adding 2^14 places that quantum at the unit in
    // the last place of an fp32, so the hardware's round-to-nearest-even does the rounding.
    const float r = bits_f32(a) + 16384.0f;
    return (uint8_t)(sign | (f32_bits(r) & 0xfu));  // m = 8 is code 0x08 = 2^-6
  }
  const uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);  // RNE on the 20 dropped mantissa bits
  return (uint8_t)(sign | (((r >> 20) - (120u << 3)) & 0x7fu));
}

VTKV_HD float fp8_e4m3fn_decode(uint8_t c) {
  const uint32_t sign = ((uint32_t)c & 0x80u) << 24;
  const uint32_t em = c & 0x7fu;
  if (em == 0x7fu) return bits_f32(sign | 0x7fc00000u);
  if (em < 8u) return bits_f32(sign | f32_bits((float)em * 0.001953125f));  // m * 2^-9
  return bits_f32(sign | ((em + (120u << 3)) << 20));
}

VTKV_HD float bf16_bits_to_f32(uint16_t v) { return bits_f32(((uint32_t)v) << 16); }

VTKV_HD uint16_t f32_to_bf16_bits_rne(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

}  // namespace vtkv
