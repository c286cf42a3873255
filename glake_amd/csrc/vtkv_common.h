// Shared helpers of the vtkv library: error reporting and HIP call checking.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/vtkv.h"

namespace vtkv {

// Per-thread message of the last failing call (returned by vtkv_last_error()).
char *error_buffer();
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

inline int elem_bytes(int dtype) {
  switch (dtype) {
    case VTKV_F32: return 4;
    case VTKV_BF16: return 2;
    case VTKV_F16: return 2;
    case VTKV_FP8_E4M3: return 1;
    default: return 0;
  }
}

// Float32 attention (csrc/vtkv_attention_f32.hip): decode rows (seq_lens) or prompt tokens (units of up to
// unit_tokens tokens); the split-K interface's buffers, a workspace for partial results, or neither.
int attention_f32(float *out, const float *q, const int64_t *k_ptrs, const int64_t *v_ptrs, const int64_t *slot_ids,
                  const int32_t *seq_lens, const int32_t *units, int unit_tokens, int num_rows, int num_heads,
                  int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                  const float *alibi_slopes, float *exp_sums, float *max_logits, float *tmp_out, int max_parts,
                  void *workspace, int64_t workspace_bytes, void *stream);

}  // namespace vtkv

#define VTKV_HIP(call)                                                                              \
  do {                                                                                              \
    hipError_t e__ = (call);                                                                        \
    if (e__ != hipSuccess)                                                                          \
      return vtkv::fail(VTKV_EHIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__, \
                        __LINE__);                                                                  \
  } while (0)

#define VTKV_REQUIRE(cond, ...)                           \
  do {                                                    \
    if (!(cond)) return vtkv::fail(VTKV_EINVAL, __VA_ARGS__); \
  } while (0)
