// Declarations shared by the format-A translation units.
#ifndef RELAX_AMD_CSRC_Q4G32_COMMON_H_
#define RELAX_AMD_CSRC_Q4G32_COMMON_H_

#include "wq_device.h"

namespace wq {

// (acc + bias[n]) -> fp16, then + residual[m,n] in fp16: the epilogue of
// tests/python/dlight/test_gpu_matmul.py:352-401.
struct Q4G32Epilogue {
  const half_t* bias;
  const half_t* residual;
  int N;
  __device__ half_t operator()(float acc, int m, int n) const {
    if (bias) acc += (float)bias[n];
    half_t h = (half_t)acc;
    if (residual) h = h + residual[(int64_t)m * N + n];
    return h;
  }
  // Row-wise form for 8 consecutive columns n .. n+7 (n % 8 == 0): same arithmetic, 16-byte accesses.
  __device__ bool wide_ok(int n_cols, const half_t* y) const {
    return n_cols % 8 == 0 &&
           ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(bias) |
             reinterpret_cast<uintptr_t>(residual)) & 15u) == 0;
  }
  __device__ half8_t apply8(const float (&v)[8], int m, int n) const {
    half8_t h;
    if (bias) {
      const half8_t b = *reinterpret_cast<const half8_t*>(bias + n);
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = (half_t)(v[i] + (float)b[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = (half_t)v[i];
    }
    if (residual) h = h + *reinterpret_cast<const half8_t*>(residual + (int64_t)m * N + n);
    return h;
  }
};

}  // namespace wq
#endif  // RELAX_AMD_CSRC_Q4G32_COMMON_H_
