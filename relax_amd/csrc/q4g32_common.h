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
};

}  // namespace wq
#endif  // RELAX_AMD_CSRC_Q4G32_COMMON_H_
