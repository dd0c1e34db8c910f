// Declarations shared by the format-B GEMV and GEMM translation units.
#ifndef RELAX_AMD_CSRC_INTB_COMMON_H_
#define RELAX_AMD_CSRC_INTB_COMMON_H_

#include "wq_device.h"
#include "wq_host.h"

namespace wq {

// Fused epilogue of the mixed-input GEMM: act(acc + bias) [binary residual] [unary].
// bias_stride == 0 broadcasts bias[n] over rows.  activation / binary_op / unary_op
// are the WQ_ACT_* / WQ_BIN_* / WQ_UN_* selectors.
struct IntbEpilogue {
  const half_t* bias;
  const half_t* residual;
  int64_t bias_stride;
  int activation, binary_op, unary_op;
};

// Streaming kernel for m <= 4 (intb_gemv.hip).  `group` is 0 (per column) or 64.
int intb_gemv_dispatch(const uint16_t* A, const int8_t* B, const uint16_t* scales, uint16_t* C,
                       int64_t m, int64_t n, int64_t k, int64_t group, int nbit,
                       const IntbEpilogue& ep, hipStream_t stream);

// Wavefronts that kernel's launch for one or two rows would have: it gives a wavefront whole columns, so a
// narrow matrix leaves the machine short of them.
int64_t intb_gemv_wavefronts(int64_t m, int64_t n, int64_t group, int nbit);

// Matrix-core streaming kernel for 1 <= m <= 64 (intb_skinny.hip).
int intb_small_batch_dispatch(const uint16_t* A, const int8_t* B, const uint16_t* scales, uint16_t* C,
                              int64_t m, int64_t n, int64_t k, int64_t group, int nbit,
                              const IntbEpilogue& ep, hipStream_t stream);

#ifdef __HIPCC__
// act(acc + bias) [binary residual] [unary], all in fp32, one rounding at the store
struct IntbGemmEpilogue {
  IntbEpilogue e;
  int N;
  __device__ half_t operator()(float v, int m, int n) const {
    if (e.bias) v += (float)e.bias[e.bias_stride ? (int64_t)m * e.bias_stride + n : n];
    v = apply_activation(v, e.activation);
    if (e.residual) {
      const float r = (float)e.residual[(int64_t)m * N + n];
      if (e.binary_op == 1) v += r;
      if (e.binary_op == 2) v *= r;
    }
    if (e.unary_op == 1) v = v > 0.0f ? v : 0.0f;
    return (half_t)v;
  }
  // Row-wise form for 8 consecutive columns n .. n+7 (n % 8 == 0): same arithmetic, 16-byte accesses.
  // (identity and relu only: eight inlined erf / exp evaluations next to 256 live accumulators
  // make the compiler spill; silu and gelu keep the element-wise form)
  __device__ bool wide_ok(int n_cols, const half_t* y) const {
    return e.activation <= 1 && n_cols % 8 == 0 && e.bias_stride % 8 == 0 &&
           ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(e.bias) |
             reinterpret_cast<uintptr_t>(e.residual)) & 15u) == 0;
  }
  __device__ half8_t apply8(const float (&v)[8], int m, int n) const {
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = v[i];
    if (e.bias) {
      const half8_t b = *reinterpret_cast<const half8_t*>(e.bias + (e.bias_stride ? (int64_t)m * e.bias_stride + n : n));
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] += (float)b[i];
    }
    if (e.activation == 1) {
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = f[i] > 0.0f ? f[i] : 0.0f;
    }
    if (e.residual) {
      const half8_t r = *reinterpret_cast<const half8_t*>(e.residual + (int64_t)m * N + n);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (e.binary_op == 1) f[i] += (float)r[i];
        if (e.binary_op == 2) f[i] *= (float)r[i];
      }
    }
    half8_t h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (half_t)((e.unary_op == 1 && !(f[i] > 0.0f)) ? 0.0f : f[i]);
    return h;
  }
};
#endif

}  // namespace wq
#endif  // RELAX_AMD_CSRC_INTB_COMMON_H_
