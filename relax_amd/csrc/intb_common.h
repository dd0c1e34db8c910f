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

}  // namespace wq
#endif  // RELAX_AMD_CSRC_INTB_COMMON_H_
