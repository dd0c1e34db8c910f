// Shape-based choice between the decode GEMV and the MFMA GEMM for format A.
#include "wq_host.h"

extern "C" int wq_q4g32_linear(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                               const uint16_t* bias, const uint16_t* residual, uint16_t* y,
                               int64_t M, int64_t N, int64_t K, wq_stream_t stream) {
  if (M <= WQ_GEMV_MAX_M) return wq_q4g32_gemv(W, S, x, bias, residual, y, M, N, K, stream);
  return wq_q4g32_gemm(W, S, x, bias, residual, y, M, N, K, stream);
}
