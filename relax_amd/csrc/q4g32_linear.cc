// Shape-based choice between the decode GEMV, the small-batch kernel and the MFMA GEMM for format A.
#include <cstdint>

#include "wq_host.h"

extern "C" int wq_q4g32_linear(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                               const uint16_t* bias, const uint16_t* residual, uint16_t* y,
                               int64_t M, int64_t N, int64_t K, wq_stream_t stream) {
  // one or two rows: the VALU streaming kernel; up to 64 rows: still one pass over the
  // weights, products on the matrix cores; beyond that the tiled GEMM.  A kernel whose
  // preconditions the operands do not meet (K range, scale alignment) is passed over
  // for the next one that serves the call.
  const bool gemv_ok = K <= 32768;
  const bool small_ok = K % 64 == 0 && (reinterpret_cast<uintptr_t>(S) & 3u) == 0;
  // (two rows of more than 8192 columns: the streaming kernel's two-row form is the slower one there; N = 4096,
  // K = 11008: 15.5 against 10.9 us, N = 8192, K = 28672: 56 against 37 us)
  const bool two_long_rows = M == 2 && K > 8192 && small_ok;
  if (M <= 2 && gemv_ok && !two_long_rows) return wq_q4g32_gemv(W, S, x, bias, residual, y, M, N, K, stream);
  if (M <= WQ_SMALL_BATCH_MAX_M && small_ok)
    return wq_q4g32_small_batch(W, S, x, bias, residual, y, M, N, K, stream);
  // up to 128 rows of a small matrix: the tiled GEMM would have too few tiles for 256
  // CUs; two passes of the small-batch kernel are faster
  if (M > WQ_SMALL_BATCH_MAX_M && M <= 2 * WQ_SMALL_BATCH_MAX_M && small_ok && N <= 8192) {
    const int64_t m0 = WQ_SMALL_BATCH_MAX_M;
    int rc = wq_q4g32_small_batch(W, S, x, bias, residual, y, m0, N, K, stream);
    if (rc) return rc;
    return wq_q4g32_small_batch(W, S, x + m0 * K, bias, residual ? residual + m0 * N : nullptr,
                                y + m0 * N, M - m0, N, K, stream);
  }
  if (M <= WQ_GEMV_MAX_M && gemv_ok) return wq_q4g32_gemv(W, S, x, bias, residual, y, M, N, K, stream);
  return wq_q4g32_gemm(W, S, x, bias, residual, y, M, N, K, stream);
}
