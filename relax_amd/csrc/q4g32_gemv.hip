// Format A (q4f16_1) decode GEMV entry point: the streaming kernel of q4_gemv.h without zero points.
#include "q4_gemv.h"

extern "C" int wq_q4g32_gemv(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                             const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M,
                             int64_t N, int64_t K, wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, "wq_q4g32_gemv: negative dimension");
  WQ_REQUIRE(K % 32 == 0, "wq_q4g32_gemv: K=%lld must be a multiple of the group size 32",
             (long long)K);
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0, "wq_q4g32_gemv: K must be positive");
  WQ_REQUIRE(W && S && x && y, "wq_q4g32_gemv: null pointer");
  WQ_REQUIRE(aligned16(W) && aligned16(x), "wq_q4g32_gemv: W and x must be 16-byte aligned");
  WQ_REQUIRE(N < (1ll << 30) && K <= 32768,
             "wq_q4g32_gemv: N=%lld K=%lld outside the supported range (K <= 32768)",
             (long long)N, (long long)K);
  return gemv_dispatch<false>("wq_q4g32_gemv", W, S, GemvZp{1, 0}, x, bias, residual, y, M, N, K, stream);
}
