// Format A (q4f16_1) small-batch entry: the shared small-batch kernel with the
// group-32 int4 weight policy.
#include "q4g32_common.h"
#include "skinny_gemm.h"

namespace wq {

// W uint32 [N, K/8], S fp16 [N, K/32]: the 32 codes at k0 are the 16 bytes at
// row + k0/2; their scale is S[n][k0/32], fetched as the aligned pair that holds it.
struct Q4G32SkinnyPolicy {
  static constexpr int kPieces = 1;
  static constexpr bool kScaleDma = true;
  static constexpr bool kCanScaleBlock = true;
  struct Args {
    const uint32_t* W;
    const half_t* S;
  };
  struct Lane {
    const char* w;
    const char* s;
  };
  __device__ __forceinline__ static void init(Lane& l, const Args& a, int n, int K, int) {
    l.w = reinterpret_cast<const char*>(a.W + (int64_t)n * (K >> 3));
    l.s = reinterpret_cast<const char*>(a.S + (int64_t)n * (K >> 5));
  }
  __device__ __forceinline__ static const char* w_addr(const Lane& l, int k0, int) { return l.w + (k0 >> 1); }
  __device__ __forceinline__ static const char* s_addr(const Lane& l, int k0) { return l.s + ((k0 >> 5) & ~1) * 2; }
  __device__ __forceinline__ static const char* s_pair_addr(const Lane& l, int k0) { return s_addr(l, k0); }
  __device__ __forceinline__ static const char* sblock_addr(const Lane& l, int g) { return l.s + g * 2; }
  // rows of K/16 bytes: every 8 scales are 16 aligned bytes when K % 256 == 0 and S is aligned
  static bool scale_block_ok(const Args& a, int64_t K) {
    return K % 256 == 0 && (reinterpret_cast<uintptr_t>(a.S) & 15u) == 0;
  }
  static bool pair_aligned(const Args& a) { return (reinterpret_cast<uintptr_t>(a.S) & 3u) == 0; }
  __device__ __forceinline__ static half_t pick_scale(const Lane&, half2_t pair, int kq) { return (kq & 1) ? pair.y : pair.x; }
  using Scale = half_t;
  __device__ __forceinline__ static half_t const_scale(const Lane&) { return (half_t)0.0f; }
  __device__ __forceinline__ static half_t null_scale() { return (half_t)0.0f; }
  __device__ __forceinline__ static void dequant(const uint4_t* pieces, half_t s, half8_t out[4]) {
    const half2_t s2 = {s, s};
    const uint32_t words[4] = {pieces[0].x, pieces[0].y, pieces[0].z, pieces[0].w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      half2_t d[4];
      q4_word_dequant_natural(words[t], s2, d);
      out[t] = half8_t{d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
    }
  }
};

}  // namespace wq

// Small-batch entry: 1 <= M <= 64, K % 64 == 0.  Called by wq_q4g32_linear.
extern "C" int wq_q4g32_small_batch(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                                    const uint16_t* bias, const uint16_t* residual, uint16_t* y,
                                    int64_t M, int64_t N, int64_t K, wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, "wq_q4g32_small_batch: negative dimension");
  WQ_REQUIRE(M <= WQ_SMALL_BATCH_MAX_M, "wq_q4g32_small_batch: M=%lld > %d", (long long)M,
             WQ_SMALL_BATCH_MAX_M);
  WQ_REQUIRE(K % 64 == 0, "wq_q4g32_small_batch: K=%lld must be a multiple of 64", (long long)K);
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0, "wq_q4g32_small_batch: K must be positive");
  WQ_REQUIRE(W && S && x && y, "wq_q4g32_small_batch: null pointer");
  WQ_REQUIRE(aligned16(W) && aligned16(x) && (reinterpret_cast<uintptr_t>(S) & 3u) == 0,
             "wq_q4g32_small_batch: W and x must be 16-byte aligned, S 4-byte aligned");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 30), "wq_q4g32_small_batch: too large");
  const Q4G32SkinnyPolicy::Args pargs{W, (const half_t*)S};
  const Q4G32Epilogue epi{(const half_t*)bias, (const half_t*)residual, (int)N};
  return launch_skinny_auto<Q4G32SkinnyPolicy, Q4G32Epilogue>("wq_q4g32_small_batch", pargs, x, y, epi,
                                                             M, N, K, stream);
}
