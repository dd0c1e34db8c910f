// Format A decode GEMV: y[m,n] = sum_k x[m,k] * ((code[n,k] - 7) * S[n,k/32]), M <= 8.
//
// The kernel is a weight stream.  One wavefront owns R consecutive output rows;
// lane l walks the row in 16-byte steps (4 words = 32 codes = exactly one scale
// group), so a wavefront-wide load is 1 KiB of contiguous weights per row and the
// matching scales are one contiguous 128-byte load.  The activations are staged
// once per workgroup in LDS, already rearranged to the (i, i+4) pairing the
// in-register unpack produces, 16-byte chunk c of group g at ((c*G + g) * 16) so
// that the 64 lanes of a wavefront read 64 consecutive chunks (no bank conflicts).
// Partial sums stay in fp32 registers and are combined with wavefront shuffles.
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;

template <int R, int MB>
__global__ __launch_bounds__(kGemvThreads) void q4g32_gemv_kernel(
    const uint4_t* __restrict__ W, const half_t* __restrict__ S, const half_t* __restrict__ x,
    const half_t* __restrict__ bias, const half_t* __restrict__ residual, half_t* __restrict__ y,
    int N, int K) {
  extern __shared__ uint4_t xs[];  // [MB][4][G] chunks of 16 bytes
  const int G = K >> 5;            // scale groups per row == 16-byte chunks of W per row
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // ---- stage x: word wi = 8 halves, stored in the (i, i+4) pairing ----
  const int nwords = K >> 3;
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    const uint4_t* xrow = reinterpret_cast<const uint4_t*>(x + (int64_t)m * K);
    for (int wi = tid; wi < nwords; wi += kGemvThreads) {
      uint4_t v = xrow[wi];
      uint32_t in[4] = {v.x, v.y, v.z, v.w}, o[4];
      pair_i_i4(in, o);
      uint4_t p = {o[0], o[1], o[2], o[3]};
      xs[(m * 4 + (wi & 3)) * G + (wi >> 2)] = p;
    }
  }
  __syncthreads();

  const int n0 = (blockIdx.x * kGemvWaves + wave) * R;
  if (n0 >= N) return;

  float acc[R][MB];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = 0.0f;

  // rows past the end are clamped for the loads and dropped at the store
  int64_t rowoff[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rowoff[r] = (int64_t)min(n0 + r, N - 1) * G;

  for (int g = lane; g < G; g += 64) {
    uint4_t wv[R];
    half_t sv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      wv[r] = __builtin_nontemporal_load(&W[rowoff[r] + g]);
      sv[r] = __builtin_nontemporal_load(&S[rowoff[r] + g]);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint4_t xv[MB];
#pragma unroll
      for (int m = 0; m < MB; ++m) xv[m] = xs[(m * 4 + c) * G + g];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t word = c == 0 ? wv[r].x : c == 1 ? wv[r].y : c == 2 ? wv[r].z : wv[r].w;
        const half2_t s2 = {sv[r], sv[r]};
        half2_t d[4];
        q4_word_dequant(word, s2, d);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
          acc[r][m] = dot2(d[0], as_half2(xv[m].x), acc[r][m]);
          acc[r][m] = dot2(d[1], as_half2(xv[m].y), acc[r][m]);
          acc[r][m] = dot2(d[2], as_half2(xv[m].z), acc[r][m]);
          acc[r][m] = dot2(d[3], as_half2(xv[m].w), acc[r][m]);
        }
      }
    }
  }

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = wave_sum(acc[r][m]);

  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = n0 + r;
      if (n >= N) break;
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        float v = acc[r][m];
        if (bias) v += (float)bias[n];
        half_t h = (half_t)v;
        if (residual) h = h + residual[(int64_t)m * N + n];
        y[(int64_t)m * N + n] = h;
      }
    }
  }
}

template <int R, int MB>
static int launch_gemv(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                       const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t N,
                       int64_t K, hipStream_t stream) {
  const size_t lds = (size_t)MB * K * 2;
  const int64_t blocks = (N + kGemvWaves * R - 1) / (kGemvWaves * R);
  auto kern = q4g32_gemv_kernel<R, MB>;
  if (lds > 64 * 1024) {
    WQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kGemvThreads), lds, stream,
                     (const uint4_t*)W, (const half_t*)S, (const half_t*)x, (const half_t*)bias,
                     (const half_t*)residual, (half_t*)y, (int)N, (int)K);
  WQ_CHECK_LAUNCH("wq_q4g32_gemv");
  return WQ_OK;
}

}  // namespace wq

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
  WQ_REQUIRE(N < (1ll << 31) && K <= 32768,
             "wq_q4g32_gemv: N=%lld K=%lld outside the supported range (K <= 32768)",
             (long long)N, (long long)K);
  // batches of up to 4 rows share one pass over the weights
  for (int64_t m0 = 0; m0 < M;) {
    const int64_t left = M - m0;
    const uint16_t* xp = x + m0 * K;
    const uint16_t* rp = residual ? residual + m0 * N : nullptr;
    uint16_t* yp = y + m0 * N;
    int rc;
    if (left >= 4 && K <= 16384) {
      rc = launch_gemv<2, 4>(W, S, xp, bias, rp, yp, N, K, stream);
      m0 += 4;
    } else if (left >= 2) {
      rc = launch_gemv<2, 2>(W, S, xp, bias, rp, yp, N, K, stream);
      m0 += 2;
    } else {
      rc = N >= 8192 ? launch_gemv<4, 1>(W, S, xp, bias, rp, yp, N, K, stream)
                     : launch_gemv<2, 1>(W, S, xp, bias, rp, yp, N, K, stream);
      m0 += 1;
    }
    if (rc != WQ_OK) return rc;
  }
  return WQ_OK;
}
