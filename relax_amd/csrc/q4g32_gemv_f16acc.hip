// Format A decode GEMV with the reference's fp16 accumulation
// (tests/python/dlight/test_gpu_reduction.py:44-51, test_gpu_gemv.py:199-206):
//   y[m,n] = sum_k x[m,k] * w[n,k]   with every product and every partial sum rounded to fp16.
// The order of the sum is not fixed by the reference (its schedules reorder it); here a lane
// adds the products of its scale groups pairwise in fp16 (v_pk_mul_f16, v_pk_add_f16: two
// roundings per term, never a fused multiply-add), then the wavefront adds the 64 lane sums as
// a tree, again in fp16.  The weights are the bit-exact dequantized values (q4_word_dequant).
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

// v + (v of the lane selected by the DPP control word), in fp16; lanes without a source add +0.0
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ half_t dpp_add_f16(half_t v) {
  const int bits = __builtin_amdgcn_update_dpp(0, (int)as_u16(v), CTRL, ROW_MASK, 0xf, true);
  return v + as_half((uint16_t)bits);
}

// fp16 sum over the wavefront, every addition rounded to fp16; the total is valid in lane 63.
__device__ __forceinline__ half_t wave_sum_f16_to_lane63(half_t v) {
  v = dpp_add_f16<0x111, 0xf>(v);  // row_shr:1
  v = dpp_add_f16<0x112, 0xf>(v);  // row_shr:2
  v = dpp_add_f16<0x114, 0xf>(v);  // row_shr:4
  v = dpp_add_f16<0x118, 0xf>(v);  // row_shr:8   -> lane 15 of each row holds the row sum
  v = dpp_add_f16<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add_f16<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// One wavefront per ROWS consecutive rows of W; lane l takes the scale groups l, l + 64, ...  MB rows of x
// (K apart; their outputs N apart) share one pass over the weights: every row of x keeps sums of its own, added
// in the order of a launch with that row alone, so batching changes no bit of the result.
template <int ROWS, int MB>
__global__ __launch_bounds__(256) void q4g32_gemv_f16acc_kernel(const uint4_t* __restrict__ W,
                                                                const half_t* __restrict__ S,
                                                                const half_t* __restrict__ x,
                                                                half_t* __restrict__ y, int N, int K) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int n0 = wave * ROWS;
  if (n0 >= N) return;
  const int G = K >> 5;
  half2_t acc[MB][ROWS];
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[m][r] = half2_t{(half_t)0.0f, (half_t)0.0f};
  // UNR scale groups per lane and row are requested before the first is multiplied (the order of the sums is
  // that of one group after the other)
  constexpr int UNR = 4;
  for (int g0 = lane; g0 < G; g0 += 64 * UNR) {
    uint4_t w4[UNR][ROWS];
    half_t sc[UNR][ROWS];
#pragma unroll
    for (int j = 0; j < UNR; ++j) {
      const int g = min(g0 + 64 * j, G - 1);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int n = min(n0 + r, N - 1);
        w4[j][r] = __builtin_nontemporal_load(&W[(int64_t)n * G + g]);
        sc[j][r] = S[(int64_t)n * G + g];
      }
    }
#pragma unroll
    for (int j = 0; j < UNR; ++j) {
      const int g = g0 + 64 * j;
      if (g >= G) break;
      // the group's 32 activations in the (i, i+4) pairing of the unpack
      uint32_t xp[MB][4][4];
#pragma unroll
      for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint4_t v = reinterpret_cast<const uint4_t*>(x + (int64_t)m * K)[g * 4 + c];
          const uint32_t in[4] = {v.x, v.y, v.z, v.w};
          pair_i_i4(in, xp[m][c]);
        }
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const half2_t s2 = {sc[j][r], sc[j][r]};
        const uint32_t words[4] = {w4[j][r].x, w4[j][r].y, w4[j][r].z, w4[j][r].w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          half2_t d[4];
          q4_word_dequant(words[c], s2, d);
#pragma unroll
          for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              // product rounded to fp16, then the sum rounded to fp16: two instructions on purpose
              half2_t p;
              asm("v_pk_mul_f16 %0, %1, %2" : "=v"(p) : "v"(d[i]), "v"(as_half2(xp[m][c][i])));
              asm("v_pk_add_f16 %0, %1, %2" : "=v"(acc[m][r]) : "v"(acc[m][r]), "v"(p));
            }
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const half_t t = wave_sum_f16_to_lane63(acc[m][r].x + acc[m][r].y);
      if (lane == 63 && n0 + r < N) y[(int64_t)m * N + n0 + r] = t;
    }
}

template <int MB>
static int launch_f16acc(const uint32_t* W, const uint16_t* S, const uint16_t* x, uint16_t* y, int64_t N, int64_t K,
                         hipStream_t stream) {
  constexpr int kRows = 2;
  const int64_t waves = (N + kRows - 1) / kRows;
  const unsigned blocks = (unsigned)((waves + 3) / 4);
  WQ_LAUNCH("wq_q4g32_gemv_f16acc", (q4g32_gemv_f16acc_kernel<kRows, MB>), dim3(blocks), dim3(256), 0, stream,
            (const uint4_t*)W, (const half_t*)S, (const half_t*)x, (half_t*)y, (int)N, (int)K);
  return WQ_OK;
}

}  // namespace wq

extern "C" int wq_q4g32_gemv_f16acc(const uint32_t* W, const uint16_t* S, const uint16_t* x, uint16_t* y,
                                    int64_t M, int64_t N, int64_t K, wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, "wq_q4g32_gemv_f16acc: negative dimension");
  WQ_REQUIRE(K % 32 == 0, "wq_q4g32_gemv_f16acc: K=%lld must be a multiple of the group size 32", (long long)K);
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0, "wq_q4g32_gemv_f16acc: K must be positive");
  WQ_REQUIRE(W && S && x && y, "wq_q4g32_gemv_f16acc: null pointer");
  WQ_REQUIRE(aligned16(W) && aligned16(x), "wq_q4g32_gemv_f16acc: W and x must be 16-byte aligned");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 30) && M <= 65536, "wq_q4g32_gemv_f16acc: too large");
  // up to 4 rows of x per pass over the weights (the low-batch case of
  // tests/python/dlight/test_gpu_low_batch_gemv.py:29-57); more rows: more passes
  for (int64_t m = 0; m < M;) {
    const int64_t mb = M - m >= 4 ? 4 : M - m >= 2 ? 2 : 1;
    const int rc = mb == 4   ? launch_f16acc<4>(W, S, x + m * K, y + m * N, N, K, stream)
                   : mb == 2 ? launch_f16acc<2>(W, S, x + m * K, y + m * N, N, K, stream)
                             : launch_f16acc<1>(W, S, x + m * K, y + m * N, N, K, stream);
    if (rc != WQ_OK) return rc;
    m += mb;
  }
  return WQ_OK;
}
