// Decode GEMV over q4f16_1 weights stored K-major, used in place (no transposed copy):
//   W uint32 [K/8, N], S fp16 [K/32, N],  w[k,n] = (((W[k/8][n] >> 4*(k%8)) & 15) - 7) * S[k/32][n]
//   y[m,n] = epilogue( sum_k x[m,k] * w[k,n] )
// (tests/python/dlight/test_gpu_reduction.py:102-165, test_gpu_gemv.py:813-830: the layout the reference
// schedules with its reduction rule).
//
// In this layout consecutive addresses are consecutive COLUMNS, so a lane owns 4 adjacent columns
// (one 16-byte load per word row; a wavefront-wide load is 1 KiB of one row of W) and the reduction
// over K runs inside the lane: no cross-lane sum.  What every lane of a wavefront multiplies by is
// the same activation, which therefore comes from LDS as a broadcast read.  A workgroup takes 256
// columns and a slice of K (whole scale groups), its 4 wavefronts every 4th group of the slice; the
// grid is column blocks x K slices, with enough slices to give every CU a workgroup or two.  Partial
// sums of the slices go to a workspace (fp32 [slices, M, N]) and a second kernel adds them in slice
// order and applies bias / cast / residual; with one slice the first kernel finishes by itself.
//
// Arithmetic as in the row-major GEMV (q4_gemv.h): with t = 1024 + code (OR into 0x6400) a group
// contributes s * (sum_k x_k t_k - c_g), c_g = 1031 * sum_k x_k; odd nibble positions are taken
// unshifted as 1024 + 16 code against x / 16, their share of c_g being 71 x.  Products exact
// (v_dot2_f32_f16), accumulation fp32; a one-hot x reproduces the dequantized row bit for bit.
#include <algorithm>

#include "wq_device.h"
#include "wq_host.h"

namespace wq {

constexpr int kKnCols = 256;   // columns per workgroup (4 per lane)
constexpr int kKnWaves = 4;
constexpr int kKnMaxRows = 4;  // activation rows per pass

// xs: [rows][groups of the slice][4 words] x 16 bytes: the pairs (x_i, x_{i+4}) of a word's 8 activations, the odd
// pairs divided by 16; cg: [rows][groups] c_g
template <int MB>
__global__ __launch_bounds__(kKnWaves * 64) void q4g32_kn_gemv_kernel(
    const uint32_t* __restrict__ W, const half_t* __restrict__ S, const half_t* __restrict__ x,
    float* __restrict__ partial, const half_t* __restrict__ bias, const half_t* __restrict__ residual,
    half_t* __restrict__ y, int N, int K, int gps) {
  extern __shared__ uint4_t smem[];
  __shared__ float red[kKnWaves][MB][kKnCols];
  const int G = K >> 5;
  const int g0 = blockIdx.y * gps;
  const int ng = min(gps, G - g0);
  uint4_t* xs = smem;
  float* cg = reinterpret_cast<float*>(smem + MB * gps * 4);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = min((int)blockIdx.x * kKnCols + lane * 4, N - 4);  // N % 4 == 0; columns past N repeat the last four

  // weights first: the loads are in flight while x is staged
  auto load = [&](uint4_t (&wv)[4], uint2_t& sv, int gi) {
    const int g = g0 + min(gi, ng - 1);
#pragma unroll
    for (int w4 = 0; w4 < 4; ++w4)
      wv[w4] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(W + (int64_t)(4 * g + w4) * N + n));
    sv = __builtin_nontemporal_load(reinterpret_cast<const uint2_t*>(S + (int64_t)g * N + n));
  };
  uint4_t wa[4], wb[4];
  uint2_t sa, sb;
  load(wa, sa, wave);
  load(wb, sb, wave + kKnWaves);

  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  for (int idx = tid; idx < MB * ng; idx += kKnWaves * 64) {
    const int m = idx / ng, gi = idx % ng;
    const uint4_t* src = reinterpret_cast<const uint4_t*>(x + (int64_t)m * K + (int64_t)(g0 + gi) * 32);
    float even = 0.0f, odd = 0.0f;
#pragma unroll
    for (int w4 = 0; w4 < 4; ++w4) {
      const uint4_t v = src[w4];
      const uint32_t in[4] = {v.x, v.y, v.z, v.w};
      uint32_t p[4];
      pair_i_i4(in, p);
      const half2_t one = {(half_t)1.0f, (half_t)1.0f};
      even = dot2(as_half2(p[0]), one, dot2(as_half2(p[2]), one, even));
      odd = dot2(as_half2(p[1]), one, dot2(as_half2(p[3]), one, odd));
      xs[(m * gps + gi) * 4 + w4] =
          uint4_t{p[0], as_u32(as_half2(p[1]) * sixteenth), p[2], as_u32(as_half2(p[3]) * sixteenth)};
    }
    cg[m * gps + gi] = 1031.0f * even + 71.0f * odd;
  }
  __syncthreads();

  float acc[MB][4];
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[m][c] = 0.0f;
  const uint32_t magic = 0x64006400u;
  auto consume = [&](const uint4_t (&wv)[4], uint2_t sv, int gi) {
    const half2_t s01 = as_half2(sv.x), s23 = as_half2(sv.y);
    const float sc[4] = {(float)s01.x, (float)s01.y, (float)s23.x, (float)s23.y};
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      float d[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int w4 = 0; w4 < 4; ++w4) {
        const uint4_t xp = xs[(m * gps + gi) * 4 + w4];  // the same address in every lane: a broadcast
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t word = c == 0 ? wv[w4].x : c == 1 ? wv[w4].y : c == 2 ? wv[w4].z : wv[w4].w;
          const uint32_t w8 = word >> 8;
          d[c] = dot2(as_half2(and_or(word, 0x000F000Fu, magic)), as_half2(xp.x), d[c]);
          d[c] = dot2(as_half2(and_or(word, 0x00F000F0u, magic)), as_half2(xp.y), d[c]);
          d[c] = dot2(as_half2(and_or(w8, 0x000F000Fu, magic)), as_half2(xp.z), d[c]);
          d[c] = dot2(as_half2(and_or(w8, 0x00F000F0u, magic)), as_half2(xp.w), d[c]);
        }
      }
      const float c_g = cg[m * gps + gi];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[m][c] += sc[c] * (d[c] - c_g);
    }
  };
  // two groups in flight per wavefront: while one is multiplied the next but one is requested
  for (int gi = wave; gi < ng; gi += 2 * kKnWaves) {
    consume(wa, sa, gi);
    load(wa, sa, gi + 2 * kKnWaves);
    if (gi + kKnWaves < ng) consume(wb, sb, gi + kKnWaves);
    load(wb, sb, gi + 3 * kKnWaves);
  }

#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int c = 0; c < 4; ++c) red[wave][m][lane * 4 + c] = acc[m][c];
  __syncthreads();
  const int col = (int)blockIdx.x * kKnCols + tid;
  if (col >= N) return;
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    float v = red[0][m][tid];
#pragma unroll
    for (int w = 1; w < kKnWaves; ++w) v += red[w][m][tid];
    if (gridDim.y > 1) {
      partial[((int64_t)blockIdx.y * MB + m) * N + col] = v;
    } else {
      if (bias) v += (float)bias[col];
      half_t h = (half_t)v;
      if (residual) h = h + residual[(int64_t)m * N + col];
      y[(int64_t)m * N + col] = h;
    }
  }
}

__global__ __launch_bounds__(256) void q4g32_kn_finish_kernel(const float* __restrict__ partial,
                                                              const half_t* __restrict__ bias,
                                                              const half_t* __restrict__ residual,
                                                              half_t* __restrict__ y, int rows, int N, int slices) {
  const int col = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (col >= N) return;
  // eight loads in flight at a time, added in slice order
  float v = 0.0f;
  for (int s0 = 0; s0 < slices; s0 += 8) {
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) p[j] = s0 + j < slices ? partial[((int64_t)(s0 + j) * rows + m) * N + col] : 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) v += p[j];
  }
  if (bias) v += (float)bias[col];
  half_t h = (half_t)v;
  if (residual) h = h + residual[(int64_t)m * N + col];
  y[(int64_t)m * N + col] = h;
}

// scale groups per K slice: slices enough for two workgroups per CU, but at least 8 groups (two per
// wavefront) each and at most 128 (4 rows x 68 bytes of staged activations per group, beside 16 KiB of partial sums)
static int kn_groups_per_slice(int64_t N, int64_t K) {
  const int64_t G = K / 32, colblocks = (N + kKnCols - 1) / kKnCols;
  int64_t slices = std::max<int64_t>(1, (2 * cu_count() + colblocks - 1) / colblocks);
  int64_t gps = std::max<int64_t>(8, (G + slices - 1) / slices);
  gps = std::min<int64_t>(gps, 128);
  return (int)std::min(gps, G);
}

}  // namespace wq

extern "C" size_t wq_q4g32_kn_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  using namespace wq;
  if (M <= 0 || N <= 0 || K < 32) return 0;
  const int gps = kn_groups_per_slice(N, K);
  const int64_t slices = (K / 32 + gps - 1) / gps;
  return slices > 1 ? (size_t)(slices * std::min<int64_t>(M, kKnMaxRows) * N * 4) : 0;
}

extern "C" int wq_q4g32_kn_gemv(const uint32_t* W_kn, const uint16_t* S_kn, const uint16_t* x, const uint16_t* bias,
                                const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K,
                                void* workspace, size_t workspace_bytes, wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, "wq_q4g32_kn_gemv: negative dimension");
  WQ_REQUIRE(K % 32 == 0, "wq_q4g32_kn_gemv: K=%lld must be a multiple of the group size 32", (long long)K);
  WQ_REQUIRE(N % 4 == 0, "wq_q4g32_kn_gemv: N=%lld must be a multiple of 4", (long long)N);
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0, "wq_q4g32_kn_gemv: K must be positive");
  if (M > WQ_KN_GEMV_MAX_M)
    return fail(WQ_EUNSUPPORTED,
                "wq_q4g32_kn_gemv: %lld rows of activations; beyond %d convert the weights once with wq_q4g32_kn_to_nk",
                (long long)M, WQ_KN_GEMV_MAX_M);
  WQ_REQUIRE(W_kn && S_kn && x && y, "wq_q4g32_kn_gemv: null pointer");
  WQ_REQUIRE(aligned16(W_kn) && aligned16(x) && ((uintptr_t)S_kn & 7u) == 0,
             "wq_q4g32_kn_gemv: W_kn and x must be 16-byte aligned, S_kn 8-byte aligned");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 24), "wq_q4g32_kn_gemv: too large");
  const int gps = kn_groups_per_slice(N, K);
  const int slices = (int)((K / 32 + gps - 1) / gps);
  const size_t need = wq_q4g32_kn_gemv_workspace_bytes(M, N, K);
  WQ_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15u) == 0),
             "wq_q4g32_kn_gemv: needs a 16-byte aligned workspace of %zu bytes (wq_q4g32_kn_gemv_workspace_bytes)", need);
  WQ_REQUIRE(slices < 65536, "wq_q4g32_kn_gemv: too many K slices");
  const dim3 grid((unsigned)((N + kKnCols - 1) / kKnCols), (unsigned)slices);
  const half_t* xh = (const half_t*)x;
  const half_t* rh = (const half_t*)residual;
  half_t* yh = (half_t*)y;
  for (int64_t m0 = 0; m0 < M;) {
    const int mb = M - m0 >= 4 ? 4 : M - m0 >= 2 ? 2 : 1;
    const size_t lds = (size_t)mb * gps * (64 + 4);
    const half_t* xr = xh + m0 * K;
    const half_t* rr = rh ? rh + m0 * N : nullptr;
    half_t* yr = yh + m0 * N;
    if (mb == 4) {
      WQ_LAUNCH("wq_q4g32_kn_gemv", q4g32_kn_gemv_kernel<4>, grid, dim3(kKnWaves * 64), lds, stream, W_kn,
                (const half_t*)S_kn, xr, (float*)workspace, (const half_t*)bias, rr, yr, (int)N, (int)K, gps);
    } else if (mb == 2) {
      WQ_LAUNCH("wq_q4g32_kn_gemv", q4g32_kn_gemv_kernel<2>, grid, dim3(kKnWaves * 64), lds, stream, W_kn,
                (const half_t*)S_kn, xr, (float*)workspace, (const half_t*)bias, rr, yr, (int)N, (int)K, gps);
    } else {
      WQ_LAUNCH("wq_q4g32_kn_gemv", q4g32_kn_gemv_kernel<1>, grid, dim3(kKnWaves * 64), lds, stream, W_kn,
                (const half_t*)S_kn, xr, (float*)workspace, (const half_t*)bias, rr, yr, (int)N, (int)K, gps);
    }
    if (slices > 1) {
      WQ_LAUNCH("wq_q4g32_kn_gemv", q4g32_kn_finish_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)mb), dim3(256), 0,
                stream, (const float*)workspace, (const half_t*)bias, rr, yr, mb, (int)N, slices);
    }
    m0 += mb;
  }
  return WQ_OK;
}
