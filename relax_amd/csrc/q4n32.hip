// q4f16_1 weights whose codes are packed along N (the decode block of
// tests/python/dlight/test_gpu_matmul.py:366-377):
//   W uint32 [K, N/8], S fp16 [K, N/32]
//   w[k, n] = (fp16((W[k, n/8] >> 4 (n % 8)) & 15) - 7) * S[k, n/32],   y = epilogue(x . w)
// A scale covers 32 consecutive n of ONE k, so this is not a transposed format A: no rearrangement
// turns its scales into scales per 32 consecutive k.  What a rearrangement does give is the weight
// stream of the MFMA GEMM (mfma_gemm_lds.h): at load time the codes are transposed to [N, K/8]
// (8 consecutive k of one column per word, as every kernel of this library reads them) and the scales
// to ST [N/32, K] (the scales of a group of 32 columns contiguous along k).  The GEMM then stages, per
// K-step of 64 k and group of 32 columns, the group's 64 scales (128 bytes: the 4 bytes per column that
// format A stages, laid out differently) and multiplies every pair of weights by its own pair of
// scales: (code - 7) is exact and the product rounds once, the reference's fp16 weight bit for bit.
#include "../../include/relax_amd_wq.h"
#include "mfma_gemm.h"
#include "mfma_gemm_lds.h"
#include "q4g32_common.h"
#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

// W_nk[n][kw] = the codes of column n at rows 8 kw .. 8 kw + 7; one thread per output word, kw fastest
__global__ __launch_bounds__(256) void q4n32_repack_kernel(const uint32_t* __restrict__ W_kn, uint32_t* __restrict__ W_nk,
                                                           int K, int N) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int K8 = K >> 3, N8 = N >> 3;
  if (idx >= (int64_t)N * K8) return;
  const int n = (int)(idx / K8), kw = (int)(idx % K8);
  const int shift = 4 * (n & 7);
  uint32_t out = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) out |= ((W_kn[(int64_t)(8 * kw + j) * N8 + (n >> 3)] >> shift) & 15u) << (4 * j);
  W_nk[idx] = out;
}

// ST[g][k] = S[k][g]
__global__ __launch_bounds__(256) void q4n32_scales_kernel(const half_t* __restrict__ S, half_t* __restrict__ ST, int K,
                                                           int G) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)G * K) return;
  const int g = (int)(idx / K), k = (int)(idx % K);
  ST[idx] = S[(int64_t)k * G + g];
}

// ---- decode: a few rows of x, the weights streamed once per row of x ---------------------------------------
// y[n] = sum_k x[k] s[k, g] (code[k, n] - 7) with g = n / 32: for the 32 rows of W_nk of one group the scales
// belong to the ACTIVATIONS, xs[k] = fp16(x[k] * ST[g][k]), and what is left is format A's decode GEMV with every
// scale 1.  A workgroup takes RPW rows of one group: it stages xs in LDS (in the pairing of the unpack, with the
// zero-point constant of every 32 k, as q4_gemv.h does) for MB rows of x, then its four wavefronts stream two rows
// of W each at a time, lane l the 16-byte pieces l, l + 64, ... of a row, every unpacked word against all MB rows.  One rounding differs from the reference: it rounds
// (code - 7) * s to fp16 and multiplies by x in fp32, here x * s is rounded and (code - 7) is exact; a one-hot x
// still returns the reference's weight bit for bit.
template <int MB>
__global__ __launch_bounds__(256) void q4n32_gemv_kernel(const uint4_t* __restrict__ W, const half_t* __restrict__ ST,
                                                         const half_t* __restrict__ x, const half_t* __restrict__ bias,
                                                         const half_t* __restrict__ residual, half_t* __restrict__ y,
                                                         int N, int K, int rpw) {
  extern __shared__ uint4_t smem[];
  const int G = K >> 5;                                             // pieces of 32 k per row
  uint4_t* xs = smem;                                               // [MB][4][G]: word ch of piece g of row m at (m * 4 + ch) * G + g
  float* cs = reinterpret_cast<float*>(smem + MB * 4 * (size_t)G);  // [MB][G]: -(1031 A + 71 B) of the piece
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * rpw;
  const half_t* st = ST + (int64_t)(n0 >> 5) * K;
  const half2_t k1031 = {(half_t)1031.0f, (half_t)1031.0f};
  const half2_t k71 = {(half_t)71.0f, (half_t)71.0f};
  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  for (int wi = tid; wi < (K >> 3); wi += 256) {  // K % 32 == 0: the 4 words of a piece sit in 4 adjacent lanes
    const uint4_t sv = reinterpret_cast<const uint4_t*>(st)[wi];
    const int g = wi >> 2, ch = wi & 3;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const uint4_t xv = reinterpret_cast<const uint4_t*>(x + (int64_t)m * K)[wi];
      const uint32_t in[4] = {as_u32(as_half2(xv.x) * as_half2(sv.x)), as_u32(as_half2(xv.y) * as_half2(sv.y)),
                              as_u32(as_half2(xv.z) * as_half2(sv.z)), as_u32(as_half2(xv.w) * as_half2(sv.w))};
      uint32_t o[4];
      pair_i_i4(in, o);  // o[i] = (xs_i, xs_{i+4})
      float c = dot2(as_half2(o[0]), k1031, 0.0f);
      c = dot2(as_half2(o[1]), k71, c);
      c = dot2(as_half2(o[2]), k1031, c);
      c = dot2(as_half2(o[3]), k71, c);
      c += dpp_shift<0xb1, 0xf>(c);
      c += dpp_shift<0x4e, 0xf>(c);
      xs[(m * 4 + ch) * G + g] = uint4_t{o[0], as_u32(as_half2(o[1]) * sixteenth), o[2], as_u32(as_half2(o[3]) * sixteenth)};
      if (ch == 0) cs[m * G + g] = -c;
    }
  }
  __syncthreads();
  const uint32_t magic = 0x64006400u;
  for (int r = wave * 2; r < rpw; r += 8) {  // two rows of W at a time share the reads of xs
    const int na = n0 + r, nb = na + 1;
    if (na >= N) break;
    const uint4_t* wa = W + (int64_t)na * G;
    const uint4_t* wb = W + (int64_t)min(nb, N - 1) * G;
    float acc_a[MB], acc_b[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc_a[m] = acc_b[m] = 0.0f;
    constexpr int UNR = 2;  // pieces per lane and row requested before the first is multiplied
    for (int g0 = lane; g0 < G; g0 += 64 * UNR) {
      uint4_t qa[UNR], qb[UNR];
#pragma unroll
      for (int j = 0; j < UNR; ++j) {
        const int g = min(g0 + 64 * j, G - 1);
        qa[j] = __builtin_nontemporal_load(&wa[g]);
        qb[j] = __builtin_nontemporal_load(&wb[g]);
      }
#pragma unroll
      for (int j = 0; j < UNR; ++j) {
        const int g = g0 + 64 * j;
        if (g >= G) break;
        float ga[MB], gb[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) ga[m] = gb[m] = cs[m * G + g];
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) {
          const uint32_t a = ch == 0 ? qa[j].x : ch == 1 ? qa[j].y : ch == 2 ? qa[j].z : qa[j].w;
          const uint32_t b = ch == 0 ? qb[j].x : ch == 1 ? qb[j].y : ch == 2 ? qb[j].z : qb[j].w;
          const uint32_t a8 = a >> 8, b8 = b >> 8;
          const half2_t a0 = as_half2(and_or(a, 0x000F000Fu, magic)), a1 = as_half2(and_or(a, 0x00F000F0u, magic));    // 1024 + (q0, q4), 1024 + 16 (q1, q5)
          const half2_t a2 = as_half2(and_or(a8, 0x000F000Fu, magic)), a3 = as_half2(and_or(a8, 0x00F000F0u, magic));
          const half2_t b0 = as_half2(and_or(b, 0x000F000Fu, magic)), b1 = as_half2(and_or(b, 0x00F000F0u, magic));
          const half2_t b2 = as_half2(and_or(b8, 0x000F000Fu, magic)), b3 = as_half2(and_or(b8, 0x00F000F0u, magic));
#pragma unroll
          for (int m = 0; m < MB; ++m) {
            const uint4_t xv = xs[(m * 4 + ch) * G + g];
            ga[m] = dot2(a0, as_half2(xv.x), ga[m]);
            ga[m] = dot2(a1, as_half2(xv.y), ga[m]);
            ga[m] = dot2(a2, as_half2(xv.z), ga[m]);
            ga[m] = dot2(a3, as_half2(xv.w), ga[m]);
            gb[m] = dot2(b0, as_half2(xv.x), gb[m]);
            gb[m] = dot2(b1, as_half2(xv.y), gb[m]);
            gb[m] = dot2(b2, as_half2(xv.z), gb[m]);
            gb[m] = dot2(b3, as_half2(xv.w), gb[m]);
          }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
          acc_a[m] += ga[m];
          acc_b[m] += gb[m];
        }
      }
    }
    const Q4G32Epilogue ep{bias, residual, N};
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const float ta = wave_sum_to_lane63(acc_a[m]), tb = wave_sum_to_lane63(acc_b[m]);
      if (lane == 63) {
        y[(int64_t)m * N + na] = ep(ta, m, na);
        if (nb < N && r + 1 < rpw) y[(int64_t)m * N + nb] = ep(tb, m, nb);
      }
    }
  }
}

template <int MB>
static int launch_q4n32_gemv(const uint32_t* W_nk, const uint16_t* ST, const uint16_t* x, const uint16_t* bias,
                             const uint16_t* residual, uint16_t* y, int64_t N, int64_t K, hipStream_t stream) {
  const size_t lds = MB * ((size_t)K * 2 + (size_t)(K / 32) * 4);
  const int cus = cu_count();
  const int rpw = N / 32 >= 4 * cus ? 32 : N / 16 >= 4 * cus ? 16 : 8;
  static DynamicLdsLimit limit;
  WQ_HIP(limit.ensure(reinterpret_cast<const void*>(q4n32_gemv_kernel<MB>), (int)lds));
  WQ_LAUNCH("wq_q4n32_linear", q4n32_gemv_kernel<MB>, dim3((unsigned)((N + rpw - 1) / rpw)), dim3(256), lds, stream,
            (const uint4_t*)W_nk, (const half_t*)ST, (const half_t*)x, (const half_t*)bias, (const half_t*)residual,
            (half_t*)y, (int)N, (int)K, rpw);
  return WQ_OK;
}

// Weight policy of gemm_lds_kernel: the code stream of format A, scales per (k, group of 32 columns).
struct Q4N32LdsPolicy {
  static constexpr int kColBytes = 32;
  static constexpr int kScaleBytes = 4;
  static constexpr int kStepStride = 32;
  struct Args {
    const uint32_t* W;  // [N, K/8]
    const half_t* ST;   // [N/32, K]
  };
  struct Frag {
    uint4_t w;
  };
  // where the 32 scales of the lane's half of the step lie in LDS, and the 8 of the MFMA being unpacked
  struct Scale {
    const unsigned char* p;
    uint4_t cur;
  };
  __device__ __forceinline__ static const char* b_src(const Args& a, int n0, int q, int N, int K) {
    const int n = q >> 1, h = q & 1;
    return reinterpret_cast<const char*>(a.W + (int64_t)min(n0 + n, N - 1) * (K >> 3)) + h * 16;
  }
  // "the 4 scale bytes of column n" of a step: bytes 4 (n % 32) .. + 3 of the 128 bytes of its group, so that
  // the 32 columns of a group stage the group's 64 scales in order
  __device__ __forceinline__ static const char* s_src(const Args& a, int n, int K) {
    return reinterpret_cast<const char*>(a.ST + (int64_t)(n >> 5) * K) + (n & 31) * 4;
  }
  __device__ __forceinline__ static int64_t s_offset(const Args&, int ks) { return (int64_t)ks * 128; }
  // p: the staged bytes of the lane's column; a sub-tile of 32 columns is one group (tiles start at multiples of 128)
  __device__ __forceinline__ static Scale read_scale(const unsigned char* p, int lh) {
    return Scale{p - ((threadIdx.x & 31) << 2) + lh * 64, uint4_t{0, 0, 0, 0}};
  }
  __device__ __forceinline__ static Scale const_scale(const Args&, int) { return Scale{nullptr, uint4_t{0, 0, 0, 0}}; }
  __device__ __forceinline__ static void read(Frag& f, const unsigned char* bslot, int n_local, int lh) {
    f.w = *reinterpret_cast<const uint4_t*>(bslot + (n_local * 2 + lh) * 16);
  }
  __device__ __forceinline__ static uint32_t pair_bits(const Frag& f, int kk, int j) {
    const uint32_t word = kk == 0 ? f.w.x : kk == 1 ? f.w.y : kk == 2 ? f.w.z : f.w.w;
    return q4_pair_bits_natural(word, j);
  }
  __device__ __forceinline__ static void phase_begin(Scale& s, int kk) {
    s.cur = *reinterpret_cast<const uint4_t*>(s.p + kk * 16);
  }
  __device__ __forceinline__ static half2_t pair_finish_at(uint32_t bits, const Scale& s, int j) {
    const half2_t off = {(half_t)1031.0f, (half_t)1031.0f};
    const uint32_t s2 = j == 0 ? s.cur.x : j == 1 ? s.cur.y : j == 2 ? s.cur.z : s.cur.w;
    return (as_half2(bits) - off) * as_half2(s2);
  }
  __device__ __forceinline__ static half2_t pair_finish(uint32_t, const Scale&) { return half2_t{}; }  // (not used)
  __device__ __forceinline__ static half2_t pair(const Frag& f, int kk, int j, const Scale& s) {
    const half2_t off = {(half_t)1031.0f, (half_t)1031.0f};
    return (as_half2(pair_bits(f, kk, j)) - off) * *reinterpret_cast<const half2_t*>(s.p + kk * 16 + j * 4);
  }
};

}  // namespace wq

extern "C" int wq_q4n32_prepare(const uint32_t* W, const uint16_t* S, uint32_t* W_nk, uint16_t* ST, int64_t K, int64_t N,
                                wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(K >= 0 && N >= 0, "wq_q4n32_prepare: negative dimension");
  WQ_REQUIRE(K % 8 == 0 && N % 32 == 0, "wq_q4n32_prepare: K=%lld must be a multiple of 8 and N=%lld of the group size 32",
             (long long)K, (long long)N);
  if (K == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(W && S && W_nk && ST, "wq_q4n32_prepare: null pointer");
  WQ_REQUIRE(K < (1ll << 30) && N < (1ll << 30), "wq_q4n32_prepare: too large");
  const int64_t words = N * (K / 8), scales = (N / 32) * K;
  WQ_LAUNCH("wq_q4n32_prepare", q4n32_repack_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, W, W_nk,
            (int)K, (int)N);
  WQ_LAUNCH("wq_q4n32_prepare", q4n32_scales_kernel, dim3((unsigned)((scales + 255) / 256)), dim3(256), 0, stream,
            (const half_t*)S, (half_t*)ST, (int)K, (int)(N / 32));
  return WQ_OK;
}

extern "C" int wq_q4n32_linear(const uint32_t* W_nk, const uint16_t* ST, const uint16_t* x, const uint16_t* bias,
                               const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K,
                               wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, "wq_q4n32_linear: negative dimension");
  WQ_REQUIRE(K % 64 == 0 && N % 32 == 0,
             "wq_q4n32_linear: K=%lld must be a multiple of 64 (a step of the matrix-core kernel) and N=%lld of the group size 32",
             (long long)K, (long long)N);
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0, "wq_q4n32_linear: K must be positive");
  WQ_REQUIRE(W_nk && ST && x && y, "wq_q4n32_linear: null pointer");
  WQ_REQUIRE(aligned16(W_nk) && aligned16(x) && (reinterpret_cast<uintptr_t>(ST) & 3u) == 0,
             "wq_q4n32_linear: W_nk and x must be 16-byte aligned, ST 4-byte aligned");
  WQ_REQUIRE(M < (1ll << 30) && N < (1ll << 30) && K < (1ll << 30), "wq_q4n32_linear: too large");
  // A few rows of x: the streaming kernel, as many rows per pass over the weights as their staged activations fit
  // the LDS.  The GEMM below costs the same from 1 to 128 rows (one round of few tiles, about 0.52 us per K-step of
  // the 128-row tiles it would use), a pass of the streaming kernel about 2 us + 0.5 us per MB of weights (measured
  // at 4096 x 4096, 11008 x 4096 and 4096 x 11008): up to 8 rows always stream, beyond that whichever is cheaper.
  if (M <= WQ_Q4N32_GEMV_MAX_M && !tuning().gemm_cfg) {
    const size_t per_row = (size_t)K * 2 + (size_t)(K / 32) * 4;
    // (64 KiB of LDS leave room for two workgroups per CU; a single row may take up to 96 KiB)
    const int64_t fit = std::min<int64_t>(4, std::max<int64_t>((int64_t)((64 * 1024) / per_row), per_row <= 96 * 1024 ? 1 : 0));
    bool stream_it = fit >= 1;
    if (stream_it && M > 8) {
      const double passes = (double)((M + fit - 1) / fit);
      const double t_stream = passes * (2.0 + 0.5 * ((double)N * (double)K / 2.0) / 1e6);
      const int64_t tiles = ((N + 127) / 128) * ((M + 127) / 128);
      const double rounds = (double)((tiles + 2 * cu_count() - 1) / (2 * cu_count()));  // two 128 x 128 tiles per CU
      const double t_gemm = 0.52 * (double)(K / 64) * rounds;
      stream_it = t_stream < t_gemm;
    }
    if (stream_it) {
      for (int64_t m = 0; m < M;) {
        const int64_t mb = std::min(fit, M - m);
        const uint16_t* r = residual ? residual + m * N : nullptr;
        const int rc = mb >= 4   ? launch_q4n32_gemv<4>(W_nk, ST, x + m * K, bias, r, y + m * N, N, K, stream)
                       : mb == 3 ? launch_q4n32_gemv<3>(W_nk, ST, x + m * K, bias, r, y + m * N, N, K, stream)
                       : mb == 2 ? launch_q4n32_gemv<2>(W_nk, ST, x + m * K, bias, r, y + m * N, N, K, stream)
                                 : launch_q4n32_gemv<1>(W_nk, ST, x + m * K, bias, r, y + m * N, N, K, stream);
        if (rc != WQ_OK) return rc;
        m += mb;
      }
      return WQ_OK;
    }
  }
  const Q4N32LdsPolicy::Args args{W_nk, (const half_t*)ST};
  const Q4G32Epilogue ep{(const half_t*)bias, (const half_t*)residual, (int)N};
  // the tile shapes of format A's GEMM (same code stream, same bytes per step)
  switch (tuning().gemm_cfg ? tuning().gemm_cfg : choose_q4_lds_cfg(M, N, cu_count())) {
    case 11: return launch_gemm_lds<Q4N32LdsPolicy, Q4G32Epilogue, 8, 2, 1, 4, 1>("wq_q4n32_linear", args, x, y, ep, M, N, K, stream);
    case 18: return launch_gemm_lds<Q4N32LdsPolicy, Q4G32Epilogue, 8, 1, 1, 4, 1>("wq_q4n32_linear", args, x, y, ep, M, N, K, stream);
    default: return launch_gemm_lds<Q4N32LdsPolicy, Q4G32Epilogue, 4, 1, 1, 4, 2>("wq_q4n32_linear", args, x, y, ep, M, N, K, stream);
  }
}
