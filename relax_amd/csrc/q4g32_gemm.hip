// Format A prefill GEMM on the gfx950 matrix cores:
//   y[m,n] = sum_k x[m,k] * ((code[n,k] - 7) * S[n,k/32])      fp16 MFMA, fp32 accumulate
//
// Work split.  A workgroup of 4 wavefronts owns a BM x BN tile of y.  The
// activation tile (BM x 64 halves per K-step) is shared through LDS; the weight
// tile never touches LDS: v_mfma_f32_32x32x16_f16 wants, in lane (j, h), the 8
// K-values of column j for K-half h — and 8 codes are exactly one uint32 of the
// packed weight.  So lane (j, h) loads the 16 bytes W[n0+j, 4h..4h+3 words of the
// step] together with their single scale, dequantizes in registers with the same
// function the decode kernel uses, and feeds the four words to four MFMAs.
//
// K labelling.  An MFMA only needs A and B to agree on which K sits in which
// (half, element) slot.  The in-register unpack yields the pairing (i, i+4) inside
// each group of 8, so the activations are rearranged to that pairing once, when
// they are written to LDS.  MFMA number kk of a K-step consumes 16-byte chunk
// (4h + kk) of every row, for both operands.
//
// LDS layout of the activation tile: row r, chunk c (16 bytes) at
// r*128 + ((c ^ (r & 7)) * 16): the XOR spreads the 32 rows a wavefront reads
// at one chunk index over all banks.
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

constexpr int kBK = 64;        // K elements per step
constexpr int kChunks = 8;     // 16-byte chunks per row per step

template <int TM, int TN, int WM, int WN>
struct GemmCfg {
  static constexpr int kThreads = 64 * WM * WN;
  static constexpr int BM = 32 * TM * WM;
  static constexpr int BN = 32 * TN * WN;
  static constexpr int kAChunks = BM * kChunks;                  // 16-byte chunks of A per step
  static constexpr int kAPerThread = kAChunks / kThreads;        // chunks each thread stages
  static constexpr int kLdsBytes = 2 * BM * kBK * 2;             // double buffered
  static_assert(kAChunks % kThreads == 0, "tile must divide evenly among threads");
};

__device__ __forceinline__ int lds_a_offset(int row, int chunk) {
  return row * (kBK * 2) + ((chunk ^ (row & 7)) << 4);
}

template <int TM, int TN, int WM, int WN, int WAVES_PER_EU>
__global__ __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(WAVES_PER_EU, WAVES_PER_EU)))
void q4g32_gemm_kernel(const uint32_t* __restrict__ W, const half_t* __restrict__ S,
                       const half_t* __restrict__ X, const half_t* __restrict__ bias,
                       const half_t* __restrict__ residual, half_t* __restrict__ Y, int M, int N,
                       int K, int tiles_m, int tiles_n) {
  using Cfg = GemmCfg<TM, TN, WM, WN>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int lj = lane & 31, lh = lane >> 5;

  // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2): give
  // every XCD a contiguous range of tiles, walked M-fastest so that neighbours on
  // one XCD share their weight rows.
  const int nblk = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblk / 8, rem = nblk % 8;
    const int xcd = pid & 7, idx = pid >> 3;
    pid = xcd * per + min(xcd, rem) + idx;
  }
  const int tile_m = pid % tiles_m, tile_n = pid / tiles_m;
  const int m0 = tile_m * Cfg::BM, n0 = tile_n * Cfg::BN;

  const int KW = K >> 3;  // words per weight row
  const int G = K >> 5;   // groups per weight row
  const int ksteps = (K + kBK - 1) / kBK;

  // ---- per-thread constants for staging A ----
  int a_row[Cfg::kAPerThread], a_chunk[Cfg::kAPerThread];
  const uint4_t* a_src[Cfg::kAPerThread];
#pragma unroll
  for (int i = 0; i < Cfg::kAPerThread; ++i) {
    const int id = tid + i * Cfg::kThreads;
    a_row[i] = id >> 3;
    a_chunk[i] = id & 7;
    const int gm = min(m0 + a_row[i], M - 1);  // clamped: rows past M are never stored
    a_src[i] = reinterpret_cast<const uint4_t*>(X + (int64_t)gm * K) + a_chunk[i];
  }

  // ---- per-thread constants for loading B ----
  const uint4_t* b_src[TN];
  const half_t* s_src[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int gn = min(n0 + (wn * TN + t) * 32 + lj, N - 1);
    b_src[t] = reinterpret_cast<const uint4_t*>(W + (int64_t)gn * KW) + lh;
    s_src[t] = S + (int64_t)gn * G + lh;
  }

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.0f;

  uint4_t a_reg[Cfg::kAPerThread];
  uint4_t b_reg[TN];
  half_t s_reg[TN];

  auto load_global = [&](int ks) {
    const bool b_ok = (ks * 2 + lh) < G;  // the last step may hold a single group
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      if (b_ok) {
        b_reg[t] = b_src[t][ks * 2];
        s_reg[t] = s_src[t][ks * 2];
      } else {
        b_reg[t] = uint4_t{0x77777777u, 0x77777777u, 0x77777777u, 0x77777777u};  // code 7 -> 0
        s_reg[t] = (half_t)0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < Cfg::kAPerThread; ++i) {
      if (ks * kChunks + a_chunk[i] < KW)
        a_reg[i] = a_src[i][ks * kChunks];
      else
        a_reg[i] = uint4_t{0u, 0u, 0u, 0u};
    }
  };

  auto store_a = [&](int buf) {
    unsigned char* base = lds + buf * (Cfg::BM * kBK * 2);
#pragma unroll
    for (int i = 0; i < Cfg::kAPerThread; ++i) {
      uint32_t in[4] = {a_reg[i].x, a_reg[i].y, a_reg[i].z, a_reg[i].w}, o[4];
      pair_i_i4(in, o);
      *reinterpret_cast<uint4_t*>(base + lds_a_offset(a_row[i], a_chunk[i])) =
          uint4_t{o[0], o[1], o[2], o[3]};
    }
  };

  load_global(0);
  store_a(0);
  // keep b_reg/s_reg of step 0; they are consumed in the first iteration
  __syncthreads();

  for (int ks = 0; ks < ksteps; ++ks) {
    const int buf = ks & 1;
    // B operands of this step, dequantized: bop[t][kk] = 8 halves
    half8_t bop[TN][4];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      const half2_t s2 = {s_reg[t], s_reg[t]};
      const uint32_t ws[4] = {b_reg[t].x, b_reg[t].y, b_reg[t].z, b_reg[t].w};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        half2_t d[4];
        q4_word_dequant(ws[kk], s2, d);
        bop[t][kk] = half8_t{d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
      }
    }
    // prefetch the next step while the matrix cores work on this one
    if (ks + 1 < ksteps) load_global(ks + 1);

    const unsigned char* abase = lds + buf * (Cfg::BM * kBK * 2);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = (wm * TM + i) * 32 + lj;
        const half8_t aop =
            *reinterpret_cast<const half8_t*>(abase + lds_a_offset(row, 4 * lh + kk));
#pragma unroll
        for (int t = 0; t < TN; ++t)
          acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop, bop[t][kk], acc[i][t], 0, 0, 0);
      }
    }

    if (ks + 1 < ksteps) store_a(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: (+bias in fp32) -> fp16 -> (+residual in fp16) ----
  // accumulator register r of lane (j, h) is element (row 8*(r/4) + 4*h + r%4, col j)
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int n = n0 + (wn * TN + t) * 32 + lj;
    if (n >= N) continue;
    const float bv = bias ? (float)bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (m < M) {
          half_t h = (half_t)(acc[i][t][r] + bv);
          if (residual) h = h + residual[(int64_t)m * N + n];
          Y[(int64_t)m * N + n] = h;
        }
      }
    }
  }
}

template <int TM, int TN, int WM, int WN, int WPE>
static int launch_gemm(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                       const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M,
                       int64_t N, int64_t K, hipStream_t stream) {
  using Cfg = GemmCfg<TM, TN, WM, WN>;
  const int tiles_m = (int)((M + Cfg::BM - 1) / Cfg::BM);
  const int tiles_n = (int)((N + Cfg::BN - 1) / Cfg::BN);
  auto kern = q4g32_gemm_kernel<TM, TN, WM, WN, WPE>;
  if (Cfg::kLdsBytes > 64 * 1024) {
    WQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::kLdsBytes));
  }
  WQ_LAUNCH("wq_q4g32_gemm", kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(Cfg::kThreads),
            Cfg::kLdsBytes, stream, W, (const half_t*)S, (const half_t*)x, (const half_t*)bias,
            (const half_t*)residual, (half_t*)y, (int)M, (int)N, (int)K, tiles_m, tiles_n);
  return WQ_OK;
}

}  // namespace wq

// Tile shape override for measurement (0 = choose from the problem shape).
static int g_gemm_cfg_override = 0;
extern "C" __attribute__((visibility("default"))) void wq_debug_set_gemm_config(int cfg) { g_gemm_cfg_override = cfg; }

extern "C" int wq_q4g32_gemm(const uint32_t* W, const uint16_t* S, const uint16_t* x,
                             const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M,
                             int64_t N, int64_t K, wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, "wq_q4g32_gemm: negative dimension");
  WQ_REQUIRE(K % 32 == 0, "wq_q4g32_gemm: K=%lld must be a multiple of the group size 32",
             (long long)K);
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0, "wq_q4g32_gemm: K must be positive");
  WQ_REQUIRE(W && S && x && y, "wq_q4g32_gemm: null pointer");
  WQ_REQUIRE(aligned16(W) && aligned16(x), "wq_q4g32_gemm: W and x must be 16-byte aligned");
  WQ_REQUIRE(M < (1ll << 30) && N < (1ll << 30) && K < (1ll << 30), "wq_q4g32_gemm: too large");
  int cfg = g_gemm_cfg_override;
  if (cfg == 0) {
    const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256);
    if (M <= 64)
      cfg = 3;
    else if (t256 >= 256 && t256 % 256 == 0)
      cfg = 1;
    else
      cfg = 2;
  }
  switch (cfg) {
    case 1: return launch_gemm<8, 2, 1, 4, 1>(W, S, x, bias, residual, y, M, N, K, stream);   // 256x256
    case 2: return launch_gemm<4, 2, 1, 4, 2>(W, S, x, bias, residual, y, M, N, K, stream);   // 128x256
    case 3: return launch_gemm<2, 1, 1, 4, 2>(W, S, x, bias, residual, y, M, N, K, stream);   // 64x128
    case 4: return launch_gemm<2, 2, 2, 2, 2>(W, S, x, bias, residual, y, M, N, K, stream);   // 128x128
    default: return fail(WQ_EINVAL, "wq_q4g32_gemm: unknown tile configuration %d", cfg);
  }
}
