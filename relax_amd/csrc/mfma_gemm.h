// Weight-only quantized GEMM on the gfx950 matrix cores, shared by both weight formats:
//   C[m,n] = epilogue( sum_k A[m,k] * dequant(B)[k,n] )       fp16 MFMA, fp32 accumulate
//
// Work split.  A workgroup of WM x WN wavefronts owns a BM x BN tile of C.  The
// activation tile (BM x 64 halves per K-step) is shared through LDS; the weight
// tile never touches LDS: v_mfma_f32_32x32x16_f16 wants, in lane (j, h), 8 K-values
// of column j for K-half h, and in every supported format those 8 values are a few
// bytes of one packed word the lane loads itself.  Per K-step (64 k) lane (j, h)
// loads the packed weights of column n0+j for k = 32h .. 32h+31 together with
// their scale, dequantizes them in registers (the Loader policy, which uses the
// same device functions as the stand-alone dequantize entry points) and feeds
// four MFMAs; MFMA number kk of the step consumes k = 32h + 8kk .. +7 of its
// lane, i.e. 16-byte chunk (4h + kk) of every activation row.
//
// K labelling.  An MFMA only needs A and B to agree on which K sits in which
// (half, element) slot.  A Loader whose unpack yields the pairing (i, i+4) inside
// each group of 8 (format A) sets kPairA, and the activations are rearranged to
// that pairing once, when they are written to LDS.
//
// LDS layout of the activation tile: row r, chunk c (16 bytes) at
// r*128 + ((c ^ (r & 7)) * 16): the XOR spreads the 32 rows a wavefront reads
// at one chunk index over all banks.
#ifndef RELAX_AMD_CSRC_MFMA_GEMM_H_
#define RELAX_AMD_CSRC_MFMA_GEMM_H_

#include "gemm_epilogue.h"
#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

constexpr int kBK = 64;     // K elements per step
constexpr int kChunks = 8;  // 16-byte chunks per activation row per step

template <int TM, int TN, int WM, int WN>
struct GemmCfg {
  static constexpr int kThreads = 64 * WM * WN;
  static constexpr int BM = 32 * TM * WM;
  static constexpr int BN = 32 * TN * WN;
  static constexpr int kAChunks = BM * kChunks;            // 16-byte chunks of A per step
  static constexpr int kAPerThread = kAChunks / kThreads;  // chunks each thread stages
  static constexpr int kLdsBytes = 2 * BM * kBK * 2;       // double buffered
  static_assert(kAChunks % kThreads == 0, "tile must divide evenly among threads");
};

__device__ __forceinline__ int lds_a_offset(int row, int chunk) {
  return row * (kBK * 2) + ((chunk ^ (row & 7)) << 4);
}

// Loader policy interface:
//   static constexpr bool kPairA;
//   struct Args;  struct Lane;  struct Frag;
//   static void init(Lane&, const Args&, int n, int lh, int K, int N);   n is already clamped
//   static void load(Frag&, const Lane&, const Args&, int ks, int lh, int K, bool ktail);
//   static void dequant(const Frag&, half8_t out[4]);                    operands of the 4 MFMAs
// Epilogue policy interface: see gemm_epilogue.h.
template <class Loader, class Epilogue, int TM, int TN, int WM, int WN, int WAVES_PER_EU, bool KTAIL>
__global__ __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(WAVES_PER_EU, WAVES_PER_EU)))
void wq_mfma_gemm_kernel(typename Loader::Args bargs, const half_t* __restrict__ X,
                         half_t* __restrict__ Y, Epilogue epilogue, int M, int N, int K,
                         int tiles_m, int tiles_n) {
  using Cfg = GemmCfg<TM, TN, WM, WN>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int lj = lane & 31, lh = lane >> 5;

  // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2): give
  // every XCD a contiguous range of tiles, walked M-fastest so that neighbours on
  // one XCD share their weight columns.
  const int nblk = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblk / 8, rem = nblk % 8;
    const int xcd = pid & 7, idx = pid >> 3;
    pid = xcd * per + min(xcd, rem) + idx;
  }
  const int tile_m = pid % tiles_m, tile_n = pid / tiles_m;
  const int m0 = tile_m * Cfg::BM, n0 = tile_n * Cfg::BN;

  const int KW = K >> 3;  // 16-byte... 8-element words per activation row
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

  // ---- per-lane weight pointers ----
  typename Loader::Lane blane[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int gn = min(n0 + (wn * TN + t) * 32 + lj, N - 1);  // clamped: never stored
    Loader::init(blane[t], bargs, gn, lh, K, N);
  }

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.0f;

  uint4_t a_reg[Cfg::kAPerThread];
  typename Loader::Frag b_reg[TN];

  auto load_global = [&](int ks) {
#pragma unroll
    for (int t = 0; t < TN; ++t) Loader::load(b_reg[t], blane[t], bargs, ks, lh, K, KTAIL);
#pragma unroll
    for (int i = 0; i < Cfg::kAPerThread; ++i) {
      if (!KTAIL || ks * kChunks + a_chunk[i] < KW)
        a_reg[i] = a_src[i][ks * kChunks];
      else
        a_reg[i] = uint4_t{0u, 0u, 0u, 0u};
    }
  };

  auto store_a = [&](int buf) {
    unsigned char* base = lds + buf * (Cfg::BM * kBK * 2);
#pragma unroll
    for (int i = 0; i < Cfg::kAPerThread; ++i) {
      uint4_t v = a_reg[i];
      if (Loader::kPairA) {
        uint32_t in[4] = {v.x, v.y, v.z, v.w}, o[4];
        pair_i_i4(in, o);
        v = uint4_t{o[0], o[1], o[2], o[3]};
      }
      *reinterpret_cast<uint4_t*>(base + lds_a_offset(a_row[i], a_chunk[i])) = v;
    }
  };

  load_global(0);
  store_a(0);
  __syncthreads();

  for (int ks = 0; ks < ksteps; ++ks) {
    const int buf = ks & 1;
    // B operands of this step, dequantized: bop[t][kk] = 8 halves
    half8_t bop[TN][4];
#pragma unroll
    for (int t = 0; t < TN; ++t) Loader::dequant(b_reg[t], bop[t]);
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

  // ---- epilogue ----
  // Row-wise through LDS (gemm_epilogue.h): the activation buffers are idle after the last
  // barrier of the loop, and each wavefront stages in a piece of its own.
  if (epilogue.wide_ok(N, Y)) {
    using ECfg = RowwiseEpilogueCfg<TM, TN>;
    static_assert(WM * WN * ECfg::kBytesPerWave <= Cfg::kLdsBytes, "epilogue staging exceeds the activation buffers");
    store_tile_rowwise<Epilogue, TM, TN>(acc, epilogue, Y, M, N, m0 + wm * TM * 32, n0 + wn * TN * 32,
                                         lds + wave * ECfg::kBytesPerWave, lane);
    return;
  }
  // element-wise: accumulator register r of lane (j, h) is element (row 8*(r/4) + 4*h + r%4, col j)
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int n = n0 + (wn * TN + t) * 32 + lj;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (m < M) Y[(int64_t)m * N + n] = epilogue(acc[i][t][r], m, n);
      }
    }
  }
}

template <class Loader, class Epilogue, int TM, int TN, int WM, int WN, int WPE>
static int launch_mfma_gemm(const char* who, const typename Loader::Args& bargs, const uint16_t* x,
                            uint16_t* y, const Epilogue& ep, int64_t M, int64_t N, int64_t K,
                            hipStream_t stream) {
  using Cfg = GemmCfg<TM, TN, WM, WN>;
  const int tiles_m = (int)((M + Cfg::BM - 1) / Cfg::BM);
  const int tiles_n = (int)((N + Cfg::BN - 1) / Cfg::BN);
  auto kern = (K % kBK == 0) ? wq_mfma_gemm_kernel<Loader, Epilogue, TM, TN, WM, WN, WPE, false>
                             : wq_mfma_gemm_kernel<Loader, Epilogue, TM, TN, WM, WN, WPE, true>;
  if (Cfg::kLdsBytes > 64 * 1024) {
    static DynamicLdsLimit limit_full, limit_tail;  // one per kernel of this launcher
    WQ_HIP((K % kBK == 0 ? limit_full : limit_tail).ensure(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes));
  }
  WQ_LAUNCH(who, kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(Cfg::kThreads), Cfg::kLdsBytes,
            stream, bargs, (const half_t*)x, (half_t*)y, ep, (int)M, (int)N, (int)K, tiles_m,
            tiles_n);
  return WQ_OK;
}

// Tile shapes.  cfg: 1 = 256x256 (one wavefront per SIMD), 2 = 128x256, 3 = 64x128
// (small M), 4 = 128x128 (2x2 wavefronts).
template <class Loader, class Epilogue>
static int launch_mfma_gemm_cfg(int cfg, const char* who, const typename Loader::Args& bargs,
                                const uint16_t* x, uint16_t* y, const Epilogue& ep, int64_t M,
                                int64_t N, int64_t K, hipStream_t stream) {
  switch (cfg) {
    case 1: return launch_mfma_gemm<Loader, Epilogue, 8, 2, 1, 4, 1>(who, bargs, x, y, ep, M, N, K, stream);
    case 2: return launch_mfma_gemm<Loader, Epilogue, 4, 2, 1, 4, 2>(who, bargs, x, y, ep, M, N, K, stream);
    case 3: return launch_mfma_gemm<Loader, Epilogue, 2, 1, 1, 4, 2>(who, bargs, x, y, ep, M, N, K, stream);
    case 4: return launch_mfma_gemm<Loader, Epilogue, 2, 2, 2, 2, 2>(who, bargs, x, y, ep, M, N, K, stream);
    default: return fail(WQ_EINVAL, "%s: unknown tile configuration %d", who, cfg);
  }
}

// Tile shape from the problem shape, from timings at M = 96 .. 2048 of the Llama-7B shapes
// (format A) and of K = 8192, N = 28672 (format B): what matters at mid M is the number of
// tiles against 256 CUs.  Register-staged kernel (fine-grained format B, and format A when K is
// not a multiple of 64): 64x128 up to M = 128, 128x128 up to 256, else 128x256.  Fully
// LDS-staged kernel: 128x128 tiles, two workgroups per CU (17) up to M = 384, above that
// 256x256 with one wavefront per SIMD (11), except for narrow matrices at moderate M, where
// 256x128 tiles (13) give the CUs twice as many tiles (N = 4096, K = 11008, M = 1024: 140 -> 131 us).
inline int choose_gemm_cfg(int64_t M, int64_t N, bool lds_staged) {
  if (!lds_staged) return M <= 128 ? 3 : M <= 256 ? 4 : 2;
  if (M <= 384) return 17;
  return (N <= 4096 && M <= 1536) ? 13 : 11;
}

// The fully LDS-staged kernel's tile shape for the 4-bit row-major formats (q4f16_1, AutoGPTQ after its
// load-time conversion): the choice above, then 256 x 128 tiles, one workgroup per CU and a four-slot ring (18)
// where they make at most one round of the machine (M = 2048, N = 4096, K = 11008: 208 -> 193 us; M = 1024:
// 141 -> 116 us; M = 256, N = 12288, K = 4096: 42 -> 39 us); up to 128 rows only for narrow matrices, where
// 128 x 128 tiles (17) are too few (N = 4096: 35 -> 30 us; N = 12288: 33 against 38 us).
inline int choose_q4_lds_cfg(int64_t M, int64_t N, int cus) {
  int cfg = choose_gemm_cfg(M, N, true);
  if ((cfg == 11 || cfg == 13 || (cfg == 17 && (M > 128 || N <= 6144))) &&
      ((M + 255) / 256) * ((N + 127) / 128) <= cus)
    cfg = 18;
  return cfg;
}

}  // namespace wq
#endif  // RELAX_AMD_CSRC_MFMA_GEMM_H_
