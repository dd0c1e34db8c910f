// Small-batch weight-streaming GEMM (2 <= M <= 64) shared by both weight formats.
//
// At small M a quantized linear layer is still a weight stream (HBM-bound), but the
// products are done by the matrix cores so that all M rows share ONE pass over the
// weights (the GEMV kernels re-read the weights every few rows and pay VALU work per
// row).  This is the counterpart of the reference's dlight LowBatchGEMV rule
// (python/tvm/dlight/gpu/low_batch_gemv.py).
//
// Work split.  A workgroup (WAVES wavefronts, arranged NW x KW) owns 16*NW output
// columns and all M rows.  Wavefront (nw, kw) owns columns n0 + 16*nw .. +15 and the
// K-steps kw, kw + KW, kw + 2*KW, ... of 128 k each.  One step of one wavefront is
// 4*TM MFMA 16x16x32: lane (j, kq) holds, for both operands, the 32 consecutive k
// 128*step + 32*kq .. +31 of column j (row j of the activations), of which MFMA t takes
// k 8t .. 8t+7.  The weight format (a Policy) says where those 32 codes live, how
// many 16-byte pieces they are and how they unpack into the four B operands, in
// natural k order, so the activations need no rearrangement.
//
// Everything travels global -> LDS with direct loads into a ring of `stages` slots,
// `stages - 1` steps ahead: per step the rows x 128 activation slab of each kw
// (shared by the NW wavefronts of that kw, each loading a part), and per wavefront
// its codes and scales (or, where the policy and K allow, all scales of the column block
// once, ahead of the ring).  A wavefront waits for its own loads with s_waitcnt vmcnt(n);
// when NW > 1 one s_barrier per step makes the shared slab visible.  The KW partial
// sums of a column block meet in LDS at the end.
//
// What bounds it: per 16 columns every workgroup re-reads all of the activations
// (from L2), and unpacking costs about two VALU operations per weight, so eight
// wavefronts per workgroup (two per SIMD) are used to overlap one wavefront's
// unpacking with another's loads, and NW grows with M and N to cut the re-reads.
#ifndef RELAX_AMD_CSRC_SKINNY_GEMM_H_
#define RELAX_AMD_CSRC_SKINNY_GEMM_H_

#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

#define WQ_SK_WAITCNT_VM(n) __builtin_amdgcn_s_waitcnt(((n)&0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

typedef const void __attribute__((address_space(1))) * wq_sk_gptr_t;
typedef void __attribute__((address_space(3))) * wq_sk_lptr_t;

// A Policy provides
//   kPieces            16-byte pieces of codes per lane and step (32 k)
//   kScaleDma          true: a scale per lane and step, fetched as the 4-byte pair that holds it
//   Args, Lane         kernel argument block / per-lane state
//   init(lane, args, n, K, N)
//   w_addr(lane, k0, p)        address of piece p of the 32 codes starting at k0 (k0 % 32 == 0)
//   s_addr(lane, k0)           4-byte aligned address of the pair holding the scale for k0   (kScaleDma)
//   Scale                      what dequant needs besides the codes (half_t, or scale and zero point)
//   pick_scale(lane, pair, kq) the lane's Scale from that pair                               (kScaleDma)
//   const_scale(lane)          the lane's Scale                                              (!kScaleDma)
//   null_scale()               a Scale that turns every code into an exact zero (weights past K)
//   dequant(pieces, s, out[4]) -> B operands of MFMA 0..3 (k 8t .. 8t+7 each), scaled
//   s_pair_addr(lane, k0)      like s_addr, for every policy (a fixed scale: the pair that holds it)
//   kCanScaleBlock             true (needs kScaleDma): the scales of a column are 2-byte values, contiguous
//                              along K, one per 32 k; where scale_block_ok(args, K) the ring kernel may
//                              fetch all scales of a column block once, 16 bytes per lane, instead of a
//                              pair per lane and step
//   sblock_addr(lane, g)       address of scale g of the lane's column (g % 8 == 0)       (kCanScaleBlock)
//   scale_block_ok(args, K)    host: every 8 scales of a column are 16 aligned bytes      (kCanScaleBlock)
//   pair_aligned(args)         host: whether those pairs are 4-byte aligned
constexpr int kScaleBlockMaxK = 11264;  // a column block's scales for all of K stay in LDS: K bytes
inline int scale_block_stride(int K) { return ((K + 1023) >> 10) << 10; }

template <typename Policy, int TH, int NW, int WAVES, bool SB = false>
struct SkinnyCfg {
  static constexpr int KW = WAVES / NW;
  static_assert(NW * KW == WAVES && (WAVES == 4 || WAVES == 8), "wavefront arrangement");
  static constexpr int kRows = 8 * TH;                   // activation rows held (M <= kRows)
  static constexpr int TM = (TH + 1) / 2;                // 16-row MFMA tiles
  static_assert((2 * TH) % NW == 0, "the slab loads divide among the wavefronts of one kw");
  static constexpr int kSlabBytes = kRows * 256;         // rows x 128 k
  static constexpr int kXBytes = KW * kSlabBytes;
  static constexpr int kWBytes = WAVES * Policy::kPieces * 1024;
  static constexpr bool kStepScale = Policy::kScaleDma && !SB;  // a scale load per lane and step
  static constexpr int kStageBytes = kXBytes + kWBytes + (kStepScale ? WAVES * 256 : 0);
  static constexpr int kXLoads = 2 * TH / NW;            // slab loads (4 rows each) per wavefront and step
  static constexpr int kLoadsPerStep = kXLoads + Policy::kPieces + (kStepScale ? 1 : 0);
  static constexpr int kMaxAhead = 63 / kLoadsPerStep;   // vmcnt holds 6 bits
  static constexpr int kRedBytes = WAVES * TM * 4 * 64 * 4;
};

// s_waitcnt vmcnt(groups * L) for a wavefront-uniform run-time `groups` (<= 8)
template <int L>
__device__ __forceinline__ void wait_newer_groups(int groups) {
  switch (groups) {
    case 0: WQ_SK_WAITCNT_VM(0); break;
    case 1: WQ_SK_WAITCNT_VM(1 * L <= 63 ? 1 * L : 63); break;
    case 2: WQ_SK_WAITCNT_VM(2 * L <= 63 ? 2 * L : 63); break;
    case 3: WQ_SK_WAITCNT_VM(3 * L <= 63 ? 3 * L : 63); break;
    case 4: WQ_SK_WAITCNT_VM(4 * L <= 63 ? 4 * L : 63); break;
    case 5: WQ_SK_WAITCNT_VM(5 * L <= 63 ? 5 * L : 63); break;
    case 6: WQ_SK_WAITCNT_VM(6 * L <= 63 ? 6 * L : 63); break;
    case 7: WQ_SK_WAITCNT_VM(7 * L <= 63 ? 7 * L : 63); break;
    default: WQ_SK_WAITCNT_VM(8 * L <= 63 ? 8 * L : 63); break;
  }
}

template <typename Policy, typename Epilogue, int TH, int NW, int WAVES, bool SB>
__global__ __launch_bounds__(64 * WAVES) void skinny_gemm_kernel(
    typename Policy::Args pargs, const half_t* __restrict__ X, half_t* __restrict__ Y, Epilogue epi,
    int M, int N, int K, int stages) {
  using Cfg = SkinnyCfg<Policy, TH, NW, WAVES, SB>;
  constexpr int KW = Cfg::KW, TM = Cfg::TM, P = Policy::kPieces;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = wave / KW, kw = wave % KW;
  const int lj = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.x * (16 * NW);
  const int total_steps = (K + 127) >> 7;               // 128-k steps over K
  const int nsteps = (total_steps + KW - 1) / KW;       // per wavefront (the last may be partly empty)
  const int ahead = stages - 1;

  // ---- per-lane sources ----
  // slab load i of this wavefront: rows 4*li .. 4*li+3 of the slab, li = nw*kXLoads + i;
  // LDS position p of a row holds the 16-byte chunk p ^ (row & 15) (bank-conflict-free reads)
  const char* x_row[Cfg::kXLoads];
  int x_chunk[Cfg::kXLoads];
#pragma unroll
  for (int i = 0; i < Cfg::kXLoads; ++i) {
    const int li = nw * Cfg::kXLoads + i;
    const int row = 4 * li + (lane >> 4);
    x_chunk[i] = (lane & 15) ^ (row & 15);
    x_row[i] = reinterpret_cast<const char*>(X + (int64_t)min(row, M - 1) * K);
  }
  typename Policy::Lane pl;
  Policy::init(pl, pargs, min(n0 + 16 * nw + lj, N - 1), K, N);  // clamped columns are never stored
  typename Policy::Scale s_fixed = Policy::null_scale();
  if (!Policy::kScaleDma) s_fixed = Policy::const_scale(pl);

  unsigned char* const w_area = lds + Cfg::kXBytes + wave * (P * 1024);
  unsigned char* const s_area = lds + Cfg::kXBytes + Cfg::kWBytes + wave * 256;
  // SB: all scales of the column block (K / 32 per column), as chunks of 32 per column: chunk c is
  // one load of one wavefront, lane (j, q) bringing scales 32c + 8q .. + 7 of column j
  unsigned char* const s_block = lds + stages * Cfg::kStageBytes + nw * ((((K + 1023) >> 10)) << 10);

  auto issue = [&](int it, int slot) {
    const int stage_off = slot * Cfg::kStageBytes;
    const int ks = it * KW + kw;
    const int k0 = 128 * ks + 32 * kq;             // this lane's 32 weights
    const int k0c = k0 < K ? k0 : 0;               // past the end: any valid address (scale is zeroed)
#pragma unroll
    for (int i = 0; i < Cfg::kXLoads; ++i) {
      const int kchunk = ks * 16 + x_chunk[i];     // 16-byte chunk index along the row
      const int64_t off = (kchunk * 8 < K) ? (int64_t)kchunk * 16 : 0;
      __builtin_amdgcn_global_load_lds(
          (wq_sk_gptr_t)(x_row[i] + off),
          (wq_sk_lptr_t)(lds + stage_off + kw * Cfg::kSlabBytes + (nw * Cfg::kXLoads + i) * 1024), 16, 0, 0);
    }
#pragma unroll
    for (int p = 0; p < P; ++p)
      __builtin_amdgcn_global_load_lds((wq_sk_gptr_t)Policy::w_addr(pl, k0c, p),
                                       (wq_sk_lptr_t)(w_area + stage_off + p * 1024), 16, 0, 0);
    if constexpr (Cfg::kStepScale)
      __builtin_amdgcn_global_load_lds((wq_sk_gptr_t)Policy::s_addr(pl, k0c),
                                       (wq_sk_lptr_t)(s_area + stage_off), 4, 0, 0);
  };

  float4_t acc[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) acc[i] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

  auto compute = [&](int it, int slot) {
    const int stage_off = slot * Cfg::kStageBytes;
    const int k0 = 128 * (it * KW + kw) + 32 * kq;
    uint4_t pieces[P];
#pragma unroll
    for (int p = 0; p < P; ++p)
      pieces[p] = *reinterpret_cast<const uint4_t*>(w_area + stage_off + p * 1024 + lane * 16);
    typename Policy::Scale s = s_fixed;
    if constexpr (Cfg::kStepScale)
      s = Policy::pick_scale(pl, *reinterpret_cast<const half2_t*>(s_area + stage_off + lane * 4), kq);
    if constexpr (SB) {
      const int g = (k0 < K ? k0 : 0) >> 5;  // chunk g / 32, fetched by lane (j, (g / 8) % 4)
      s = *reinterpret_cast<const half_t*>(s_block + (g >> 5) * 1024 + (((g >> 3) & 3) * 16 + lj) * 16 +
                                           (g & 7) * 2);
    }
    if (k0 >= K) s = Policy::null_scale();  // code * 0 = exact zero for the weights past K
    half8_t bop[4];
    Policy::dequant(pieces, s, bop);
    const unsigned char* slab = lds + stage_off + kw * Cfg::kSlabBytes;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        // rows past the slab (M <= 8 uses half a tile) re-read a held row: never stored
        const int row = (16 * i + lj < Cfg::kRows) ? 16 * i + lj : 16 * i + (lj & 7);
        const half8_t aop =
            *reinterpret_cast<const half8_t*>(slab + row * 256 + (((4 * kq + t) ^ (row & 15)) << 4));
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, bop[t], acc[i], 0, 0, 0);
      }
    }
  };

  // ---- prologue: the scale block (its loads are older than every step's, so each wavefront's
  // part has landed when its first wait returns; the barrier of step 0 covers the others'), then
  // fill the ring ----
  if constexpr (SB) {
    for (int c = kw; c * 1024 < K; c += KW) {
      const int g = 32 * c + 8 * kq;
      __builtin_amdgcn_global_load_lds((wq_sk_gptr_t)Policy::sblock_addr(pl, g * 32 < K ? g : 0),
                                       (wq_sk_lptr_t)(s_block + c * 1024), 16, 0, 0);
    }
  }
  for (int p = 0; p < ahead && p < nsteps; ++p) issue(p, p);
  int cslot = 0;                       // slot of the step being computed
  int islot = ahead % stages;          // slot the next issue goes to
  for (int it = 0; it < nsteps; ++it) {
    const int newer = min(ahead - 1, nsteps - 1 - it);  // steps issued after step `it`
    wait_newer_groups<Cfg::kLoadsPerStep>(newer);
    if (NW > 1 || (SB && KW > 1 && it == 0)) __builtin_amdgcn_s_barrier();
    // the slot refilled now was computed in the previous iteration (by everyone: barrier above)
    if (it + ahead < nsteps) {
      issue(it + ahead, islot);
      islot = islot + 1 == stages ? 0 : islot + 1;
    }
    compute(it, cslot);
    cslot = cslot + 1 == stages ? 0 : cslot + 1;
  }

  // ---- reduce the KW partial sums of each column block through LDS, then store ----
  if (KW > 1) {
    __syncthreads();  // all ring slots idle
    float* red = reinterpret_cast<float*>(lds);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[((wave * TM + i) * 4 + r) * 64 + lane] = acc[i][r];
    __syncthreads();
    if (kw == 0) {
#pragma unroll
      for (int o = 1; o < KW; ++o)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][r] += red[(((wave + o) * TM + i) * 4 + r) * 64 + lane];
    }
  }
  if (kw == 0) {
    const int col = n0 + 16 * nw + lj;
    if (col < N) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = 16 * i + 4 * kq + r;
          if (m < M) Y[(int64_t)m * N + col] = epi(acc[i][r], m, col);
        }
    }
  }
}


constexpr int kSkinnyLdsBudget = 156 * 1024;  // of the 160 KB of a CU

// ---------------------------------------------------------------------------------
// M <= 16: the activations stay in registers.
//
// The ring kernel above re-reads the activations once per workgroup and keeps two thirds
// of its loads in flight on those slabs; loads retire in order, so its weight stream is
// only as deep as the slab ring.  For one 16-row tile the activations fit the register
// file instead: a workgroup's WAVES wavefronts split K into contiguous runs of NSTEP
// steps of 128 k, and wavefront w keeps the MFMA A operands of its run (16 rows x
// 128*NSTEP k: 16*NSTEP registers) for the whole kernel.  The workgroups are persistent
// (one per CU) and walk over 16-column tiles; the only loads inside the walk are the
// codes and scales, through a wavefront-private ring in LDS that runs kDepth steps ahead
// (across tiles).  Per tile the WAVES partial sums meet in LDS and one wavefront (taking
// turns) adds them and stores.  Measured: with loads only it streams 2 TB/s however
// deep the ring (and no more from sixteen wavefronts than from eight), so it wins where
// the ring kernel pays most for the slabs (K = 8192, many tiles per CU) and loses at
// K = 4096.
//
// Every policy hands its scale over as a 4-byte pair per lane and step here
// (Policy::s_pair_addr), so that the walk has no load the compiler must wait for.
template <typename Policy, int NSTEP, int WAVES>
struct XregCfg {
  static constexpr int kStepBytes = Policy::kPieces * 1024 + 256;
  static constexpr int kLoadsPerStep = Policy::kPieces + 1;
  static constexpr int kRedBytes = 2 * WAVES * 1024;
  static constexpr int kFit = (kSkinnyLdsBudget - kRedBytes) / (WAVES * kStepBytes);
  static constexpr int kCount = 63 / kLoadsPerStep + 1;  // vmcnt holds 6 bits
  static constexpr int kWant = 3 * NSTEP;
  static constexpr int kDepth = kFit < kCount ? (kFit < kWant ? kFit : kWant) : (kCount < kWant ? kCount : kWant);
  static_assert(kDepth >= 2, "ring too small");
  static constexpr int kLdsBytes = WAVES * kDepth * kStepBytes + kRedBytes;
};

template <typename Policy, typename Epilogue, int NSTEP, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void skinny_xreg_kernel(
    typename Policy::Args pargs, const half_t* __restrict__ X, half_t* __restrict__ Y, Epilogue epi,
    int M, int N, int K) {
  using Cfg = XregCfg<Policy, NSTEP, WAVES>;
  constexpr int P = Policy::kPieces, L = Cfg::kLoadsPerStep, D = Cfg::kDepth;
  constexpr int QA = D / NSTEP;  // the step D ahead of step s is step (s + D) % NSTEP, QA or QA + 1 tiles ahead
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lj = lane & 15, kq = lane >> 4;
  const int tiles = (N + 15) >> 4;
  const int grid = gridDim.x;
  unsigned char* const ring = lds + wave * (D * Cfg::kStepBytes);
  float4_t* const red = reinterpret_cast<float4_t*>(lds + WAVES * D * Cfg::kStepBytes);

  // ---- the A operands of this wavefront's run of K (zero past M and past K) ----
  half8_t a[NSTEP][4];
  int k0c[NSTEP];  // this lane's 32 weights of step s (any valid k when past K: they meet zeros)
#pragma unroll
  for (int s = 0; s < NSTEP; ++s) {
    const int k0 = (wave * NSTEP + s) * 128 + 32 * kq;
    const bool held = lj < M && k0 < K;
    k0c[s] = k0 < K ? k0 : 0;
    const half_t* src = held ? X + (int64_t)lj * K + k0 : X;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const half8_t v = *reinterpret_cast<const half8_t*>(src + 8 * t);
      a[s][t] = held ? v : half8_t{};
    }
  }

  // lane state of the tiles QA and QA + 1 tiles ahead (whose loads are being issued)
  typename Policy::Lane pl[2];
  bool valid[2] = {false, false};
  auto set_tile = [&](int which, int tile) {
    valid[which] = tile < tiles;  // past the end: every lane re-reads one address
    Policy::init(pl[which], pargs, min(min(tile, tiles - 1) * 16 + lj, N - 1), K, N);
  };
  auto issue = [&](int which, int s, int slot) {
    unsigned char* dst = ring + slot * Cfg::kStepBytes;
#pragma unroll
    for (int p = 0; p < P; ++p)
      __builtin_amdgcn_global_load_lds(
          (wq_sk_gptr_t)(valid[which] ? Policy::w_addr(pl[which], k0c[s], p) : reinterpret_cast<const char*>(X)),
          (wq_sk_lptr_t)(dst + p * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds(
        (wq_sk_gptr_t)(valid[which] ? Policy::s_pair_addr(pl[which], k0c[s]) : reinterpret_cast<const char*>(X)),
        (wq_sk_lptr_t)(dst + P * 1024), 4, 0, 0);
  };

  // ---- prologue: the first D steps (slot = flat step % D) ----
#pragma unroll
  for (int f = 0; f < D; ++f) {
    if (f % NSTEP == 0) set_tile(0, blockIdx.x + (f / NSTEP) * grid);
    issue(0, f % NSTEP, f);
  }
  // the activations are in registers before the walk starts
#pragma unroll
  for (int s = 0; s < NSTEP; ++s)
#pragma unroll
    for (int t = 0; t < 4; ++t) asm volatile("" : "+v"(a[s][t]));
  typename Policy::Lane pl0;  // for pick_scale, which depends on the lane only
  Policy::init(pl0, pargs, min(blockIdx.x * 16 + lj, N - 1), K, N);
  set_tile(0, blockIdx.x + QA * grid);

  int slot = 0;  // of step 0 of the current tile
  int turn = 0;
  for (int tile = blockIdx.x; tile < tiles; tile += grid) {
    set_tile(1, tile + (QA + 1) * grid);
    float4_t acc = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < NSTEP; ++s) {
      WQ_SK_WAITCNT_VM((D - 1) * L);  // issued after this step's loads: the D - 1 steps that follow it
      int sl = slot + s;
      if (sl >= D) sl -= D;
      const unsigned char* src = ring + sl * Cfg::kStepBytes;
      uint4_t pieces[P];
#pragma unroll
      for (int p = 0; p < P; ++p) pieces[p] = *reinterpret_cast<const uint4_t*>(src + p * 1024 + lane * 16);
      const half2_t pair = *reinterpret_cast<const half2_t*>(src + P * 1024 + lane * 4);
      half8_t bop[4];
      Policy::dequant(pieces, Policy::pick_scale(pl0, pair, kq), bop);
#pragma unroll
      for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s][t], bop[t], acc, 0, 0, 0);
      // the slot is free once its contents are in registers; it takes the step D ahead
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue((s + D) / NSTEP - QA, (s + D) % NSTEP, sl);
    }
    slot = (slot + NSTEP) % D;
    pl[0] = pl[1];
    valid[0] = valid[1];

    // ---- the WAVES partial sums of the tile meet in LDS (two buffers, by turns) ----
    float4_t* const buf = red + (turn & 1) * (WAVES * 64);
    buf[wave * 64 + lane] = acc;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (wave == turn % WAVES) {
      float4_t sum = buf[lane];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        const float4_t v = buf[w * 64 + lane];
        sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
      }
      const int col = tile * 16 + lj;
      if (col < N) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = 4 * kq + r;
          if (m < M) Y[(int64_t)m * N + col] = epi(sum[r], m, col);
        }
      }
    }
    ++turn;
  }
  WQ_SK_WAITCNT_VM(0);  // the loads past the last tile land before the LDS is given back
}

template <typename Policy, typename Epilogue, int NSTEP, int WAVES>
static int launch_xreg(const char* who, const typename Policy::Args& pargs, const uint16_t* x, uint16_t* y,
                       const Epilogue& epi, int64_t M, int64_t N, int64_t K, hipStream_t stream) {
  using Cfg = XregCfg<Policy, NSTEP, WAVES>;
  auto kern = skinny_xreg_kernel<Policy, Epilogue, NSTEP, WAVES>;
  const int64_t tiles = (N + 15) / 16;
  const int64_t blocks = tiles < cu_count() ? tiles : cu_count();
  static DynamicLdsLimit limit;  // per instantiation
  WQ_HIP(limit.ensure(reinterpret_cast<const void*>(kern), 160 * 1024));
  WQ_LAUNCH(who, kern, dim3((unsigned)blocks), dim3(64 * WAVES), Cfg::kLdsBytes, stream, pargs,
            (const half_t*)x, (half_t*)y, epi, (int)M, (int)N, (int)K);
  return WQ_OK;
}

// K up to 64 steps of 128 (8192) is held by 8 wavefronts x 4 or 8 steps (64 or 128 registers;
// 11 steps for K = 11008 spill)
inline bool xreg_fits(int64_t M, int64_t K) { return M <= 16 && K <= 64 * 128; }

template <typename Policy, typename Epilogue>
static int launch_xreg_auto(const char* who, const typename Policy::Args& pargs, const uint16_t* x,
                            uint16_t* y, const Epilogue& epi, int64_t M, int64_t N, int64_t K,
                            hipStream_t stream) {
  const int64_t steps = (K + 127) / 128;
  if (steps <= 32) return launch_xreg<Policy, Epilogue, 4, 8>(who, pargs, x, y, epi, M, N, K, stream);
  return launch_xreg<Policy, Epilogue, 8, 8>(who, pargs, x, y, epi, M, N, K, stream);
}

// overrides for tests and measurement (tuning.h; 0 = automatic)
// waves: 1 = the ring kernel, 2 = the kernel that holds the activations in registers (where it fits)
struct SkinnyTuning {
  int nw, stages, waves;
};
inline SkinnyTuning skinny_tuning() {
  const Tuning& t = tuning();
  return SkinnyTuning{t.skinny_nw, t.skinny_stages, t.skinny_waves};
}

template <typename Policy, typename Epilogue, int TH, int NW, int WAVES, bool SB = false>
static int launch_skinny(const char* who, const typename Policy::Args& pargs, const uint16_t* x, uint16_t* y,
                         const Epilogue& epi, int64_t M, int64_t N, int64_t K, int want_stages,
                         hipStream_t stream) {
  // one fetch of all scales where the policy allows it and the block is small (two column
  // blocks at most: more would cost a workgroup per CU)
  if constexpr (!SB && Policy::kCanScaleBlock && NW <= 2) {
    if (K <= kScaleBlockMaxK && Policy::scale_block_ok(pargs, K) &&
        2 * SkinnyCfg<Policy, TH, NW, WAVES, true>::kStageBytes + NW * scale_block_stride((int)K) <=
            kSkinnyLdsBudget)
      return launch_skinny<Policy, Epilogue, TH, NW, WAVES, true>(who, pargs, x, y, epi, M, N, K, want_stages,
                                                                  stream);
  }
  using Cfg = SkinnyCfg<Policy, TH, NW, WAVES, SB>;
  auto kern = skinny_gemm_kernel<Policy, Epilogue, TH, NW, WAVES, SB>;
  const int64_t blocks = (N + 16 * NW - 1) / (16 * NW);
  int stages = want_stages;
  if (stages > Cfg::kMaxAhead + 1) stages = Cfg::kMaxAhead + 1;
  if (stages > 9) stages = 9;
  const int sblock_bytes = SB ? NW * scale_block_stride((int)K) : 0;  // after the ring
  if (stages * Cfg::kStageBytes + sblock_bytes > kSkinnyLdsBudget)
    stages = (kSkinnyLdsBudget - sblock_bytes) / Cfg::kStageBytes;
  WQ_REQUIRE(stages >= 2, "%s: internal: no room for a 2-slot ring", who);
  int lds_bytes = stages * Cfg::kStageBytes + sblock_bytes;
  if (lds_bytes < Cfg::kRedBytes) lds_bytes = Cfg::kRedBytes;
  static DynamicLdsLimit limit;  // per instantiation
  WQ_HIP(limit.ensure(reinterpret_cast<const void*>(kern), 160 * 1024));
  WQ_LAUNCH(who, kern, dim3((unsigned)blocks), dim3(64 * WAVES), lds_bytes, stream, pargs,
            (const half_t*)x, (half_t*)y, epi, (int)M, (int)N, (int)K, stages);
  return WQ_OK;
}

// Picks the arrangement from the shape (timings of the Llama-7B layer shapes): few
// columns per workgroup while the matrix is small, so that every CU gets work; more
// columns per workgroup for tall matrices and larger M, where the re-reads of the
// activations (once per workgroup) would otherwise outweigh the weight stream.
template <typename Policy, typename Epilogue>
static int launch_skinny_auto(const char* who, const typename Policy::Args& pargs, const uint16_t* x,
                              uint16_t* y, const Epilogue& epi, int64_t M, int64_t N, int64_t K,
                              hipStream_t stream) {
  const SkinnyTuning t = skinny_tuning();
  // activations in registers where that kernel is the faster one: 4096 < K <= 8192 and at least
  // four column tiles per CU (N = 28672, K = 8192: q4f16_1 at M = 16 58 -> 47 us, int8 at M = 4
  // 60 -> 48 us; with two tiles per CU, or at K = 4096, the ring kernel is the faster one)
  if (xreg_fits(M, K) && Policy::pair_aligned(pargs) && (t.waves == 2 || (t.waves == 0 && K > 4096 && N / 16 >= 4 * (int64_t)cu_count())))
    return launch_xreg_auto<Policy, Epilogue>(who, pargs, x, y, epi, M, N, K, stream);
  const int64_t per_cu = (N / 16) / cu_count();
  int nw = 1;
  if (per_cu >= 2) nw = M <= 8 ? (per_cu >= 4 ? 2 : 1) : M <= 16 ? 2 : 4;
  // wide matrices and more than 16 rows: all eight wavefronts side by side (128 columns per
  // workgroup, each wavefront the whole K), which halves the re-reads of x again, as long as
  // most CUs still get a workgroup (int8, K = 8192, N = 28672, M = 64: 80 -> 62 us)
  if (M > 16 && N / 128 >= (cu_count() * 5) / 8) nw = 8;
  // ... corrected for how the workgroups fill the machine.  A workgroup of nw wavefronts takes nw column tiles
  // and stages the activations once, which costs about as much as one tile (two from 33 rows on): the launch
  // lasts about (rounds of the CUs) x (nw + that).  Fewer wavefronts side by side where that is shorter
  // (N = 8192 with 4: 128 workgroups on 256 CUs; K = 28672, M = 32: 102 -> 62 us), two instead of one where
  // one leaves a second, partly filled round (N = 5120, K = 13824, M = 32: 43 -> 31 us; N = 6144, K = 4096,
  // M = 64: 22 -> 14 us).  Up to 8 rows the choice above stands (measured either way).
  if (M > 8 && !t.nw) {
    const int64_t tiles = (N + 15) / 16, cus = cu_count();
    const double cx = M > 32 ? 2.0 : 1.0;
    auto cost = [&](int w) { return (double)((tiles + w * cus - 1) / (w * cus)) * (w + cx); };
    while (nw > 1 && cost(nw / 2) < cost(nw) - 1e-9) nw /= 2;
    if (nw == 1 && cost(2) < cost(1) - 1e-9) nw = 2;
  }
  if (t.nw) nw = t.nw;
  if (M <= 8 && nw >= 4) nw = 2;  // 8 rows are two slab loads: at most two wavefronts share them
  // three ring slots for four or more wavefronts side by side, and for two when every workgroup has a CU of
  // its own anyway (N = 8192, K = 28672, M = 16: 67 -> 46 us; with more workgroups than CUs the third slot
  // costs a resident workgroup: N = 10240, K = 8192, M = 16: 20.9 -> 27.4 us)
  const int64_t wgs = ((N + 15) / 16 + nw - 1) / nw;
  const int stages = t.stages ? t.stages : (nw >= 4 || (nw == 2 && M > 8 && wgs <= cu_count()) ? 3 : 2);
  // eight wavefronts where two ring slots of that arrangement fit LDS, else four
#define WQ_SK_GO(TH, NW, WAVES)                                                                        \
  do {                                                                                                 \
    if constexpr (2 * SkinnyCfg<Policy, TH, NW, WAVES>::kStageBytes <= kSkinnyLdsBudget)               \
      return launch_skinny<Policy, Epilogue, TH, NW, WAVES>(who, pargs, x, y, epi, M, N, K, stages,    \
                                                            stream);                                   \
    else                                                                                               \
      return launch_skinny<Policy, Epilogue, TH, NW, 4>(who, pargs, x, y, epi, M, N, K, stages,        \
                                                        stream);                                       \
  } while (0)
  if (M <= 8) {
    if (nw == 2) WQ_SK_GO(1, 2, 8);
    WQ_SK_GO(1, 1, 8);
  }
  if (M <= 16 && nw != 8) {
    if (nw == 4) WQ_SK_GO(2, 4, 8);
    if (nw == 2) WQ_SK_GO(2, 2, 8);
    WQ_SK_GO(2, 1, 8);
  }
  if (M <= 32) {
    if (nw == 8) WQ_SK_GO(4, 8, 8);
    if (nw == 4) WQ_SK_GO(4, 4, 8);
    if (nw == 2) WQ_SK_GO(4, 2, 8);
    WQ_SK_GO(4, 1, 8);
  }
  if (nw == 8) WQ_SK_GO(8, 8, 8);
  if (nw == 4) WQ_SK_GO(8, 4, 8);
  if (nw == 2) WQ_SK_GO(8, 2, 8);
  WQ_SK_GO(8, 1, 8);
#undef WQ_SK_GO
}

}  // namespace wq
#endif  // RELAX_AMD_CSRC_SKINNY_GEMM_H_
