// Prefill GEMM, fully LDS-staged variant for the gfx950 matrix cores, both weight formats:
//   y[m,n] = epilogue( sum_k x[m,k] * dequant(w)[n,k] )
//
// Every operand of a K-step (64 k) travels global -> LDS with the direct
// global_load_lds_dwordx4 path: no staging registers, no VALU work, and the loads
// of the next two or more steps are in flight while a step is multiplied (a ring of 3 slots, or of up to 6
// where one workgroup per CU leaves room in LDS; what pays is a 4-slot ring under 256 x 128 tiles).  Per slot:
//   A   BM rows x 128 B of activations, 16-byte chunk c of row r at slot position
//       c ^ ((r >> 1) & 7) (the swizzle is applied to the GLOBAL address each lane fetches,
//       because the LDS side of a direct load is fixed: lane l writes 16 bytes at
//       base + 16*l);
//   B   BN columns x 32 or 64 B of packed codes, still packed, in the order the weight
//       format's policy fetches them;
//   S   (format A only) BN x 4 B: the two scales of the step.
// A wavefront then reads, per K-step, TM*4 activation fragments, and per weight
// sub-tile its 32 codes (16 or 32 bytes) plus one scale: MFMA lane (j, h) needs 8
// K-values of column j per MFMA, so the weights are dequantized in registers by the
// policy's bit-exact pair function (natural K order, hence no rearrangement of the
// activations) and never exist in LDS as fp16.
//
// Synchronisation: vector memory operations retire in order, so s_waitcnt vmcnt(loads of
// one step) means "this wavefront's loads of the step before have landed"; one raw
// s_barrier per K-step then says the same for the whole workgroup (the fence in
// __syncthreads would force vmcnt(0)).  The schedule inside a K-step is described at
// gemm_lds_tile.
//
// A weight policy provides
//   kColBytes            packed bytes per column and K-step (32 or 64)
//   kScaleBytes          bytes of scales per column and K-step staged in LDS (4 or 0)
//   Args, Frag, Scale    kernel arguments; a lane's packed codes of one column for one step; what
//                        pair() needs besides the codes (the scale in both halves of a register,
//                        plus the zero point where the format has one)
//   b_src(args, n0, q, N, K)   global address (step 0) of 16-byte chunk q of the B tile at column n0
//   kStepStride          bytes between consecutive K-steps of a chunk
//   s_src(args, n, K)    global address (step 0) of the 4 scale bytes of column n       (kScaleBytes > 0)
//   s_offset(args, ks)   byte offset of step ks from there                              (kScaleBytes > 0)
//   read_scale(p, lh)    Scale from the 4 staged bytes of a column, for lane half lh    (kScaleBytes > 0)
//   const_scale(args, n) the Scale of column n                                          (kScaleBytes == 0)
//   read(frag, bslot, n_local, lh)   LDS -> registers
//   pair(frag, kk, j, scale)   dequantized weights (k = 8kk + 2j, 8kk + 2j + 1) of the lane's column,
//                              = pair_finish(pair_bits(frag, kk, j), scale): the two exact fp16 integers
//                              as a bit pattern, then (integer - offset) * scale.  The K loop runs the two
//                              halves in different MFMA slots: a chain of four dependent VALU operations
//                              does not fit behind one MFMA, two do.
// and, only where the scale of a weight depends on its k inside the step (scales along N):
//   phase_begin(scale, kk)     called once per column sub-tile in front of the phase that unpacks the weights
//                              of MFMA kk: fetches what pair_finish_at needs for them
//   pair_finish_at(bits, scale, j)   pair_finish for pair j of that MFMA
#ifndef RELAX_AMD_CSRC_MFMA_GEMM_LDS_H_
#define RELAX_AMD_CSRC_MFMA_GEMM_LDS_H_

#include <algorithm>
#include <cmath>
#include <type_traits>

#include "gemm_epilogue.h"
#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

template <class Policy, int TM, int TN, int WM, int WN, int WPE>
struct LdsGemmCfg {
  static_assert(WM * WN == 4, "four wavefronts per workgroup");
  static constexpr int kThreads = 256;
  static constexpr int BM = 32 * TM * WM;
  static constexpr int BN = 32 * TN * WN;
  static constexpr int kAOff = 0;
  static constexpr int kBOff = BM * 128;
  static constexpr int kSOff = kBOff + BN * Policy::kColBytes;
  static constexpr int kStageBytes = kSOff + BN * Policy::kScaleBytes;
  // ring slots: loads of kStages - 1 steps are in flight while a step is multiplied; four where a
  // single workgroup per CU leaves room for them in the 160 KiB of LDS
  static constexpr int kFit = (158 * 1024) / kStageBytes;
  static constexpr int kStages = WPE == 1 ? (kFit >= 6 ? 6 : kFit >= 4 ? kFit : 3) : 3;
  static constexpr int kLdsBytes = kStages * kStageBytes;
  static constexpr int kALoads = BM / 32;   // direct loads per wavefront per step (64 chunks each)
  static constexpr int kBLoads = BN * Policy::kColBytes / 4096;
  static_assert(BN % 128 == 0 && BN <= 256, "B tile: 128 or 256 columns");
  static constexpr int kSLoads = Policy::kScaleBytes ? 1 : 0;
  static constexpr int kLoadsPerStage = kALoads + kBLoads + kSLoads;
};

// XOR pattern of the activation tile: consecutive rows alternate between the two
// 128-byte halves of the bank space, so pairs of rows share one pattern value.
#define WQ_SWZ(r) (((r) >> 1) & 7)
#define WQ_WAITCNT_VM(n) __builtin_amdgcn_s_waitcnt(((n)&0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))
// the same with lgkmcnt(0): this wavefront's LDS reads have returned as well
#define WQ_WAITCNT_VM_LGKM0(n) __builtin_amdgcn_s_waitcnt(((n)&0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0x0 << 8))

template <class P, class = void>
struct ScalePerK : std::false_type {};
template <class P>
struct ScalePerK<P, std::void_t<decltype(&P::phase_begin)>> : std::true_type {};

typedef const void __attribute__((address_space(1))) * wq_gptr_t;
typedef void __attribute__((address_space(3))) * wq_lptr_t;

// One output tile of TME*32*WM rows x BN columns starting at (m0, n0).  TME is the
// number of 32-row sub-tiles per wavefront that are actually computed: TM for a full
// tile, TM/2 or TM/4 for the split tiles of the last, partially filled round.
//
// Schedule of one K-step (four phases kk = 0..3 of TME*TN MFMAs each).  Nothing but
// MFMAs may sit on the critical path of a wavefront that has its SIMD to itself, so
// every other instruction is slotted between them:
//   phases 0-2  per MFMA slot one LDS read of an activation fragment of phase kk+1 (the first
//               TME slots) and one half of the unpacking of a weight pair of phase kk+1 (bit
//               pattern in an early slot, arithmetic in a later one); in phase 0 also all direct
//               loads of step ks+2, one every few slots (the texture path accepts 64 B per cycle
//               and CU: issued in a burst they block the wavefront for hundreds of cycles);
//   phase 3     first s_waitcnt vmcnt (this wavefront's loads of step ks+1 have landed)
//               and s_barrier (everyone's have); then, between its MFMAs, the packed
//               weights, the first activation fragments and the first weight pairs of
//               step ks+1, so that step ks+1 starts multiplying at once.
// One barrier per K-step suffices (three slots shown): slot (ks+2)%3 = (ks-1)%3 is refilled by loads issued after
// the barrier of step ks-1, and every wavefront has waited for its last LDS reads of that slot
// (the phase-3 fragments of step ks-1) before that barrier.
template <class Policy, class Epilogue, int TM, int TN, int WM, int WN, int WPE, int TME>
__device__ __forceinline__ void gemm_lds_tile(const typename Policy::Args& wargs,
                                              const half_t* __restrict__ X, half_t* __restrict__ Y,
                                              const Epilogue& epilogue, int M, int N, int K, int m0,
                                              int n0, unsigned char* lds) {
  using Cfg = LdsGemmCfg<Policy, TM, TN, WM, WN, WPE>;
  constexpr int kALoadsE = Cfg::kALoads * TME / TM;  // direct A loads per wavefront per step
  constexpr int L = kALoadsE + Cfg::kBLoads + Cfg::kSLoads;  // direct loads per wavefront per step
  constexpr int NSLOT = TME * TN;                    // MFMAs per phase
  constexpr int NPAIR = TN * 4;                      // weight pairs to unpack per phase
  static_assert(kALoadsE >= 1, "tile too small to split further");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int lj = lane & 31, lh = lane >> 5;
  const int ksteps = K >> 6;

  // ---- global sources of this lane's direct loads (rows past M / N are clamped:
  //      they only feed accumulators that are never stored) ----
  const char* a_src[kALoadsE];
#pragma unroll
  for (int i = 0; i < kALoadsE; ++i) {
    const int s = (wave * kALoadsE + i) * 64 + lane;  // LDS chunk slot
    const int r = s >> 3, c = (s & 7) ^ WQ_SWZ(r);
    a_src[i] = reinterpret_cast<const char*>(X + (int64_t)min(m0 + r, M - 1) * K) + c * 16;
  }
  const char* b_src[Cfg::kBLoads];
#pragma unroll
  for (int i = 0; i < Cfg::kBLoads; ++i)
    b_src[i] = Policy::b_src(wargs, n0, (wave * Cfg::kBLoads + i) * 64 + lane, N, K);
  // scales staged per step (format A): 64 columns per wavefront (with BN = 128 wavefronts 2
  // and 3 repeat the loads of wavefronts 0 and 1)
  const char* s_src = nullptr;
  if (Cfg::kSLoads) s_src = Policy::s_src(wargs, min(n0 + (wave * 64) % Cfg::BN + lane, N - 1), K);

  // direct load number idx (0 .. L-1) of step ks
  auto issue_one = [&](int ks, int idx) {
    unsigned char* slot = lds + (ks % Cfg::kStages) * Cfg::kStageBytes;
    if (idx < kALoadsE) {
      __builtin_amdgcn_global_load_lds((wq_gptr_t)(a_src[idx] + (int64_t)ks * 128),
                                       (wq_lptr_t)(slot + Cfg::kAOff + (wave * kALoadsE + idx) * 1024), 16, 0, 0);
    } else if (idx < kALoadsE + Cfg::kBLoads) {
      const int i = idx - kALoadsE;
      __builtin_amdgcn_global_load_lds((wq_gptr_t)(b_src[i] + (int64_t)ks * Policy::kStepStride),
                                       (wq_lptr_t)(slot + Cfg::kBOff + (wave * Cfg::kBLoads + i) * 1024), 16, 0, 0);
    } else {
      __builtin_amdgcn_global_load_lds((wq_gptr_t)(s_src + Policy::s_offset(wargs, ks)),
                                       (wq_lptr_t)(slot + Cfg::kSOff + (wave * 64 % Cfg::BN) * 4), 4, 0, 0);
    }
  };

  float16_t acc[TME][TN];
#pragma unroll
  for (int i = 0; i < TME; ++i)
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.0f;

  typename Policy::Frag bw[TN];   // this lane's packed weights (and scale) of the step being unpacked
  typename Policy::Scale bs[TN];
  if (!Cfg::kSLoads) {
#pragma unroll
    for (int t = 0; t < TN; ++t) bs[t] = Policy::const_scale(wargs, min(n0 + (wn * TN + t) * 32 + lj, N - 1));
  }
  half8_t aop[2][TME], bop[2][TN];
  auto read_b = [&](const unsigned char* slot) {
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      const int n = (wn * TN + t) * 32 + lj;
      Policy::read(bw[t], slot + Cfg::kBOff, n, lh);
      if (Cfg::kSLoads) bs[t] = Policy::read_scale(slot + Cfg::kSOff + n * 4, lh);
    }
  };
  auto read_a = [&](const unsigned char* slot, int kk, half8_t (&dst)[TME]) {
#pragma unroll
    for (int i = 0; i < TME; ++i) {
      const int row = (wm * TME + i) * 32 + lj;
      dst[i] = *reinterpret_cast<const half8_t*>(slot + Cfg::kAOff + row * 128 +
                                                 (((4 * lh + kk) ^ WQ_SWZ(row)) << 4));
    }
  };

  // ---- prologue: steps 0 .. kStages - 2 in flight, operands of step 0 ready ----
  constexpr int AHEAD = Cfg::kStages - 1;  // steps of loads in flight while a step is multiplied
#pragma unroll
  for (int st = 0; st < AHEAD; ++st) {
    if (st < ksteps) {
#pragma unroll
      for (int idx = 0; idx < L; ++idx) issue_one(st, idx);
    }
  }
  // loads retire in order: step 0 has landed once at most the loads of the later steps are outstanding
  static_assert(AHEAD * L <= 63, "vmcnt holds 6 bits");
  const int first_later = min(AHEAD, ksteps) - 1;
  if (first_later >= 5) {
    WQ_WAITCNT_VM(5 * L);
  } else if (first_later == 4) {
    WQ_WAITCNT_VM(4 * L);
  } else if (first_later == 3) {
    WQ_WAITCNT_VM(3 * L);
  } else if (first_later == 2) {
    WQ_WAITCNT_VM(2 * L);
  } else if (ksteps >= 2) {
    WQ_WAITCNT_VM(L);
  } else {
    WQ_WAITCNT_VM(0);
  }
  __builtin_amdgcn_s_barrier();
  read_b(lds);
  read_a(lds, 0, aop[0]);
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    half2_t d[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = Policy::pair(bw[t], 0, j, bs[t]);
    bop[0][t] = half8_t{d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
  }

  // Phase 3 prepares the next step unconditionally: in the last step it reads a slot that
  // holds stale data and unpacks it for nobody.  (A run-time branch around those LDS reads
  // would make the compiler wait for them before the first MFMA of the phase.)
  for (int ks = 0; ks < ksteps; ++ks) {
    const unsigned char* slot = lds + (ks % Cfg::kStages) * Cfg::kStageBytes;
    const unsigned char* next_slot = lds + ((ks + 1) % Cfg::kStages) * Cfg::kStageBytes;
    const bool ahead2 = ks + AHEAD < ksteps;  // there is a step to request in this one
    const int later = min(AHEAD - 1, ksteps - 2 - ks);  // steps requested beyond ks + 1 when phase 3 waits
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int cur = kk & 1, nxt = cur ^ 1;
      const unsigned char* const a_from = kk == 3 ? next_slot : slot;  // activation fragments of the next phase
      const int a_kk = kk == 3 ? 0 : kk + 1;
      if (kk == 3) {
        // loads of step ks+1 landed (those of ks+2 may be in flight), own LDS reads done
        if (later >= 4) {
          WQ_WAITCNT_VM_LGKM0(4 * L);
        } else if (later == 3) {
          WQ_WAITCNT_VM_LGKM0(3 * L);
        } else if (later == 2) {
          WQ_WAITCNT_VM_LGKM0(2 * L);
        } else if (later == 1) {
          WQ_WAITCNT_VM_LGKM0(L);
        } else {
          WQ_WAITCNT_VM_LGKM0(0);
        }
        __builtin_amdgcn_s_barrier();
        read_b(next_slot);
      }
      half2_t dq[TN][4];
      uint32_t pb[NPAIR];
      // Slots of the unpacking: the bit patterns in the first half of the usable slots, the
      // arithmetic in the second half; in phase 3 the packed weights were requested from LDS
      // just above, so the first slots stay free.
      const int first = kk < 3 ? 0 : NSLOT * 3 / 8, usable = NSLOT - first, half = usable / 2;
      if constexpr (ScalePerK<Policy>::value) {
#pragma unroll
        for (int t = 0; t < TN; ++t) Policy::phase_begin(bs[t], (kk + 1) & 3);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int sl = 0; sl < NSLOT; ++sl) {
        const int i = sl / TN, t = sl % TN;
        acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[cur][i], bop[cur][t], acc[i][t], 0, 0, 0);
        // one activation fragment of the next phase per slot
        if (sl < TME) {
          const int row = (wm * TME + sl) * 32 + lj;
          aop[nxt][sl] = *reinterpret_cast<const half8_t*>(a_from + Cfg::kAOff + row * 128 +
                                                           (((4 * lh + a_kk) ^ WQ_SWZ(row)) << 4));
        }
#pragma unroll
        for (int p = 0; p < NPAIR; ++p) {
          const int tt = p >> 2, j = p & 3;
          if (sl == first + p * half / NPAIR) pb[p] = Policy::pair_bits(bw[tt], (kk + 1) & 3, j);
          if (sl == first + half + p * (usable - half) / NPAIR) {
            if constexpr (ScalePerK<Policy>::value) dq[tt][j] = Policy::pair_finish_at(pb[p], bs[tt], j);
            else dq[tt][j] = Policy::pair_finish(pb[p], bs[tt]);
          }
        }
        // direct loads of step ks+AHEAD, all in phase 0 (into the slot of step ks-1, free since the
        // barrier of its phase 3): timed on the GPU, one phase with loads and three without beat
        // the same loads spread over two phases (by 1-2 %) or over all four (by 15 %)
        if (kk == 0 && ahead2) {
          const int l0 = sl * L / NSLOT, l1 = (sl + 1) * L / NSLOT;
#pragma unroll
          for (int idx = l0; idx < l1; ++idx) issue_one(ks + AHEAD, idx);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int t = 0; t < TN; ++t)
        bop[nxt][t] = half8_t{dq[t][0].x, dq[t][0].y, dq[t][1].x, dq[t][1].y,
                              dq[t][2].x, dq[t][2].y, dq[t][3].x, dq[t][3].y};
    }
  }

  // ---- epilogue ----
  // Row-wise through LDS (gemm_epilogue.h); the ring is idle now: every real read of it was
  // waited for before the last barrier, and each wavefront stages in a piece of its own.
  if (epilogue.wide_ok(N, Y)) {
    using ECfg = RowwiseEpilogueCfg<TME, TN>;
    static_assert(4 * ECfg::kBytesPerWave <= Cfg::kLdsBytes, "epilogue staging exceeds the ring");
    store_tile_rowwise<Epilogue, TME, TN>(acc, epilogue, Y, M, N, m0 + wm * TME * 32, n0 + wn * TN * 32,
                                          lds + wave * ECfg::kBytesPerWave, lane);
    return;
  }
  // element-wise: accumulator register r of lane (j, h) is element (row 8*(r/4) + 4*h + r%4, col j)
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int n = n0 + (wn * TN + t) * 32 + lj;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < TME; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + (wm * TME + i) * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (m < M) Y[(int64_t)m * N + n] = epilogue(acc[i][t][r], m, n);
      }
    }
  }
}

// Row slices (1, 2 or 4; 8 where the policy carries the extra copy of the tile body, `fine`) that the tiles of
// the last, partially filled round are cut into: as many as still run all at once.  (Every slice unpacks all
// columns of its tile, so slices get less efficient as they get lower: eight only pay on 32 tiles or fewer:
// M = 256, N = 4096, K = 11008 format A 73.6 -> 68.6 us.)  A rest that already has a CU per tile is only cut if every slice gets a
// CU of its own: two slices sharing a CU take as long as the whole tile, and read its weights twice.
inline int lds_tail_split(int rest, int slots, int cus, int TM, int a_loads, bool fine = false) {
  const int room = rest <= cus ? cus : slots;
  if (fine && TM % 8 == 0 && a_loads % 8 == 0 && rest * 8 <= room) return 8;
  for (int sp : {4, 2})
    if (TM % sp == 0 && a_loads % sp == 0 && rest * sp <= room) return sp;
  return 1;
}

// Relative duration of the LDS-staged GEMM on an M x N problem under tile configuration 11 (256 x 256
// tiles), 17 (128 x 128, two workgroups per CU) or 18 (256 x 128): rounds of the machine times tile
// area over the rate one CU sustains on such tiles.  The rates are tile areas per microsecond measured
// at K = 8192, N = 28672 with int8 weights (128 x 128 alone on its CU 193, two per CU 243 together;
// 256 x 128: 254; 256 x 256: 294); row slices of a cut tile run at 0.74 (halves) and 0.56 (quarters) of
// them (a slice unpacks all columns of its tile whatever its height; fitted to launches that are one cut round:
// N = 4096 .. 12288, M = 192 .. 1024, where 0.85 / 0.75 chose 256 x 256 tiles 10 .. 15 % too slow).  The model reproduces the measured times at M = 65 .. 2048 within 6 %.
inline double lds_cfg_cost(int cfg, int64_t M, int64_t N, int cus) {
  const int BM = cfg == 17 ? 128 : 256, BN = cfg == 11 ? 256 : 128, per_cu = cfg == 17 ? 2 : 1;
  const double rate_alone = cfg == 17 ? 193.0 : cfg == 18 ? 254.0 : 294.0;
  const double rate_full = cfg == 17 ? 243.0 : rate_alone;  // per CU, every slot taken
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const int slots = cus * per_cu;
  const int rest = (int)(tiles % slots);
  const double area = (double)BM * BN;
  double t = (double)(tiles / slots) * per_cu * area / rate_full;
  if (rest) {
    const int split = lds_tail_split(rest, slots, cus, BM / 32, BM / 32);
    const bool alone = rest * split <= cus;
    const double slice = split == 4 ? 0.56 : split == 2 ? 0.74 : 1.0;
    t += area / split * (alone ? 1 : per_cu) / ((alone ? rate_alone : rate_full) * slice);
  }
  return t;
}

// Policy::kFineTail = true: the kernels of that policy also hold the tile body for slices of TM / 8 sub-tiles.
template <class P, class = void>
struct FineTail : std::false_type {};
template <class P>
struct FineTail<P, std::void_t<decltype(P::kFineTail)>> : std::bool_constant<P::kFineTail> {};

// Workgroup -> work item.  The first n_full workgroups compute whole tiles (as many
// as fill complete rounds of the machine); the tiles of the last, partially filled
// round are cut into `split` row slices of TM/split sub-tiles so that the round is
// shorter instead of leaving most CUs idle while a few finish whole tiles.
template <class Policy, class Epilogue, int TM, int TN, int WM, int WN, int WAVES_PER_EU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WAVES_PER_EU, WAVES_PER_EU)))
void gemm_lds_kernel(typename Policy::Args wargs, const half_t* __restrict__ X, half_t* __restrict__ Y,
                     Epilogue epilogue, int M, int N, int K, int tiles_m, int tiles_n, int n_full,
                     int split, int group_m) {
  using Cfg = LdsGemmCfg<Policy, TM, TN, WM, WN, WAVES_PER_EU>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  // Tiles are numbered in bands of group_m rows of tiles, N-fastest inside a band and M-fastest inside a column of
  // the band, and workgroups go to the XCDs round-robin: XCD x (own L2) takes a contiguous range of that order,
  // so the tiles it runs at one time are group_m tiles high and share their activation rows and weight columns
  // through its L2.  The same for the slices of the last, partial round.
  auto tile_of = [&](int t, int& tile_m, int& tile_n) {
    const int width = group_m * tiles_n, band = t / width, in_band = t - band * width;
    const int first_m = band * group_m, rows = min(group_m, tiles_m - first_m);
    tile_m = first_m + in_band % rows;
    tile_n = in_band / rows;
  };
  int pid = blockIdx.x;
  if (pid < n_full) {
    const int per = n_full / 8, rem = n_full % 8;
    const int xcd = pid & 7, idx = pid >> 3;
    int tile_m, tile_n;
    tile_of(xcd * per + min(xcd, rem) + idx, tile_m, tile_n);
    gemm_lds_tile<Policy, Epilogue, TM, TN, WM, WN, WAVES_PER_EU, TM>(wargs, X, Y, epilogue, M, N, K,
                                                        tile_m * Cfg::BM, tile_n * Cfg::BN, lds);
    return;
  }
  int q = pid - n_full;
  if (n_full > 0) {  // (a launch of one partial round keeps the plain order: measured 2-3 % faster there)
    const int slices = ((int)gridDim.x - n_full), per = slices / 8, rem = slices % 8;
    const int xcd = q & 7, idx = q >> 3;  // n_full is a multiple of the CU count: the XCD of this workgroup is q mod 8
    q = xcd * per + min(xcd, rem) + idx;
  }
  const int part = q % split;
  int tile_m, tile_n;
  tile_of(n_full + q / split, tile_m, tile_n);
  const int m0 = tile_m * Cfg::BM + part * (Cfg::BM / split), n0 = tile_n * Cfg::BN;
  if (m0 >= M) return;  // a slice that lies entirely past the last row
  if (split == 2) {
    if constexpr (TM % 2 == 0)
      gemm_lds_tile<Policy, Epilogue, TM, TN, WM, WN, WAVES_PER_EU, TM / 2>(wargs, X, Y, epilogue, M, N, K, m0, n0, lds);
  } else if (split == 4) {
    if constexpr (TM % 4 == 0)
      gemm_lds_tile<Policy, Epilogue, TM, TN, WM, WN, WAVES_PER_EU, TM / 4>(wargs, X, Y, epilogue, M, N, K, m0, n0, lds);
  } else if (split == 8) {
    if constexpr (TM % 8 == 0 && FineTail<Policy>::value)
      gemm_lds_tile<Policy, Epilogue, TM, TN, WM, WN, WAVES_PER_EU, TM / 8>(wargs, X, Y, epilogue, M, N, K, m0, n0, lds);
  } else {
    gemm_lds_tile<Policy, Epilogue, TM, TN, WM, WN, WAVES_PER_EU, TM>(wargs, X, Y, epilogue, M, N, K, m0, n0, lds);
  }
}

template <class Policy, class Epilogue, int TM, int TN, int WM, int WN, int WPE>
static int launch_gemm_lds(const char* who, const typename Policy::Args& wargs, const uint16_t* x,
                           uint16_t* y, const Epilogue& ep, int64_t M, int64_t N, int64_t K,
                           hipStream_t stream) {
  using Cfg = LdsGemmCfg<Policy, TM, TN, WM, WN, WPE>;
  const int tiles_m = (int)((M + Cfg::BM - 1) / Cfg::BM);
  const int tiles_n = (int)((N + Cfg::BN - 1) / Cfg::BN);
  auto kern = gemm_lds_kernel<Policy, Epilogue, TM, TN, WM, WN, WPE>;
  static DynamicLdsLimit limit;
  WQ_HIP(limit.ensure(reinterpret_cast<const void*>(kern), Cfg::kLdsBytes));
  // Whole rounds of the machine run whole tiles; the tiles of the last, partial
  // round are cut into 2 or 4 row slices when that lets them all run at once.
  const int per_cu = std::max(1, std::min(WPE, (160 * 1024) / Cfg::kLdsBytes));
  const int slots = cu_count() * per_cu;
  const int total = tiles_m * tiles_n;
  const int n_full = (total / slots) * slots;
  const int rest = total - n_full;
  const int split = tuning().gemm_tail_split ? lds_tail_split(rest, slots, cu_count(), TM, Cfg::kALoads, FineTail<Policy>::value) : 1;
  // height of the block of tiles an XCD runs at one time: the activation rows of a tile against its weight
  // columns, in bytes per step of K, decide how a block of slots / 8 tiles is best shaped
  const double ratio = (double)(Cfg::BN * Policy::kColBytes) / (double)(Cfg::BM * 128);
  const double want = std::sqrt((double)(slots / 8) * ratio);
  int group_m = 1;
  while (group_m * 1.5 < want) group_m *= 2;
  group_m = std::max(1, std::min(group_m, tiles_m));
  if (n_full == 0) group_m = tiles_m;  // one partial round: M-fastest, workgroup i takes slice i
  WQ_LAUNCH(who, kern, dim3((unsigned)(n_full + rest * split)), dim3(256), Cfg::kLdsBytes, stream, wargs,
            (const half_t*)x, (half_t*)y, ep, (int)M, (int)N, (int)K, tiles_m, tiles_n, n_full, split, group_m);
  return WQ_OK;
}

}  // namespace wq
#endif  // RELAX_AMD_CSRC_MFMA_GEMM_LDS_H_
