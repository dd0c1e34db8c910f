// Decode GEMV over [N, K/8] int4 weights: y[m,n] = sum_k x[m,k] * ((code[n,k] - 7) * S[n,k/32])
// (format A), or with a zero point per group, (code - zp) * s (template parameter ZP).
//
// The kernel is a weight stream bounded by HBM bandwidth, so the design goal is
// to keep many 16-byte loads in flight per CU, to put nothing (no LDS staging, no
// barrier) between the start of a workgroup and its first weight loads, and to
// spend as few VALU instructions per weight word as possible.
//
// Work split.  A row set is ROWS consecutive output rows and belongs to one
// wavefront (or to `parts` wavefronts when K > 64*32*GPL); lane l of wavefront
// `part` owns the scale groups g = (j*parts + part)*64 + l, j < GPL, of every row
// of the set: 16 bytes of W (4 words = 32 codes) and one scale per group, so a
// wavefront-wide load is 1 KiB of contiguous weights (128 bytes of scales).
// All ROWS*GPL weight loads of a lane are independent and issued back to back.
//
// Activations.  The workgroup (4 wavefronts, 4 row sets) first issues one pass of
// coalesced loads over x, THEN its weight loads: vector loads complete in issue
// order, so x can be processed while the weights are still in flight.  Each
// thread rearranges its 8 activations to the pairing of the unpack, folds the
// zero point into the group constant c_g (below) and writes the result to LDS;
// after one barrier every lane copies the activations of its own groups into
// registers, where they stay for all rows.  x is therefore read from L2 once per
// workgroup instead of once per wavefront, and its rearrangement costs a dozen
// VALU instructions per thread.
//
// Reduction.  DPP row shifts inside a wavefront (total in lane 63); only when
// parts > 1 do partial sums cross wavefronts, through a few LDS words.
//
// Arithmetic.  With t = 1024 + code (the fp16 number obtained by OR-ing the code
// into the mantissa of 0x6400) the group's contribution is
//     s * ( sum_k x_k * t_k  -  c_g ),    c_g = sum_k x_k * 1031
// so the subtraction of the zero point and the multiplication by the scale are
// done once per group instead of once per weight; c_g depends only on x.  Codes
// in odd nibble positions are taken without a shift as 1024 + 16*code and meet
// activations pre-multiplied by 1/16; their share of c_g uses 64 + 7 = 71 instead
// of 1031.  Products are exact in fp32 (v_dot2_f32_f16), accumulation is fp32.
// The result differs from the reference's "round each weight to fp16 first" only
// by those roundings, far inside the 1e-2 tolerance; a one-hot x still reproduces
// a dequantized column bit for bit.  The bit-exact dequantization itself is
// q4_word_dequant, used by the dequantize entry point and by the MFMA GEMM.
#pragma once
#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

constexpr int kGemvMaxWaves = 16;

// Few groups per lane means more wavefronts share a row: allow larger workgroups there.
template <int GPL>
constexpr int gemv_max_threads() {
  return GPL == 1 ? 1024 : GPL == 2 ? 512 : 256;
}

// What the zero-point variant adds to the launch: S holds (scale, zero point) fp16 pairs
// [N, groups], one per `ratio` consecutive 32-code groups.
struct GemvZp {
  int ratio;   // 32-code groups per scale group
  int groups;  // scale groups per row
};

template <int ROWS, int GPL>
struct GemvFrag {
  uint4_t w[ROWS][GPL];
  half2_t s[ROWS][GPL];  // .x scale; .y zero point (ZP only)
};

template <int ROWS, int MB, int GPL, bool ZP>
__global__ __launch_bounds__(gemv_max_threads<GPL>()) void q4g32_gemv_kernel(
    const uint4_t* __restrict__ W, const half_t* __restrict__ S, const half_t* __restrict__ x,
    const half_t* __restrict__ bias, const half_t* __restrict__ residual, half_t* __restrict__ y,
    int N, int K, int parts, int nsets, GemvZp zp) {
  extern __shared__ uint4_t smem[];
  __shared__ float red[2][kGemvMaxWaves][ROWS * MB];
  const int G = K >> 5;
  uint4_t* xs = smem;                                       // [MB][4][G] rearranged chunks
  float* cs = reinterpret_cast<float*>(smem + MB * 4 * G);  // [MB][G]    -c_g  (ZP: then [MB][G] -sum x)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nthreads = blockDim.x;
  const int sets_per_block = (nthreads >> 6) / parts;
  const int part = wave % parts;
  const int set_in_block = wave / parts;
  const int stride = gridDim.x * sets_per_block;  // row sets between two turns of this workgroup
  int base = blockIdx.x * sets_per_block;         // first row set of the workgroup's current turn

  int g[GPL];
  int sg[GPL];  // index of the group's scale within its row
  bool active[GPL];
#pragma unroll
  for (int j = 0; j < GPL; ++j) {
    const int gj = (j * parts + part) * 64 + lane;
    active[j] = gj < G;
    g[j] = active[j] ? gj : G - 1;  // idle lanes shadow a real group and get a zero scale
    sg[j] = ZP ? g[j] / zp.ratio : g[j];
  }
  const int srow_len = ZP ? zp.groups : G;

  // All loads of one row set: independent, issued back to back.  Row sets and
  // rows past the end are clamped here and dropped at the store; the row base is
  // wave-uniform.
  auto load = [&](GemvFrag<ROWS, GPL>& f, int base_) {
    const int n0_ = min(base_ + set_in_block, nsets - 1) * ROWS;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const uint4_t* wrow = W + (int64_t)min(n0_ + r, N - 1) * G;
      const int64_t soff = (int64_t)min(n0_ + r, N - 1) * srow_len;
#pragma unroll
      for (int j = 0; j < GPL; ++j) {
        f.w[r][j] = __builtin_nontemporal_load(&wrow[g[j]]);
        if constexpr (ZP) {
          f.s[r][j] = as_half2(__builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(S) + soff + sg[j]));
        } else {
          f.s[r][j].x = __builtin_nontemporal_load(&S[soff + sg[j]]);
        }
      }
    }
  };

  // ---- 1. activations: thread t takes words t, t + nthreads, ... (8 halves each) ----
  constexpr int kMaxXW = 8;  // words of x per thread and batch row: K <= 8*8*nthreads
  const int nwords = K >> 3;
  uint4_t xraw[MB][kMaxXW];
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int i = 0; i < kMaxXW; ++i) {
      const int wi = tid + i * nthreads;
      if (wi < nwords) xraw[m][i] = reinterpret_cast<const uint4_t*>(x + (int64_t)m * K)[wi];
    }

  // ---- 2. weights and scales of the first row set: issued now, consumed last ----
  GemvFrag<ROWS, GPL> fa, fb;
  load(fa, base);

  // ---- 3. rearrange x, fold the zero point into c_g, publish through LDS ----
  // without zero points the constant 7 is folded here: 1024 + 7 and 64 + 7
  const half2_t k1031 = {(half_t)(ZP ? 1024.0f : 1031.0f), (half_t)(ZP ? 1024.0f : 1031.0f)};
  const half2_t k71 = {(half_t)(ZP ? 64.0f : 71.0f), (half_t)(ZP ? 64.0f : 71.0f)};
  const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int i = 0; i < kMaxXW; ++i) {
      const int wi = tid + i * nthreads;
      if (wi < nwords) {  // nwords % 4 == 0 and nthreads % 4 == 0: a quad is in or out together
        const uint4_t v = xraw[m][i];
        const uint32_t in[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
        pair_i_i4(in, o);  // o[i] = (x_i, x_{i+4})
        float c = dot2(as_half2(o[0]), k1031, 0.0f);
        c = dot2(as_half2(o[1]), k71, c);
        c = dot2(as_half2(o[2]), k1031, c);
        c = dot2(as_half2(o[3]), k71, c);
        // the 4 words of a group sit in 4 adjacent lanes
        c += dpp_shift<0xb1, 0xf>(c);  // quad_perm [1,0,3,2]
        c += dpp_shift<0x4e, 0xf>(c);  // quad_perm [2,3,0,1]
        const int grp = wi >> 2, ch = wi & 3;
        xs[(m * 4 + ch) * G + grp] = uint4_t{o[0], as_u32(as_half2(o[1]) * sixteenth), o[2],
                                             as_u32(as_half2(o[3]) * sixteenth)};
        if (ch == 0) cs[m * G + grp] = -c;
        if constexpr (ZP) {  // the zero point multiplies the plain sum of the group's activations
          float t = dot2(as_half2(o[0]), ones, 0.0f);
          t = dot2(as_half2(o[1]), ones, t);
          t = dot2(as_half2(o[2]), ones, t);
          t = dot2(as_half2(o[3]), ones, t);
          t += dpp_shift<0xb1, 0xf>(t);
          t += dpp_shift<0x4e, 0xf>(t);
          if (ch == 0) cs[(MB + m) * G + grp] = -t;
        }
      }
    }
  __syncthreads();

  // ---- 4. this lane's activations -> registers, for the whole kernel ----
  uint4_t xv[MB][GPL][4];
  float cg[MB][GPL];
  float cz[ZP ? MB : 1][GPL];
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int j = 0; j < GPL; ++j) {
#pragma unroll
      for (int c = 0; c < 4; ++c) xv[m][j][c] = xs[(m * 4 + c) * G + g[j]];
      cg[m][j] = cs[m * G + g[j]];
      if constexpr (ZP) cz[m][j] = cs[(MB + m) * G + g[j]];
    }

  const uint32_t magic = 0x64006400u;
  int turn = 0;

  // ---- 5. one row set: 1 shift + 4 and_or + 4 dot2 per word, reduce, store ----
  auto process = [&](const GemvFrag<ROWS, GPL>& f, int base_) {
    const int set = base_ + set_in_block;
    const bool set_ok = set < nsets;  // uniform per wavefront
    const int n0 = min(set, nsets - 1) * ROWS;
    float acc[ROWS][MB];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[r][m] = 0.0f;
#pragma unroll
      for (int j = 0; j < GPL; ++j) {
        float grp[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
          if constexpr (ZP) grp[m] = fmaf((float)f.s[r][j].y, cz[m][j], cg[m][j]);
          else grp[m] = cg[m][j];
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint4_t w4 = f.w[r][j];
          const uint32_t word = c == 0 ? w4.x : c == 1 ? w4.y : c == 2 ? w4.z : w4.w;
          const uint32_t w8 = word >> 8;
          const half2_t t0 = as_half2(and_or(word, 0x000F000Fu, magic));  // 1024 + (q0, q4)
          const half2_t t1 = as_half2(and_or(word, 0x00F000F0u, magic));  // 1024 + 16*(q1, q5)
          const half2_t t2 = as_half2(and_or(w8, 0x000F000Fu, magic));    // 1024 + (q2, q6)
          const half2_t t3 = as_half2(and_or(w8, 0x00F000F0u, magic));    // 1024 + 16*(q3, q7)
#pragma unroll
          for (int m = 0; m < MB; ++m) {
            float d = grp[m];
            d = dot2(t0, as_half2(xv[m][j][c].x), d);
            d = dot2(t1, as_half2(xv[m][j][c].y), d);
            d = dot2(t2, as_half2(xv[m][j][c].z), d);
            d = dot2(t3, as_half2(xv[m][j][c].w), d);
            grp[m] = d;
          }
        }
        const float sf = active[j] ? (float)f.s[r][j].x : 0.0f;
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[r][m] = fmaf(sf, grp[m], acc[r][m]);
      }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);

    auto finish = [&](float v, int r, int m) {
      const int n = n0 + r;
      if (n < N) {
        if (bias) v += (float)bias[n];
        half_t h = (half_t)v;
        if (residual) h = h + residual[(int64_t)m * N + n];
        y[(int64_t)m * N + n] = h;
      }
    };
    if (parts == 1) {
      if (lane == 63 && set_ok) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
#pragma unroll
          for (int m = 0; m < MB; ++m) finish(acc[r][m], r, m);
      }
    } else {
      // partial sums cross wavefronts through LDS; the buffer alternates between
      // turns so that one barrier per turn is enough
      float(*rb)[ROWS * MB] = red[turn & 1];
      if (lane == 63) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
#pragma unroll
          for (int m = 0; m < MB; ++m) rb[wave][r * MB + m] = acc[r][m];
      }
      __syncthreads();
      if (part == 0 && lane < ROWS * MB && set_ok) {
        float v = 0.0f;
        for (int w = 0; w < parts; ++w) v += rb[wave + w][lane];
        finish(v, lane / MB, lane % MB);
      }
    }
    ++turn;
  };

  // ---- 6. the workgroup's turns, loads of the next turn in flight during this one ----
  // `base` is uniform over the workgroup, so every wavefront takes the same number of turns.
  while (true) {
    if (base >= nsets) break;
    if (base + stride < nsets) load(fb, base + stride);
    process(fa, base);
    base += stride;
    if (base >= nsets) break;
    if (base + stride < nsets) load(fa, base + stride);
    process(fb, base);
    base += stride;
  }
}

template <bool ZP>
constexpr size_t gemv_lds_bytes(int MB, int64_t K) {
  return (size_t)MB * K * 2 + (size_t)MB * (K / 32) * 4 * (ZP ? 2 : 1);
}

// Workgroups of <ROWS, MB, GPL> for this shape, and how many of them one CU holds at a time.
template <int ROWS, int MB, int GPL, bool ZP>
static bool gemv_geometry(int64_t N, int64_t K, int64_t* nblocks, int* resident_per_cu) {
  const int G = (int)(K / 32);
  const int parts = (G + 64 * GPL - 1) / (64 * GPL);
  const int sets_per_block = parts >= 4 ? 1 : 4 / parts;
  const int threads = 64 * parts * sets_per_block;
  if (parts > kGemvMaxWaves || threads > gemv_max_threads<GPL>()) return false;
  const size_t lds = gemv_lds_bytes<ZP>(MB, K);
  if (lds > 60 * 1024) return false;
  const int64_t nsets = (N + ROWS - 1) / ROWS;
  *nblocks = (nsets + sets_per_block - 1) / sets_per_block;
  // the last answer of the occupancy query, per instantiation: (threads, lds, workgroups per CU)
  // packed into one atomic word, so that concurrent callers read a consistent triple
  static std::atomic<uint64_t> cache{0};
  const uint64_t key = ((uint64_t)threads << 48) | ((uint64_t)lds << 16);
  uint64_t c = cache.load(std::memory_order_acquire);
  if ((c & ~0xffffull) != key || c == 0) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, q4g32_gemv_kernel<ROWS, MB, GPL, ZP>, threads, lds) != hipSuccess)
      return false;
    c = key | (uint64_t)(n & 0xffff);
    cache.store(c, std::memory_order_release);
  }
  *resident_per_cu = (int)(c & 0xffff);
  return true;
}

template <int ROWS, int MB, int GPL, bool ZP>
static int launch_gemv(const char* who, const uint32_t* W, const uint16_t* S, const GemvZp& zp, const uint16_t* x,
                       const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t N,
                       int64_t K, int blocks_per_cu, hipStream_t stream) {
  const int G = (int)(K / 32);
  const int parts = (G + 64 * GPL - 1) / (64 * GPL);
  const int sets_per_block = parts >= 4 ? 1 : 4 / parts;
  const int threads = 64 * parts * sets_per_block;
  if (parts > kGemvMaxWaves || threads > gemv_max_threads<GPL>())
    return fail(WQ_EUNSUPPORTED, "%s: K=%lld needs %d threads per row set", who, (long long)K,
                threads);
  const int64_t nsets = (N + ROWS - 1) / ROWS;
  int64_t blocks = (nsets + sets_per_block - 1) / sets_per_block;
  // More workgroups than `blocks_per_cu` per CU: persistent workgroups that take several
  // turns, with the loads of the next turn in flight during the current one.
  const int forced_per_cu = tuning().gemv_blocks_per_cu;
  const int64_t cap = (int64_t)cu_count() * (forced_per_cu ? forced_per_cu : blocks_per_cu);
  if (blocks > cap) blocks = cap;
  if (K > 8 * 8 * (int64_t)threads)
    return fail(WQ_EUNSUPPORTED, "%s: K=%lld too large for %d threads", who, (long long)K,
                threads);
  const size_t lds = gemv_lds_bytes<ZP>(MB, K);
  auto kern = q4g32_gemv_kernel<ROWS, MB, GPL, ZP>;
  if (lds > 60 * 1024) {
    static DynamicLdsLimit limit;
    WQ_HIP(limit.ensure(reinterpret_cast<const void*>(kern), (int)lds));
  }
  WQ_LAUNCH(who, kern, dim3((unsigned)blocks), dim3(threads), lds, stream, (const uint4_t*)W, (const half_t*)S, (const half_t*)x,
            (const half_t*)bias, (const half_t*)residual, (half_t*)y, (int)N, (int)K, parts,
            (int)nsets, zp);
  return WQ_OK;
}

// rows == 0 chooses the rows per wavefront from the shape (timings of the Llama-7B layers):
// what costs most at these kernel lengths (4 .. 12 us) is a second, partly filled round of
// workgroups, so take the most rows per wavefront (4, 2, 1) for which all workgroups are
// resident at once and every CU still has at least two; if nothing fits (tall matrices, long rows),
// persistent workgroups that take several turns each.
template <int MB, int GPL, bool ZP>
static int launch_gemv_rows(const char* who, int rows, const uint32_t* W, const uint16_t* S, const GemvZp& zp, const uint16_t* x,
                            const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t N,
                            int64_t K, hipStream_t stream) {
  int bpc = 32;
  if (rows == 0) {
    const int cus = cu_count();
    int64_t nb = 0;
    int per_cu = 0;
    if (gemv_geometry<4, MB, GPL, ZP>(N, K, &nb, &per_cu) && nb >= 2 * cus && nb <= (int64_t)cus * per_cu) {
      rows = 4;
    } else if (gemv_geometry<2, MB, GPL, ZP>(N, K, &nb, &per_cu) && nb >= 2 * cus && nb <= (int64_t)cus * per_cu) {
      rows = 2;
    } else if (gemv_geometry<1, MB, GPL, ZP>(N, K, &nb, &per_cu) && nb <= (int64_t)cus * per_cu) {
      rows = 1;
    } else {
      // tall or long: persistent workgroups, as many per CU as are resident at once and at most four (rows of
      // more than 8192 columns need workgroups of 7 .. 16 wavefronts and up to 60 KB of LDS, of which two or three
      // fit: N = 8192, K = 28672 with four per CU 31.0 us, with two, two rows per wavefront, 25.0 us; N = 4096,
      // K = 14336: 10.1 -> 8.8 us)
      rows = K > 8192 ? 2 : 1;
      const bool fits = rows == 2 ? gemv_geometry<2, MB, GPL, ZP>(N, K, &nb, &per_cu)
                                  : gemv_geometry<1, MB, GPL, ZP>(N, K, &nb, &per_cu);
      bpc = fits && per_cu >= 1 ? std::min(4, per_cu) : 4;
    }
  }
  switch (rows) {
    case 1: return launch_gemv<1, MB, GPL, ZP>(who, W, S, zp, x, bias, residual, y, N, K, bpc, stream);
    case 2: return launch_gemv<2, MB, GPL, ZP>(who, W, S, zp, x, bias, residual, y, N, K, bpc, stream);
    default: return launch_gemv<4, MB, GPL, ZP>(who, W, S, zp, x, bias, residual, y, N, K, bpc, stream);
  }
}

// Two rows of x share one pass over the weights (four in registers spill and run slower than two passes).
template <bool ZP>
static int gemv_dispatch(const char* who, const uint32_t* W, const uint16_t* S, const GemvZp& zp, const uint16_t* x,
                         const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                         int64_t K, hipStream_t stream) {
  const int G = (int)(K / 32);
  // groups per lane: one wavefront covers a whole row when K <= 64*32*GPL
  // (rows longer than 256 groups are split over several wavefronts)
  int gpl = tuning().gemv_gpl ? tuning().gemv_gpl
                       : (G <= 64 ? 1 : G <= 128 ? 2 : G <= 192 ? 3 : G <= 256 ? 4 : G <= 384 ? 3 : 2);
  const int rows = tuning().gemv_rows;  // 0 = from the shape
  // pairs of rows of x share one pass over the weights
  for (int64_t m0 = 0; m0 < M;) {
    const int64_t left = M - m0;
    const uint16_t* xp = x + m0 * K;
    const uint16_t* rp = residual ? residual + m0 * N : nullptr;
    uint16_t* yp = y + m0 * N;
    int rc;
    if (left >= 2) {
      rc = gpl >= 2 ? launch_gemv_rows<2, 2, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream)
                    : launch_gemv_rows<2, 1, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream);
      m0 += 2;
    } else {
      rc = gpl == 1   ? launch_gemv_rows<1, 1, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream)
           : gpl == 2 ? launch_gemv_rows<1, 2, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream)
           : gpl == 3 ? launch_gemv_rows<1, 3, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream)
           : gpl == 4 ? launch_gemv_rows<1, 4, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream)
                      : launch_gemv_rows<1, 6, ZP>(who, rows, W, S, zp, xp, bias, rp, yp, N, K, stream);
      m0 += 1;
    }
    if (rc != WQ_OK) return rc;
  }
  return WQ_OK;
}

}  // namespace wq
