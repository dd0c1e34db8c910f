// Format B (fp16 x int8/int4, preprocessed layout): dequantization entry point and
// the small-M (decode) GEMV.
//
// Layout recap (see intb_preprocess.hip).  int8: column pairs are interleaved,
// [N/2][K/64][2][64 bytes]; a 16-byte piece holds 16 consecutive k of one column,
// word j of the piece = bytes (k0+2j, k0+2j+8, k0+2j+1, k0+2j+9), each stored as
// q + 128.  int4: column quads, [N/4][K/64][4][32 bytes]; a 16-byte piece holds 32
// consecutive k of one column, nibbles (i, i+4) of word j = (k0+2j+8i, k0+2j+8i+1),
// each stored as q + 8.  In both cases a packed fp16 pair comes out as (k, k+1).
//
// GEMV.  One wavefront streams R column groups (pairs / quads): lane l reads the
// 16-byte pieces l, l+64, ... of the group, which keeps the lane on one column
// ((l%8)/4 resp. (l%8)/2) for the whole kernel.  The activations are staged once
// per workgroup in LDS (natural order: no rearrangement is needed for this
// format) together with a per-piece constant that folds the unsigned offset:
//   sum_k x_k q_k = sum_k x_k (1024 + u_k)  -  (1024 + bias) * sum_k x_k
// where 1024 + u is the fp16 number made by placing u in the mantissa of 0x6400.
// (int4: codes with k%16 >= 8 are taken unshifted as 1024 + 16u and meet
// activations pre-multiplied by 1/16.)  The per-channel scale multiplies the
// finished sum; fine-grained scales multiply each 64-row tile.
#include "tuning.h"
#include "wq_device.h"
#include "wq_host.h"
#include "intb_common.h"

namespace wq {

// ------------------------------------------------------------------ dequantize
// One thread per 16-byte piece; writes fp16 [K, N] row-major (the reference's
// decode output), bit-exact: exact integer -> fp16, one rounding in the multiply.
template <int NBIT>
__global__ __launch_bounds__(256) void intb_dequant_kernel(const uint4_t* __restrict__ B,
                                                           const half_t* __restrict__ scales,
                                                           half_t* __restrict__ out, int K, int N,
                                                           int group, int64_t npieces) {
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= npieces) return;
  constexpr int I = NBIT == 8 ? 2 : 4;             // interleaved columns
  constexpr int PPT = NBIT == 8 ? 4 : 2;           // pieces per column per tile
  constexpr int KPP = 64 / PPT;                    // k per piece
  const int64_t per_group = (int64_t)(K / 64) * I * PPT;
  const int64_t cg = p / per_group, rem = p % per_group;
  const int tile = (int)(rem / (I * PPT)), within = (int)(rem % (I * PPT));
  const int n = (int)(cg * I + within / PPT);
  const int k0 = tile * 64 + (within % PPT) * KPP;
  const half_t s = group > 0 ? scales[(int64_t)(k0 / group) * N + n] : scales[n];
  const half2_t s2 = {s, s};
  const uint4_t v = B[p];
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  if (NBIT == 8) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const half2_t lo = u8x2_to_half2(w[j], 0x04020400u) * s2;  // (k0+2j, k0+2j+1)
      const half2_t hi = u8x2_to_half2(w[j], 0x04030401u) * s2;  // (k0+2j+8, k0+2j+9)
      out[(int64_t)(k0 + 2 * j) * N + n] = lo.x;
      out[(int64_t)(k0 + 2 * j + 1) * N + n] = lo.y;
      out[(int64_t)(k0 + 2 * j + 8) * N + n] = hi.x;
      out[(int64_t)(k0 + 2 * j + 9) * N + n] = hi.y;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      half2_t d[4];
      u4_word_minus8(w[j], d);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const half2_t q = d[i] * s2;  // (k0+2j+8i, k0+2j+8i+1)
        out[(int64_t)(k0 + 2 * j + 8 * i) * N + n] = q.x;
        out[(int64_t)(k0 + 2 * j + 8 * i + 1) * N + n] = q.y;
      }
    }
  }
}

// ------------------------------------------------------------------------ GEMV
constexpr int kIntbGemvThreads = 512;  // at most: 4 .. 8 wavefronts per workgroup, chosen at launch

__device__ __forceinline__ half_t intb_finish(float v, int m, int n, int N, const IntbEpilogue& ep) {
  if (ep.bias) v += (float)ep.bias[ep.bias_stride ? (int64_t)m * ep.bias_stride + n : n];
  v = apply_activation(v, ep.activation);
  if (ep.residual) {
    const float r = (float)ep.residual[(int64_t)m * N + n];
    if (ep.binary_op == 1) v += r;
    if (ep.binary_op == 2) v *= r;
  }
  if (ep.unary_op == 1) v = v > 0.0f ? v : 0.0f;
  return (half_t)v;
}

// R column groups per wavefront, MB rows of A, U pieces per lane in flight per group.
template <int NBIT, int R, int MB, int U>
__global__ __launch_bounds__(kIntbGemvThreads) void intb_gemv_kernel(
    const uint4_t* __restrict__ B, const half_t* __restrict__ scales, const half_t* __restrict__ A,
    half_t* __restrict__ C, int N, int K, int group, int ngroups, int ks_log2, IntbEpilogue ep) {
  constexpr int I = NBIT == 8 ? 2 : 4;      // interleaved columns per group
  constexpr int PPT = NBIT == 8 ? 4 : 2;    // pieces per column per tile
  constexpr int XQ = NBIT == 8 ? 2 : 4;     // 16-byte chunks of x per piece
  extern __shared__ uint4_t smem[];
  uint4_t* xs = smem;                                        // [MB][K/8] chunks of 8 halves
  float* cs = reinterpret_cast<float*>(smem + MB * (K >> 3));  // [MB][K/16 or K/32] folded offsets
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ncs = K / (NBIT == 8 ? 16 : 32);
  const int pieces = (K / 64) * I * PPT;    // 16-byte pieces per column group
  // 2^ks_log2 neighbouring wavefronts of a workgroup share the groups of one and split K (a narrow
  // matrix has too few column groups to give every SIMD its wavefronts otherwise)
  const int gwave = blockIdx.x * ((int)blockDim.x >> 6) + wave;
  const int kpart = gwave & ((1 << ks_log2) - 1);
  const int gset = (gwave >> ks_log2) * R;  // first group of this wave
  float* red = cs + MB * ncs;               // [wavefronts][R][I][MB] partial sums of the K parts

  // ---- stage x (natural order) and the per-piece offset constants ----
  {
    const half2_t kA = NBIT == 8 ? half2_t{(half_t)1152.0f, (half_t)1152.0f}
                                 : half2_t{(half_t)1032.0f, (half_t)1032.0f};
    const half2_t kB = NBIT == 8 ? kA : half2_t{(half_t)72.0f, (half_t)72.0f};
    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    const int nchunks = K >> 3;
    for (int m = 0; m < MB; ++m)
      for (int ci = tid; ci < nchunks; ci += (int)blockDim.x) {
        uint4_t v = reinterpret_cast<const uint4_t*>(A + (int64_t)m * K)[ci];
        // chunk ci covers k = 8ci..8ci+7; (k % 16) >= 8 for odd ci
        const bool upper = ci & 1;
        const half2_t kk = (NBIT == 4 && upper) ? kB : kA;
        float c = dot2(as_half2(v.x), kk, 0.0f);
        c = dot2(as_half2(v.y), kk, c);
        c = dot2(as_half2(v.z), kk, c);
        c = dot2(as_half2(v.w), kk, c);
        if (NBIT == 4 && upper) {
          v = uint4_t{as_u32(as_half2(v.x) * sixteenth), as_u32(as_half2(v.y) * sixteenth),
                      as_u32(as_half2(v.z) * sixteenth), as_u32(as_half2(v.w) * sixteenth)};
        }
        // sum over the 2 (int8) or 4 (int4) adjacent chunks of one piece
        c += dpp_quad<0xb1>(c);
        if (NBIT == 4) c += dpp_quad<0x4e>(c);
        xs[m * nchunks + ci] = v;
        if ((ci & (XQ - 1)) == 0) cs[m * ncs + ci / XQ] = -c;
      }
  }
  __syncthreads();
  if (gset >= ngroups && ks_log2 == 0) return;  // (with a split of K every wavefront goes on to the barrier below)

  // lane geometry: piece index p = lane + 64*it; column and k-position follow from p % 8
  const int col_in_group = (lane & 7) / PPT;
  const int sub = lane & (PPT - 1);  // which 16 (int8) / 32 (int4) k of the tile

  float acc[R][MB];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = 0.0f;

  const uint32_t magic = 0x64006400u;
  // fine-grained scales [K/64, N]: the R*I columns of this wavefront are adjacent, so one 8-byte
  // (int8) or 16-byte (int4) load per tile fetches the scales of all of them (gset is a multiple of
  // R and N / I of 16: the load stays inside the row); needs 16-byte aligned scales
  constexpr bool kVecFits = R * I * 2 == 8 || R * I * 2 == 16;
  const bool vec_scales = kVecFits && group > 0 && (reinterpret_cast<uintptr_t>(scales) & 15u) == 0;
  // this wavefront's part of K: whole rounds of 64 U pieces
  const int rounds = (pieces + 64 * U - 1) / (64 * U);
  const int rounds_part = (rounds + (1 << ks_log2) - 1) >> ks_log2;
  const int p_begin = gset < ngroups ? min(kpart * rounds_part * 64 * U, pieces) : 0;
  const int p_end = gset < ngroups ? min(p_begin + rounds_part * 64 * U, pieces) : 0;
  for (int p0 = p_begin; p0 < p_end; p0 += 64 * U) {
    uint4_t wv[R][U];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint4_t* src = B + (int64_t)min(gset + r, ngroups - 1) * pieces;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = min(p0 + 64 * u + lane, pieces - 1);
        wv[r][u] = __builtin_nontemporal_load(&src[p]);
      }
    }
    uint4_t sv[U];
    if (vec_scales) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int tile_u = min(p0 + 64 * u + lane, pieces - 1) >> 3;
        const half_t* sp = scales + (int64_t)tile_u * N + gset * I;
        if (R * I * 2 == 16) {
          sv[u] = *reinterpret_cast<const uint4_t*>(sp);
        } else {
          const uint2_t t = *reinterpret_cast<const uint2_t*>(sp);
          sv[u] = uint4_t{t.x, t.y, 0u, 0u};
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + 64 * u + lane;
      const bool ok = p < pieces;
      const int tile = min(p, pieces - 1) >> 3;
      const int xi = (tile * PPT + sub);  // piece-sized slot of x
      float part[R][MB];
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const float c0 = cs[m * ncs + xi];
#pragma unroll
        for (int r = 0; r < R; ++r) part[r][m] = c0;
      }
      if (NBIT == 8) {
        // piece = 4 words; word j -> pairs (2j, 2j+1) and (2j+8, 2j+9): x chunk 0 resp. 1
        uint4_t xa[MB], xb[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
          xa[m] = xs[m * (K >> 3) + xi * 2];
          xb[m] = xs[m * (K >> 3) + xi * 2 + 1];
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint32_t w[4] = {wv[r][u].x, wv[r][u].y, wv[r][u].z, wv[r][u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const half2_t lo = as_half2(__builtin_amdgcn_perm(0x64646464u, w[j], 0x04020400u));
            const half2_t hi = as_half2(__builtin_amdgcn_perm(0x64646464u, w[j], 0x04030401u));
#pragma unroll
            for (int m = 0; m < MB; ++m) {
              const uint32_t xlo = j == 0 ? xa[m].x : j == 1 ? xa[m].y : j == 2 ? xa[m].z : xa[m].w;
              const uint32_t xhi = j == 0 ? xb[m].x : j == 1 ? xb[m].y : j == 2 ? xb[m].z : xb[m].w;
              part[r][m] = dot2(lo, as_half2(xlo), part[r][m]);
              part[r][m] = dot2(hi, as_half2(xhi), part[r][m]);
            }
          }
        }
      } else {
        // piece = 4 words; word j, pair i -> (2j+8i, 2j+8i+1): x chunk i, dword j
        uint4_t xc[MB][4];
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
          for (int i = 0; i < 4; ++i) xc[m][i] = xs[m * (K >> 3) + xi * 4 + i];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint32_t w[4] = {wv[r][u].x, wv[r][u].y, wv[r][u].z, wv[r][u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t w8 = w[j] >> 8;
            const half2_t t0 = as_half2(and_or(w[j], 0x000F000Fu, magic));  // 1024 + u      pair i=0
            const half2_t t1 = as_half2(and_or(w[j], 0x00F000F0u, magic));  // 1024 + 16u    pair i=1
            const half2_t t2 = as_half2(and_or(w8, 0x000F000Fu, magic));    //               pair i=2
            const half2_t t3 = as_half2(and_or(w8, 0x00F000F0u, magic));    //               pair i=3
#pragma unroll
            for (int m = 0; m < MB; ++m) {
              auto pick = [&](const uint4_t& q) {
                return as_half2(j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w);
              };
              float d = part[r][m];
              d = dot2(t0, pick(xc[m][0]), d);
              d = dot2(t1, pick(xc[m][1]), d);
              d = dot2(t2, pick(xc[m][2]), d);
              d = dot2(t3, pick(xc[m][3]), d);
              part[r][m] = d;
            }
          }
        }
      }
      // fine-grained scales multiply per 64-row tile, per-channel scales at the end
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float sf = ok ? 1.0f : 0.0f;
        if (vec_scales) {
          // half (r * I + col_in_group) of the vector
          const int h = r * I + col_in_group;
          const uint32_t word = (h >> 1) == 0 ? sv[u].x : (h >> 1) == 1 ? sv[u].y : (h >> 1) == 2 ? sv[u].z : sv[u].w;
          const half2_t pair = as_half2(word);
          sf = ok ? (float)((h & 1) ? pair.y : pair.x) : 0.0f;
        } else if (group > 0) {
          const int n = min(gset + r, ngroups - 1) * I + col_in_group;
          sf = ok ? (float)scales[(int64_t)tile * N + n] : 0.0f;
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[r][m] = fmaf(sf, part[r][m], acc[r][m]);
      }
    }
  }

  // ---- reduce over the lanes that share a column: lanes with equal (lane % 8) / PPT ----
  // xor 1, 2 (int8: within the 4 lanes of a column; int4: xor 1 only), then 8, 16, 32.
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      float v = acc[r][m];
      v += dpp_quad<0xb1>(v);                 // xor 1
      if (NBIT == 8) v += dpp_quad<0x4e>(v);  // xor 2
      v += __shfl_xor(v, 8, 64);
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      acc[r][m] = v;
    }
  const bool holder = lane < 8 && (lane & (PPT - 1)) == 0;  // one lane per column of a group
  if (ks_log2) {
    // the parts of K meet in LDS; the wavefront of part 0 adds them in order of K
    if (holder) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MB; ++m) red[((wave * R + r) * I + col_in_group) * MB + m] = acc[r][m];
    }
    __syncthreads();
    if (kpart != 0 || gset >= ngroups) return;
    if (holder) {
      for (int k = 1; k < (1 << ks_log2); ++k)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MB; ++m) acc[r][m] += red[(((wave + k) * R + r) * I + col_in_group) * MB + m];
    }
  }
  if (holder) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int g = gset + r;
      if (g >= ngroups) break;
      const int n = g * I + col_in_group;
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        float v = acc[r][m];
        if (group <= 0) v *= (float)scales[n];
        C[(int64_t)m * N + n] = intb_finish(v, m, n, N, ep);
      }
    }
  }
}

template <int NBIT, int R, int MB, int U = (NBIT == 8 ? 4 : 1)>
static int launch_intb_gemv(const uint16_t* A, const int8_t* B, const uint16_t* scales, uint16_t* C,
                            int64_t N, int64_t K, int64_t group, const IntbEpilogue& ep,
                            hipStream_t stream) {
  constexpr int I = NBIT == 8 ? 2 : 4;
  const int ngroups = (int)(N / I);
  // Wavefronts per workgroup: every workgroup stages x for itself (the more wavefronts, the less of that), and all
  // workgroups are resident at once, so the launch is as long as the CU with most of them: 4 .. 8 wavefronts,
  // whichever leaves the fullest last round (K = 8192, N = 28672, int4, two groups per wavefront: 3584 wavefronts
  // are 896 workgroups of 4, i.e. 3.5 per CU, or 512 of 7, i.e. 2 per CU).
  // A narrow matrix has too few column groups for that.  int4 at one row (one piece per lane in flight, the most
  // arithmetic per byte) then lets 2, 4 or 8 neighbouring wavefronts share a group and split K, whichever brings
  // the launch closest to 18 wavefronts per CU (K = 28672, N = 8192: 47 us unsplit, 37 us through the small-batch
  // kernel, 22.5 us split 4 ways; K = 13824, N = 5120: 17.4 -> 10.4 us split 8 ways; N = 22016: 2 ways, N = 28672:
  // none).  int8 keeps whole columns: its wavefronts have four pieces per lane in flight, and a split measured
  // 5 .. 10 % slower on most shapes.
  const int64_t group_waves = (ngroups + R - 1) / R;
  constexpr int PPT = NBIT == 8 ? 4 : 2;
  const int64_t k_rounds = ((K / 64) * I * PPT + 64 * U - 1) / (64 * U);
  int ks_log2 = 0;
  if (tuning().intb_k_split) {
    while ((1 << ks_log2) < tuning().intb_k_split && ks_log2 < 3) ++ks_log2;
  } else if (NBIT == 4 && MB == 1) {
    const double want = 18.0 * cu_count();
    double best_d = -1.0;
    for (int s = 0; s <= 3 && (k_rounds >> s) >= 1; ++s) {
      const double ratio = (double)(group_waves << s) / want;
      const double d = ratio > 1.0 ? ratio : 1.0 / ratio;  // distance on a logarithmic scale
      if (best_d < 0.0 || d < best_d) best_d = d, ks_log2 = s;
    }
  }
  const int64_t total_waves = group_waves << ks_log2;
  // (measured at M = 1: int4 per-channel 22.7 us with 4, 21.6 with 7; int8 group-64 46.0 with 4, 40.9 with 7, 48.8 with 8;
  // int8 per-channel, 7168 wavefronts: 37.9 .. 38.3 us with any of them)
  int waves = 4;
  double best = -1.0;
  for (int w = 4; w <= 8; ++w) {
    if (w & ((1 << ks_log2) - 1)) continue;  // the wavefronts of a group sit in one workgroup
    const int64_t b = (total_waves + w - 1) / w;
    const int64_t rounds = (b + cu_count() - 1) / cu_count();
    const double fill = (double)b / (double)(rounds * cu_count());  // 1: every CU has the same number
    if (fill > best - 1e-9) {  // the fullest last round; among equals the most wavefronts
      best = std::max(best, fill);
      waves = w;
    }
  }
  const int64_t blocks = (total_waves + waves - 1) / waves;
  const size_t lds = (size_t)MB * K * 2 + (size_t)MB * (K / (NBIT == 8 ? 16 : 32)) * 4 +
                     (ks_log2 ? (size_t)waves * R * I * MB * 4 : 0);
  auto kern = intb_gemv_kernel<NBIT, R, MB, U>;
  if (lds > 60 * 1024) {
    static DynamicLdsLimit limit;  // per instantiation
    WQ_HIP(limit.ensure(reinterpret_cast<const void*>(kern), (int)lds));
  }
  WQ_LAUNCH("wq_fpA_intB_gemm(gemv)", kern, dim3((unsigned)blocks), dim3((unsigned)(64 * waves)), lds,
            stream, (const uint4_t*)B, (const half_t*)scales, (const half_t*)A, (half_t*)C, (int)N,
            (int)K, (int)group, ngroups, ks_log2, ep);
  return WQ_OK;
}

// column groups per wavefront at one row (two rows: always 2)
static int intb_gemv_groups_per_wave(int64_t group, int nbit) {
  return tuning().gemv_rows ? tuning().gemv_rows : (group > 0 || nbit == 4 ? 2 : 1);
}

int64_t intb_gemv_wavefronts(int64_t m, int64_t n, int64_t group, int nbit) {
  const int I = nbit == 8 ? 2 : 4;
  const int R = m >= 2 ? 2 : intb_gemv_groups_per_wave(group, nbit);
  return (n / I + R - 1) / R;
}

// Called by the dispatcher in intb_gemm.hip for m <= 4.
int intb_gemv_dispatch(const uint16_t* A, const int8_t* B, const uint16_t* scales, uint16_t* C,
                       int64_t m, int64_t n, int64_t k, int64_t group, int nbit,
                       const IntbEpilogue& ep_in, hipStream_t stream) {
  if (k > 32768) return fail(WQ_EUNSUPPORTED, "wq_fpA_intB_gemm: k=%lld > 32768 at small m", (long long)k);
  for (int64_t m0 = 0; m0 < m;) {
    IntbEpilogue ep = ep_in;
    if (ep.bias && ep.bias_stride) ep.bias += m0 * ep.bias_stride;
    if (ep.residual) ep.residual += m0 * n;
    const uint16_t* a = A + m0 * k;
    uint16_t* c = C + m0 * n;
    int rc;
    if (m - m0 >= 2) {
      rc = nbit == 8 ? launch_intb_gemv<8, 2, 2>(a, B, scales, c, n, k, group, ep, stream)
                     : launch_intb_gemv<4, 2, 2>(a, B, scales, c, n, k, group, ep, stream);
      m0 += 2;
    } else {
      // column groups per wavefront and pieces per lane in flight per group (K = 8192, N = 28672, M = 1).  int8: one
      // group with per-channel scales (40.4 -> 37.9 us), two with group scales, whose 8- or 16-byte scale vectors
      // then serve both (45.4 against 48.1 us), four pieces (66 registers).  int4: two groups, ONE piece: with four
      // pieces the compiler keeps 16 LDS operands per piece in registers (154: three wavefronts per SIMD); one piece
      // needs 68 (seven per SIMD): per-channel 27.2 -> 22.2 us, group-64 27.1 -> 23.2 us.
      const int R = intb_gemv_groups_per_wave(group, nbit);
      if (R == 1)
        rc = nbit == 8 ? launch_intb_gemv<8, 1, 1>(a, B, scales, c, n, k, group, ep, stream)
                       : launch_intb_gemv<4, 1, 1>(a, B, scales, c, n, k, group, ep, stream);
      else
        rc = nbit == 8 ? launch_intb_gemv<8, 2, 1>(a, B, scales, c, n, k, group, ep, stream)
                       : launch_intb_gemv<4, 2, 1>(a, B, scales, c, n, k, group, ep, stream);
      m0 += 1;
    }
    if (rc != WQ_OK) return rc;
  }
  return WQ_OK;
}

}  // namespace wq

extern "C" int wq_intb_dequantize(const int8_t* B, const uint16_t* scales, uint16_t* out, int64_t K,
                                  int64_t N, int weight_nbit, int64_t group_size,
                                  wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(weight_nbit == 8 || weight_nbit == 4, "wq_intb_dequantize: weight_nbit must be 8 or 4");
  WQ_REQUIRE(K >= 0 && N >= 0 && K % 64 == 0 && N % 64 == 0,
             "wq_intb_dequantize: K=%lld and N=%lld must be multiples of 64", (long long)K,
             (long long)N);
  WQ_REQUIRE(group_size <= 0 || group_size == 64 || group_size == K,
             "wq_intb_dequantize: group_size must be 64 (fine-grained) or <= 0 / k (per column)");
  if (K * N == 0) return WQ_OK;
  WQ_REQUIRE(B && scales && out, "wq_intb_dequantize: null pointer");
  WQ_REQUIRE(aligned16(B), "wq_intb_dequantize: B must be 16-byte aligned");
  WQ_REQUIRE(K < (1ll << 31) && N < (1ll << 31), "wq_intb_dequantize: tensor too large");
  const int group = (group_size > 0 && group_size != K) ? (int)group_size : 0;
  const int64_t npieces = K * N * weight_nbit / 8 / 16;
  const int64_t blocks = (npieces + 255) / 256;
  if (weight_nbit == 8) {
    WQ_LAUNCH("wq_intb_dequantize", intb_dequant_kernel<8>, dim3((unsigned)blocks), dim3(256), 0,
              (hipStream_t)stream, (const uint4_t*)B, (const half_t*)scales, (half_t*)out, (int)K,
              (int)N, group, npieces);
  } else {
    WQ_LAUNCH("wq_intb_dequantize", intb_dequant_kernel<4>, dim3((unsigned)blocks), dim3(256), 0,
              (hipStream_t)stream, (const uint4_t*)B, (const half_t*)scales, (half_t*)out, (int)K,
              (int)N, group, npieces);
  }
  return WQ_OK;
}
