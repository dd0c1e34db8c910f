// Format B GEMM entry points: fp16 activations x preprocessed int8 / int4 weights,
// the MI355X-native counterpart of fastertransformer::gemm_fp16_int_bias_act and
// gemm_fp16_int_bias_act_residual (call sites python/tvm/contrib/cutlass/gemm_operation.py:441-458).
// m <= 2 goes to the streaming GEMV (intb_gemv.hip), m <= 64 to the small-batch
// kernel (intb_skinny.hip), larger m to the shared MFMA GEMM (mfma_gemm.h) with the
// weight loaders below.
#include "intb_common.h"
#include "mfma_gemm.h"
#include "mfma_gemm_lds.h"

int wq_gemm_cfg_override();

namespace wq {

// Per K-step (one 64-row tile) lane (j, h) needs k = 32h..32h+31 of column n.
// int8: two 16-byte pieces (16 k each) at ((n/2)*(K/64) + ks)*8 + (n%2)*4 + 2h (16-byte units);
// int4: one 16-byte piece (32 k) at ((n/4)*(K/64) + ks)*8 + (n%4)*2 + h.
// Both come out in natural k order, so the activations are stored unpermuted.
template <int NBIT>
struct IntbLoader {
  static constexpr bool kPairA = false;
  static constexpr int kPieces = NBIT == 8 ? 2 : 1;
  struct Args {
    const uint4_t* B;
    const half_t* scales;
    int group;  // 0 = per column, 64 = one scale per K-step
  };
  struct Lane {
    const uint4_t* w;
    const half_t* s;  // per column: &scales[n]; fine-grained: &scales[n] with row stride N
    int N;
  };
  struct Frag {
    uint4_t w[kPieces];
    half_t s;
  };
  __device__ __forceinline__ static void init(Lane& l, const Args& a, int n, int lh, int K, int N) {
    constexpr int I = NBIT == 8 ? 2 : 4;
    l.w = a.B + ((int64_t)(n / I) * (K >> 6)) * 8 + (n % I) * (8 / I) + lh * kPieces;
    l.s = a.scales + n;
    l.N = N;
  }
  __device__ __forceinline__ static void load(Frag& f, const Lane& l, const Args& a, int ks, int, int, bool) {
#pragma unroll
    for (int p = 0; p < kPieces; ++p) f.w[p] = l.w[(int64_t)ks * 8 + p];
    f.s = a.group ? l.s[(int64_t)ks * l.N] : l.s[0];
  }
  __device__ __forceinline__ static void dequant(const Frag& f, half8_t out[4]) {
    const half2_t s2 = {f.s, f.s};
    if (NBIT == 8) {
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const uint32_t w[4] = {f.w[p].x, f.w[p].y, f.w[p].z, f.w[p].w};
        half2_t lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          lo[j] = u8x2_to_half2(w[j], 0x04020400u) * s2;  // k = 2j, 2j+1
          hi[j] = u8x2_to_half2(w[j], 0x04030401u) * s2;  // k = 2j+8, 2j+9
        }
        out[2 * p] = half8_t{lo[0].x, lo[0].y, lo[1].x, lo[1].y, lo[2].x, lo[2].y, lo[3].x, lo[3].y};
        out[2 * p + 1] = half8_t{hi[0].x, hi[0].y, hi[1].x, hi[1].y, hi[2].x, hi[2].y, hi[3].x, hi[3].y};
      }
    } else {
      const uint32_t w[4] = {f.w[0].x, f.w[0].y, f.w[0].z, f.w[0].w};
      half2_t d[4][4];  // d[j][i] = (k = 2j+8i, 2j+8i+1)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u4_word_minus8(w[j], d[j]);
#pragma unroll
        for (int i = 0; i < 4; ++i) d[j][i] = d[j][i] * s2;
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
        out[kk] = half8_t{d[0][kk].x, d[0][kk].y, d[1][kk].x, d[1][kk].y,
                          d[2][kk].x, d[2][kk].y, d[3][kk].x, d[3][kk].y};
    }
  }
};


// Weight policy of the fully LDS-staged kernel (mfma_gemm_lds.h) for the preprocessed layouts
// with per-column scales.  A K-step (one 64-row tile) of I = 2 (int8) or 4 (int4) interleaved
// columns is 128 contiguous bytes, so the B tile is fetched in whole 128-byte lines; the scale
// of a column never changes and stays in a register.
// GROUPED (scales fp16 [K/64, N], one per column and K-step): a lane stages the 4 bytes that hold
// the scales of its column and the neighbouring one, and the reader takes its half.
template <int NBIT, bool GROUPED = false>
struct IntbLdsPolicy {
  static constexpr int I = NBIT == 8 ? 2 : 4;
  static constexpr int kColBytes = 128 / I;
  static constexpr int kScaleBytes = GROUPED ? 4 : 0;
  static constexpr int kStepStride = 128;
  struct Args {
    const uint4_t* B;
    const half_t* scales;
    int N;
  };
  struct Frag {
    uint4_t w[NBIT == 8 ? 2 : 1];
  };
  __device__ __forceinline__ static const char* b_src(const Args& a, int n0, int q, int N, int K) {
    const int group = min(n0 / I + (q >> 3), N / I - 1);  // columns past N re-read the last group
    return reinterpret_cast<const char*>(a.B) + ((int64_t)group * (K >> 6)) * 128 + (q & 7) * 16;
  }
  using Scale = half2_t;  // the column's scale, twice
  __device__ __forceinline__ static const char* s_src(const Args& a, int n, int) {
    return reinterpret_cast<const char*>(a.scales + (n & ~1));  // the aligned pair of columns (N is even)
  }
  __device__ __forceinline__ static int64_t s_offset(const Args& a, int ks) { return (int64_t)ks * a.N * 2; }
  // p = the 4 staged bytes of the lane's column; columns are staged 4 bytes apart from an 8-byte
  // aligned base, so bit 2 of the address is the parity of the column
  __device__ __forceinline__ static Scale read_scale(const unsigned char* p, int) {
    const half2_t pair = *reinterpret_cast<const half2_t*>(p);
    const half_t s = (reinterpret_cast<uintptr_t>(p) & 4) ? pair.y : pair.x;
    return Scale{s, s};
  }
  __device__ __forceinline__ static Scale const_scale(const Args& a, int n) {
    const half_t s = a.scales[n];
    return Scale{s, s};
  }
  __device__ __forceinline__ static void read(Frag& f, const unsigned char* bslot, int n_local, int lh) {
    if (NBIT == 8) {
      const unsigned char* p = bslot + ((n_local >> 1) * 8 + (n_local & 1) * 4 + 2 * lh) * 16;
      f.w[0] = *reinterpret_cast<const uint4_t*>(p);
      f.w[NBIT == 8 ? 1 : 0] = *reinterpret_cast<const uint4_t*>(p + 16);
    } else {
      f.w[0] = *reinterpret_cast<const uint4_t*>(bslot + ((n_local >> 2) * 8 + (n_local & 3) * 2 + lh) * 16);
    }
  }
  // int8: piece kk/2 holds 16 k; word j of it holds k = 2j, 2j+1 (bytes 0, 2) and 2j+8, 2j+9 (bytes 1, 3).
  // int4: word j holds k = 2j + 8i, 2j + 8i + 1 in nibbles i, i + 4.
  __device__ __forceinline__ static uint32_t pair_bits(const Frag& f, int kk, int j) {
    if (NBIT == 8) {
      const uint4_t& p = f.w[NBIT == 8 ? (kk >> 1) : 0];
      const uint32_t word = j == 0 ? p.x : j == 1 ? p.y : j == 2 ? p.z : p.w;
      return __builtin_amdgcn_perm(0x64646464u, word, (kk & 1) ? 0x04030401u : 0x04020400u);  // 1024 + u8
    }
    const uint32_t word = j == 0 ? f.w[0].x : j == 1 ? f.w[0].y : j == 2 ? f.w[0].z : f.w[0].w;
    return and_or(word >> (4 * kk), 0x000F000Fu, 0x64006400u);                                // 1024 + u4
  }
  __device__ __forceinline__ static half2_t pair_finish(uint32_t bits, half2_t s2) {
    const half_t o = (half_t)(NBIT == 8 ? 1152.0f : 1032.0f);  // 1024 + the bias of the stored codes
    return (as_half2(bits) - half2_t{o, o}) * s2;
  }
  __device__ __forceinline__ static half2_t pair(const Frag& f, int kk, int j, half2_t s2) { return pair_finish(pair_bits(f, kk, j), s2); }
};

template <int NBIT, bool GROUPED>
static int intb_gemm_lds(int cfg, const char* who, const int8_t* B, const uint16_t* scales, const uint16_t* A,
                         uint16_t* C, const IntbGemmEpilogue& gep, int64_t m, int64_t n, int64_t k,
                         hipStream_t stream) {
  using P = IntbLdsPolicy<NBIT, GROUPED>;
  const typename P::Args largs{(const uint4_t*)B, (const half_t*)scales, (int)n};
  switch (cfg) {
    case 11: return launch_gemm_lds<P, IntbGemmEpilogue, 8, 2, 1, 4, 1>(who, largs, A, C, gep, m, n, k, stream);
    case 12: return launch_gemm_lds<P, IntbGemmEpilogue, 4, 2, 1, 4, 2>(who, largs, A, C, gep, m, n, k, stream);
    case 17: return launch_gemm_lds<P, IntbGemmEpilogue, 4, 1, 1, 4, 2>(who, largs, A, C, gep, m, n, k, stream);
    case 18: return launch_gemm_lds<P, IntbGemmEpilogue, 8, 1, 1, 4, 1>(who, largs, A, C, gep, m, n, k, stream);
    default: return fail(WQ_EINVAL, "%s: unknown tile configuration %d", who, cfg);
  }
}

static int intb_gemm_common(const char* who, const uint16_t* A, const int8_t* B,
                            const uint16_t* scales, const uint16_t* bias, const uint16_t* residual,
                            uint16_t* C, int activation, int binary_op, int unary_op, int64_t m,
                            int64_t n, int64_t k, int64_t group_size, int64_t bias_stride,
                            int nbit, hipStream_t stream) {
  WQ_REQUIRE(nbit == 8 || nbit == 4, "%s: weight_nbit must be 8 or 4, got %d", who, nbit);
  WQ_REQUIRE(m >= 0 && n >= 0 && k >= 0, "%s: negative dimension", who);
  WQ_REQUIRE(k % 64 == 0 && n % 64 == 0, "%s: k=%lld and n=%lld must be multiples of 64", who,
             (long long)k, (long long)n);
  WQ_REQUIRE(activation >= 0 && activation <= 3, "%s: unknown activation %d", who, activation);
  WQ_REQUIRE(binary_op >= 0 && binary_op <= 2 && unary_op >= 0 && unary_op <= 1,
             "%s: unknown binary_op %d / unary_op %d", who, binary_op, unary_op);
  WQ_REQUIRE(group_size <= 0 || group_size == 64 || group_size == k,
             "%s: group_size must be 64 (fine-grained) or <= 0 / k (per column), got %lld", who,
             (long long)group_size);
  WQ_REQUIRE(bias_stride == 0 || bias_stride >= n, "%s: bias_stride %lld smaller than n", who,
             (long long)bias_stride);
  if (m == 0 || n == 0) return WQ_OK;
  WQ_REQUIRE(k > 0, "%s: k must be positive", who);
  WQ_REQUIRE(A && B && scales && C, "%s: null pointer", who);
  WQ_REQUIRE(binary_op == 0 || residual, "%s: binary_op needs a residual tensor", who);
  WQ_REQUIRE(aligned16(A) && aligned16(B), "%s: A and B must be 16-byte aligned", who);
  WQ_REQUIRE(m < (1ll << 30) && n < (1ll << 30) && k < (1ll << 30), "%s: too large", who);
  const int group = (group_size > 0 && group_size != k) ? 64 : 0;
  const IntbEpilogue ep{(const half_t*)bias, binary_op ? (const half_t*)residual : nullptr,
                        bias_stride, activation, binary_op, unary_op};
  if (wq_gemm_cfg_override() == 0) {
    // one or two rows of a wide matrix: the VALU streaming kernel; up to 64 rows: still one pass over
    // the weights, products on the matrix cores; beyond that the tiled GEMM
    // fine-grained scales whose pairs are not 4-byte aligned go to the register-staged GEMM below
    const bool small_ok = !group || (reinterpret_cast<uintptr_t>(scales) & 3u) == 0;
    // The streaming kernel gives a wavefront whole columns: with fewer than 8 wavefronts per CU (int8 with group
    // scales, or two rows: N < 8192; two rows of int4: N < 16384) the small-batch kernel, which also splits K, is
    // the faster one (int8 group-64, M = 1, K = 4096, N = 4096: 6.7 -> 5.7 us; int4, M = 2, K = 28672, N = 8192:
    // 56 -> 32 us).  One row of int4 stays: there the streaming kernel splits K itself (intb_gemv.hip).
    // (rows per wavefront forced by a test: the streaming kernel is what is asked for)
    const bool narrow = intb_gemv_wavefronts(m, n, group, nbit) < 8 * (int64_t)cu_count() && small_ok &&
                        !tuning().gemv_rows && !(nbit == 4 && m == 1);
    if (m <= 2 && !narrow) return intb_gemv_dispatch(A, B, scales, C, m, n, k, group, nbit, ep, stream);
    if (m <= WQ_SMALL_BATCH_MAX_M && small_ok)
      return intb_small_batch_dispatch(A, B, scales, C, m, n, k, group, nbit, ep, stream);
    // up to 128 rows of a small matrix: the tiled GEMM has too few tiles for 256 CUs, two passes of the
    // small-batch kernel (64 rows, then the rest) are faster: n <= 4096 (int8, k = 11008, m = 128: 70 -> 55 us;
    // k = 4096: 28.4 -> 26.9 us), and up to 96 rows of a long, moderately wide one (k = 13824, n = 5120, m = 96:
    // 88 -> 75 us; k = n = 8192: 54 -> 50 us).  Wider matrices keep the GEMM (n = 11008, k = 4096: 31 against 36 us).
    if (m <= 2 * WQ_SMALL_BATCH_MAX_M && small_ok && (n <= 4096 || (m <= 96 && n <= 8192 && k >= 8192))) {
      const int64_t m0 = WQ_SMALL_BATCH_MAX_M;
      if (int rc = intb_small_batch_dispatch(A, B, scales, C, m0, n, k, group, nbit, ep, stream)) return rc;
      IntbEpilogue ep2 = ep;
      if (ep2.bias && ep2.bias_stride) ep2.bias += m0 * ep2.bias_stride;
      if (ep2.residual) ep2.residual += m0 * n;
      return intb_small_batch_dispatch(A + m0 * k, B, scales, C + m0 * n, m - m0, n, k, group, nbit, ep2, stream);
    }
  }
  const IntbGemmEpilogue gep{ep, (int)n};
  // the fully LDS-staged kernel under the tile shape (11, 17 or 18) whose rounds of the machine come out
  // shortest; fine-grained scales whose pairs are not 4-byte aligned: the register-staged kernel (1..4).
  // silu / gelu run the element-wise epilogue, whose inlined exp / erf code does not fit next to the 256
  // accumulator registers of the 256x256 tile (11): they choose between the other two
  const bool lds_ok = !group || (reinterpret_cast<uintptr_t>(scales) & 3u) == 0;
  int cfg = wq_gemm_cfg_override();
  if (!cfg && !lds_ok) cfg = choose_gemm_cfg(m, n, false);
  if (!cfg) {
    double best = 0;
    for (int c : {17, 18, 11}) {
      if (c == 11 && activation >= WQ_ACT_SILU) continue;
      const double t = lds_cfg_cost(c, m, n, cu_count());
      if (!cfg || t < best) cfg = c, best = t;
    }
  }
  if (cfg >= 11 && lds_ok) {
    if (group)
      return nbit == 8 ? intb_gemm_lds<8, true>(cfg, who, B, scales, A, C, gep, m, n, k, stream)
                       : intb_gemm_lds<4, true>(cfg, who, B, scales, A, C, gep, m, n, k, stream);
    return nbit == 8 ? intb_gemm_lds<8, false>(cfg, who, B, scales, A, C, gep, m, n, k, stream)
                     : intb_gemm_lds<4, false>(cfg, who, B, scales, A, C, gep, m, n, k, stream);
  }
  if (cfg >= 11) cfg = cfg == 17 ? 4 : cfg == 11 ? 1 : 2;
  if (nbit == 8) {
    const IntbLoader<8>::Args bargs{(const uint4_t*)B, (const half_t*)scales, group};
    return launch_mfma_gemm_cfg<IntbLoader<8>, IntbGemmEpilogue>(cfg, who, bargs, A, C, gep, m, n, k, stream);
  }
  const IntbLoader<4>::Args bargs{(const uint4_t*)B, (const half_t*)scales, group};
  return launch_mfma_gemm_cfg<IntbLoader<4>, IntbGemmEpilogue>(cfg, who, bargs, A, C, gep, m, n, k, stream);
}

}  // namespace wq

extern "C" int wq_fpA_intB_gemm(const uint16_t* A, const int8_t* B, const uint16_t* scales,
                                const uint16_t* bias, uint16_t* C, int activation, int64_t m,
                                int64_t n, int64_t k, int64_t group_size, int64_t bias_stride,
                                int weight_nbit, void* /*workspace*/, size_t /*workspace_bytes*/,
                                wq_stream_t stream) {
  return wq::intb_gemm_common("wq_fpA_intB_gemm", A, B, scales, bias, nullptr, C, activation,
                              WQ_BIN_NONE, WQ_UN_IDENTITY, m, n, k, group_size, bias_stride,
                              weight_nbit, (hipStream_t)stream);
}

extern "C" int wq_fpA_intB_gemm_residual(const uint16_t* A, const int8_t* B, const uint16_t* scales,
                                         const uint16_t* bias, const uint16_t* residual,
                                         uint16_t* C, int activation, int binary_op, int unary_op,
                                         int64_t m, int64_t n, int64_t k, int64_t group_size,
                                         int weight_nbit, void* /*workspace*/,
                                         size_t /*workspace_bytes*/, wq_stream_t stream) {
  if (!residual)
    return wq::fail(WQ_EINVAL, "wq_fpA_intB_gemm_residual: residual must not be null");
  if (binary_op != WQ_BIN_PLUS && binary_op != WQ_BIN_MULTIPLY)
    return wq::fail(WQ_EINVAL, "wq_fpA_intB_gemm_residual: binary_op must be plus or multiply");
  return wq::intb_gemm_common("wq_fpA_intB_gemm_residual", A, B, scales, bias, residual, C,
                              activation, binary_op, unary_op, m, n, k, group_size, 0, weight_nbit,
                              (hipStream_t)stream);
}
