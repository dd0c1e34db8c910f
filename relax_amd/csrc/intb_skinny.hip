// Format B (fpA_intB) small-batch path: the shared small-batch kernel with the
// weight policies of the preprocessed int8 / int4 layouts.
#include "intb_common.h"
#include "skinny_gemm.h"

namespace wq {

// Preprocessed layouts, in 16-byte units (K-tile = 64 k):
//   int8: unit ((n/2)*(K/64) + tile)*8 + (n%2)*4 + 2h + p   holds k = 64*tile + 32h + 16p + {2j + {0,1,8,9}}
//         in word j, bytes {0,2,1,3}
//   int4: unit ((n/4)*(K/64) + tile)*8 + (n%4)*2 + h         holds k = 64*tile + 32h + {2j + 8i + {0,1}}
//         in word j, nibbles {i, i+4}
// so the 32 codes at k0 (k0 % 32 == 0) are 32 resp. 16 contiguous bytes.
template <int NBIT, bool GROUPED>
struct IntbSkinnyPolicy {
  static constexpr int kPieces = NBIT == 8 ? 2 : 1;
  static constexpr bool kScaleDma = GROUPED;
  static constexpr bool kCanScaleBlock = false;
  struct Args {
    const uint4_t* B;
    const half_t* scales;
  };
  struct Lane {
    const uint4_t* w;   // unit of (tile 0, h 0) of this lane's column
    const half_t* s;    // &scales[n & ~1] (grouped) or &scales[n]
    int N;
    int odd;
  };
  __device__ __forceinline__ static void init(Lane& l, const Args& a, int n, int K, int N) {
    constexpr int I = NBIT == 8 ? 2 : 4;
    l.w = a.B + ((int64_t)(n / I) * (K >> 6)) * 8 + (n % I) * (8 / I);
    l.s = a.scales + (GROUPED ? (n & ~1) : n);
    l.N = N;
    l.odd = n & 1;
  }
  __device__ __forceinline__ static const char* w_addr(const Lane& l, int k0, int p) {
    return reinterpret_cast<const char*>(l.w + (int64_t)(k0 >> 6) * 8 + ((k0 >> 5) & 1) * kPieces + p);
  }
  // fine-grained scales are [K/64, N]: the pair (n & ~1, n | 1) of the lane's K-tile
  __device__ __forceinline__ static const char* s_addr(const Lane& l, int k0) {
    return reinterpret_cast<const char*>(l.s + (int64_t)(k0 >> 6) * l.N);
  }
  __device__ __forceinline__ static const char* s_pair_addr(const Lane& l, int k0) {
    if (GROUPED) return s_addr(l, k0);
    return reinterpret_cast<const char*>(reinterpret_cast<uintptr_t>(l.s) & ~(uintptr_t)3);  // &scales[n & ~1]
  }
  static bool pair_aligned(const Args& a) { return (reinterpret_cast<uintptr_t>(a.scales) & 3u) == 0; }
  __device__ __forceinline__ static half_t pick_scale(const Lane& l, half2_t pair, int) { return l.odd ? pair.y : pair.x; }
  using Scale = half_t;
  __device__ __forceinline__ static half_t const_scale(const Lane& l) { return l.s[0]; }
  __device__ __forceinline__ static half_t null_scale() { return (half_t)0.0f; }
  __device__ __forceinline__ static void dequant(const uint4_t* pieces, half_t s, half8_t out[4]) {
    const half2_t s2 = {s, s};
    if (NBIT == 8) {
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const uint32_t w[4] = {pieces[p].x, pieces[p].y, pieces[p].z, pieces[p].w};
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
      const uint32_t w[4] = {pieces[0].x, pieces[0].y, pieces[0].z, pieces[0].w};
      half2_t d[4][4];  // d[j][i] = (k = 2j+8i, 2j+8i+1)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u4_word_minus8(w[j], d[j]);
#pragma unroll
        for (int i = 0; i < 4; ++i) d[j][i] = d[j][i] * s2;
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
        out[t] = half8_t{d[0][t].x, d[0][t].y, d[1][t].x, d[1][t].y, d[2][t].x, d[2][t].y, d[3][t].x, d[3][t].y};
    }
  }
};

template <int NBIT, bool GROUPED>
static int intb_small_batch_t(const uint16_t* A, const int8_t* B, const uint16_t* scales, uint16_t* C,
                              int64_t m, int64_t n, int64_t k, const IntbEpilogue& ep, hipStream_t stream) {
  using Policy = IntbSkinnyPolicy<NBIT, GROUPED>;
  const typename Policy::Args pargs{(const uint4_t*)B, (const half_t*)scales};
  const IntbGemmEpilogue gep{ep, (int)n};
  return launch_skinny_auto<Policy, IntbGemmEpilogue>("wq_fpA_intB_gemm(small batch)", pargs, A, C, gep, m, n,
                                                      k, stream);
}

int intb_small_batch_dispatch(const uint16_t* A, const int8_t* B, const uint16_t* scales, uint16_t* C,
                              int64_t m, int64_t n, int64_t k, int64_t group, int nbit,
                              const IntbEpilogue& ep, hipStream_t stream) {
  WQ_REQUIRE(m >= 1 && m <= WQ_SMALL_BATCH_MAX_M, "wq_fpA_intB_gemm(small batch): m out of range");
  WQ_REQUIRE((reinterpret_cast<uintptr_t>(scales) & 3u) == 0 || !group,
             "wq_fpA_intB_gemm: fine-grained scales must be 4-byte aligned");
  if (nbit == 8)
    return group ? intb_small_batch_t<8, true>(A, B, scales, C, m, n, k, ep, stream)
                 : intb_small_batch_t<8, false>(A, B, scales, C, m, n, k, ep, stream);
  return group ? intb_small_batch_t<4, true>(A, B, scales, C, m, n, k, ep, stream)
               : intb_small_batch_t<4, false>(A, B, scales, C, m, n, k, ep, stream);
}

}  // namespace wq
