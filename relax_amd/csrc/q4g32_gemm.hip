// Format A prefill GEMM: y[m,n] = sum_k x[m,k] * ((code[n,k] - 7) * S[n,k/32]).
// The kernel is the shared MFMA GEMM (mfma_gemm.h); this file supplies the weight
// loader for the q4f16_1 layout and the epilogue of the reference's prefill
// PrimFunc (tests/python/dlight/test_gpu_matmul.py:378-401).
#include "mfma_gemm.h"
#include "q4g32_common.h"
#include "mfma_gemm_lds.h"

namespace wq {

// Lane (j, h) of a K-step needs k = 32h..32h+31 of weight row n: exactly one scale
// group, i.e. 4 consecutive words (16 bytes) of W and one scale; word kk is the
// B operand of MFMA kk.
struct Q4G32Loader {
  static constexpr bool kPairA = true;  // q4_word_dequant yields the (i, i+4) pairing
  struct Args {
    const uint32_t* W;
    const half_t* S;
  };
  struct Lane {
    const uint4_t* w;
    const half_t* s;
  };
  struct Frag {
    uint4_t w;
    half_t s;
  };
  __device__ __forceinline__ static void init(Lane& l, const Args& a, int n, int lh, int K, int) {
    l.w = reinterpret_cast<const uint4_t*>(a.W + (int64_t)n * (K >> 3)) + lh;
    l.s = a.S + (int64_t)n * (K >> 5) + lh;
  }
  __device__ __forceinline__ static void load(Frag& f, const Lane& l, const Args&, int ks, int lh, int K,
                              bool ktail) {
    if (ktail && (ks * 2 + lh) >= (K >> 5)) {  // the last step may hold a single group
      f.w = uint4_t{0x77777777u, 0x77777777u, 0x77777777u, 0x77777777u};  // code 7 -> weight 0
      f.s = (half_t)0.0f;
    } else {
      f.w = l.w[ks * 2];
      f.s = l.s[ks * 2];
    }
  }
  __device__ __forceinline__ static void dequant(const Frag& f, half8_t out[4]) {
    const half2_t s2 = {f.s, f.s};
    const uint32_t ws[4] = {f.w.x, f.w.y, f.w.z, f.w.w};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      half2_t d[4];
      q4_word_dequant(ws[kk], s2, d);
      out[kk] = half8_t{d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
    }
  }
};


// Weight policy of the fully LDS-staged kernel (mfma_gemm_lds.h) for format A: per K-step a
// column is 32 bytes of codes (chunk (n, h) of the B tile = 16 bytes = one scale group) and two
// scales (4 bytes, staged in LDS with the codes).
struct Q4G32LdsPolicy {
  static constexpr bool kFineTail = true;  // a last round of few tiles may be cut into eight row slices
  static constexpr int kColBytes = 32;
  static constexpr int kScaleBytes = 4;
  static constexpr int kStepStride = 32;
  struct Args {
    const uint32_t* W;
    const half_t* S;
  };
  struct Frag {
    uint4_t w;
  };
  using Scale = half2_t;  // the group's scale, twice
  __device__ __forceinline__ static const char* b_src(const Args& a, int n0, int q, int N, int K) {
    const int n = q >> 1, h = q & 1;
    return reinterpret_cast<const char*>(a.W + (int64_t)min(n0 + n, N - 1) * (K >> 3)) + h * 16;
  }
  __device__ __forceinline__ static const char* s_src(const Args& a, int n, int K) {
    return reinterpret_cast<const char*>(a.S + (int64_t)n * (K >> 5));
  }
  __device__ __forceinline__ static int64_t s_offset(const Args&, int ks) { return (int64_t)ks * 4; }
  __device__ __forceinline__ static Scale read_scale(const unsigned char* p, int lh) {
    const half_t s = *reinterpret_cast<const half_t*>(p + lh * 2);
    return Scale{s, s};
  }
  __device__ __forceinline__ static Scale const_scale(const Args&, int) { return Scale{(half_t)0.0f, (half_t)0.0f}; }
  __device__ __forceinline__ static void read(Frag& f, const unsigned char* bslot, int n_local, int lh) {
    f.w = *reinterpret_cast<const uint4_t*>(bslot + (n_local * 2 + lh) * 16);
  }
  __device__ __forceinline__ static uint32_t pair_bits(const Frag& f, int kk, int j) {
    const uint32_t word = kk == 0 ? f.w.x : kk == 1 ? f.w.y : kk == 2 ? f.w.z : f.w.w;
    return q4_pair_bits_natural(word, j);
  }
  __device__ __forceinline__ static half2_t pair_finish(uint32_t bits, half2_t s2) {
    const half2_t off = {(half_t)1031.0f, (half_t)1031.0f};
    return (as_half2(bits) - off) * s2;
  }
  __device__ __forceinline__ static half2_t pair(const Frag& f, int kk, int j, half2_t s2) { return pair_finish(pair_bits(f, kk, j), s2); }
};

}  // namespace wq

// Tile shape override for measurement (0 = choose from the problem shape).
int wq_gemm_cfg_override() { return wq::tuning().gemm_cfg; }

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
  int cfg = tuning().gemm_cfg ? tuning().gemm_cfg : choose_q4_lds_cfg(M, N, cu_count());
  const Q4G32Loader::Args bargs{W, (const half_t*)S};
  const Q4G32LdsPolicy::Args largs{W, (const half_t*)S};
  const Q4G32Epilogue ep{(const half_t*)bias, (const half_t*)residual, (int)N};
  // 11..18: the fully LDS-staged kernel (needs K % 64 == 0 and 4-byte aligned scale pairs)
  if (cfg >= 11 && K % 64 == 0 && ((uintptr_t)S & 3u) == 0) {
    switch (cfg) {
      case 11: return launch_gemm_lds<Q4G32LdsPolicy, Q4G32Epilogue, 8, 2, 1, 4, 1>("wq_q4g32_gemm", largs, x, y, ep, M, N, K, stream);
      case 12: return launch_gemm_lds<Q4G32LdsPolicy, Q4G32Epilogue, 4, 2, 1, 4, 2>("wq_q4g32_gemm", largs, x, y, ep, M, N, K, stream);
      case 13: return launch_gemm_lds<Q4G32LdsPolicy, Q4G32Epilogue, 4, 2, 2, 2, 2>("wq_q4g32_gemm", largs, x, y, ep, M, N, K, stream);
      case 14: return launch_gemm_lds<Q4G32LdsPolicy, Q4G32Epilogue, 4, 4, 2, 2, 1>("wq_q4g32_gemm", largs, x, y, ep, M, N, K, stream);
      case 17: return launch_gemm_lds<Q4G32LdsPolicy, Q4G32Epilogue, 4, 1, 1, 4, 2>("wq_q4g32_gemm", largs, x, y, ep, M, N, K, stream);
      case 18: return launch_gemm_lds<Q4G32LdsPolicy, Q4G32Epilogue, 8, 1, 1, 4, 1>("wq_q4g32_gemm", largs, x, y, ep, M, N, K, stream);
      default: return fail(WQ_EINVAL, "wq_q4g32_gemm: unknown tile configuration %d", cfg);
    }
  }
  if (cfg >= 11) cfg = cfg == 17 ? 4 : (cfg == 11 || cfg == 14) ? 1 : 2;  // 12, 13, 18 -> 128 x 256  // not eligible: register-staged kernel, same tile
  return launch_mfma_gemm_cfg<Q4G32Loader, Q4G32Epilogue>(cfg, "wq_q4g32_gemm", bargs, x, y, ep, M,
                                                          N, K, stream);
}
