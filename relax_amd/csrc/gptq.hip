// AutoGPTQ checkpoints: K-major int4 codes with packed zero points and a group index
// (tests/python/dlight/test_gpu_gemv.py:636-665):
//   qweight uint32 [K/8, N], qzeros uint32 [G, N/8], scales fp16 [G, N], g_idx int32 [K]
//   w[k,n] = (fp16(code) - (fp16(zero) + 1)) * scales[g_idx[k], n],   y = residual + x . w
//
// The reference's GEMV rule leaves this function unscheduled because the scale depends on k
// through g_idx.  Here the dependence is removed once, when the checkpoint is loaded:
//   * the K rows are sorted by group (stable), so that every group is a run of K/G
//     consecutive rows; `perm` records the order and the activations are gathered through it
//     by a small kernel in front of the linear (one pass over x instead of one per workgroup);
//   * the words are transposed to the [N, K/8] layout of the other kernels of this library
//     (a word holds 8 consecutive k of one column in both layouts);
//   * scale and zero point + 1 are interleaved as fp16 pairs SZ [N, G, 2], the 4 bytes that
//     one lane needs for one group.
// After that the weight stream is the one of format A with one more multiply-add per group,
// and the streaming GEMV (q4_gemv.h), the small-batch kernel (skinny_gemm.h) and the MFMA GEMM
// (mfma_gemm_lds.h) all take it.
// A g_idx whose groups do not all have K/G members is rejected by the preparation.
#include <mutex>
#include <vector>

#include "mfma_gemm.h"
#include "mfma_gemm_lds.h"
#include "q4_gemv.h"
#include "q4g32_common.h"
#include "skinny_gemm.h"

namespace wq {

// ---- the reference's decode, bit for bit, from the checkpoint layout --------------------
// Thread (kw, n) unpacks the 8 codes of one word: reads coalesced along n, writes 8 rows.
__global__ __launch_bounds__(256) void gptq_dequant_kernel(const uint32_t* __restrict__ qweight,
                                                           const uint32_t* __restrict__ qzeros,
                                                           const half_t* __restrict__ scales,
                                                           const int* __restrict__ g_idx, half_t* __restrict__ out,
                                                           int K, int N, int G) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int kw = blockIdx.y;
  if (n >= N) return;
  const uint32_t word = qweight[(int64_t)kw * N + n];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int k = kw * 8 + i;
    const int g = min(max(g_idx[k], 0), G - 1);  // entries outside [0, G) are clamped, never followed
    const uint32_t zero = (qzeros[(int64_t)g * (N >> 3) + (n >> 3)] >> (4 * (n & 7))) & 15u;
    const half_t zp = (half_t)(float)zero + (half_t)1.0f;
    const half_t code = (half_t)(float)((word >> (4 * i)) & 15u);
    out[(int64_t)k * N + n] = (code - zp) * scales[(int64_t)g * N + n];
  }
}

// ---- preparation ---------------------------------------------------------------------------
// One thread per group scans g_idx in ascending k and lists the group's rows.  status bit 0:
// some group does not have exactly `gs` members (this also catches entries outside [0, G));
// bit 1: the order differs from 0, 1, 2, ...
__global__ __launch_bounds__(64) void gptq_perm_kernel(const int* __restrict__ g_idx, int* __restrict__ perm,
                                                       int* __restrict__ status, int K, int G, int gs) {
  const int g = blockIdx.x * 64 + threadIdx.x;
  if (g >= G) return;
  int count = 0, flags = 0;
  for (int k = 0; k < K; ++k) {
    if (g_idx[k] == g) {
      if (count < gs) {
        perm[g * gs + count] = k;
        if (k != g * gs + count) flags |= 2;
      }
      ++count;
    }
  }
  if (count != gs) flags |= 1;
  if (flags) atomicOr(status, flags);
}

// W_nk[n][kw'] = the 8 codes of column n at rows perm[8kw' .. 8kw'+7]; 64x64 word tiles through
// LDS: reads coalesced along n, writes coalesced along kw'.
__global__ __launch_bounds__(256) void gptq_repack_kernel(const uint32_t* __restrict__ qweight,
                                                          const int* __restrict__ perm, uint32_t* __restrict__ W_nk,
                                                          int KW, int N) {
  __shared__ uint32_t tile[64][65];
  const int kw0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = 0; i < 16; ++i) {
    const int kw = kw0 + ty * 16 + i, n = n0 + tx;
    if (kw < KW && n < N) {
      uint32_t word = 0;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int k = perm[kw * 8 + c];
        word |= ((qweight[(int64_t)(k >> 3) * N + n] >> (4 * (k & 7))) & 15u) << (4 * c);
      }
      tile[ty * 16 + i][tx] = word;
    }
  }
  __syncthreads();
  for (int i = 0; i < 16; ++i) {
    const int n = n0 + ty * 16 + i, kw = kw0 + tx;
    if (kw < KW && n < N) W_nk[(int64_t)n * KW + kw] = tile[tx][ty * 16 + i];
  }
}

// SZ[n][g] = (scales[g][n], fp16(zero[g][n] + 1))
__global__ __launch_bounds__(256) void gptq_sz_kernel(const uint32_t* __restrict__ qzeros,
                                                      const half_t* __restrict__ scales, half2_t* __restrict__ SZ,
                                                      int N, int G) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int g = blockIdx.y;
  if (n >= N) return;
  const uint32_t zero = (qzeros[(int64_t)g * (N >> 3) + (n >> 3)] >> (4 * (n & 7))) & 15u;
  SZ[(int64_t)n * G + g] = half2_t{scales[(int64_t)g * N + n], (half_t)(float)(zero + 1u)};
}

// xp[m][k'] = x[m][perm[k']]: one row per workgroup, read coalesced into LDS, gathered from there
// (K <= 32768: 64 KiB), written coalesced as pairs.
__global__ __launch_bounds__(256) void gptq_gather_x_kernel(const half_t* __restrict__ x, const int* __restrict__ perm,
                                                            half_t* __restrict__ xp, int K) {
  extern __shared__ uint4_t gather_smem[];
  half_t* row = reinterpret_cast<half_t*>(gather_smem);
  const int64_t m = blockIdx.x;
  const uint4_t* src = reinterpret_cast<const uint4_t*>(x + m * K);
  for (int i = threadIdx.x; i < (K >> 3); i += 256) gather_smem[i] = src[i];
  __syncthreads();
  half2_t* dst = reinterpret_cast<half2_t*>(xp + m * K);
  const int2* p2 = reinterpret_cast<const int2*>(perm);
  for (int i = threadIdx.x; i < (K >> 1); i += 256) {
    const int2 p = p2[i];
    dst[i] = half2_t{row[p.x], row[p.y]};
  }
}

// The same for a few rows: thread per output pair, straight from global memory.
__global__ __launch_bounds__(256) void gptq_gather_x_direct_kernel(const half_t* __restrict__ x,
                                                                   const int* __restrict__ perm,
                                                                   half_t* __restrict__ xp, int K) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (i < (K >> 1)) {
    const int2 p = reinterpret_cast<const int2*>(perm)[i];
    reinterpret_cast<half2_t*>(xp + m * K)[i] = half2_t{x[m * K + p.x], x[m * K + p.y]};
  }
}

// ---- any g_idx: groups of unequal size ------------------------------------------------------
// The rows of a group, in ascending k, are padded to a multiple of 32 and the whole layer becomes
// K' / 32 sub-groups of exactly 32 rows (sub-group -> group map `sub2grp`); perm'[k'] is the row of
// the checkpoint at position k', or -1 for padding.  Padding contributes nothing because its
// ACTIVATION is gathered as zero (a zero weight cannot be encoded when zero + 1 = 16).
__global__ __launch_bounds__(256) void gptq_repack_padded_kernel(const uint32_t* __restrict__ qweight,
                                                                 const int* __restrict__ perm,
                                                                 uint32_t* __restrict__ W_nk, int KW, int N) {
  __shared__ uint32_t tile[64][65];
  const int kw0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = 0; i < 16; ++i) {
    const int kw = kw0 + ty * 16 + i, n = n0 + tx;
    if (kw < KW && n < N) {
      uint32_t word = 0;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int k = perm[kw * 8 + c];
        if (k >= 0) word |= ((qweight[(int64_t)(k >> 3) * N + n] >> (4 * (k & 7))) & 15u) << (4 * c);
      }
      tile[ty * 16 + i][tx] = word;
    }
  }
  __syncthreads();
  for (int i = 0; i < 16; ++i) {
    const int n = n0 + ty * 16 + i, kw = kw0 + tx;
    if (kw < KW && n < N) W_nk[(int64_t)n * KW + kw] = tile[tx][ty * 16 + i];
  }
}

// SZ[n][sub] = (scales[g][n], fp16(zero[g][n] + 1)) with g = sub2grp[sub]
__global__ __launch_bounds__(256) void gptq_sz_mapped_kernel(const uint32_t* __restrict__ qzeros,
                                                             const half_t* __restrict__ scales,
                                                             const int* __restrict__ sub2grp,
                                                             half2_t* __restrict__ SZ, int N, int GS) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int sub = blockIdx.y;
  if (n >= N) return;
  const int g = sub2grp[sub];
  const uint32_t zero = (qzeros[(int64_t)g * (N >> 3) + (n >> 3)] >> (4 * (n & 7))) & 15u;
  SZ[(int64_t)n * GS + sub] = half2_t{scales[(int64_t)g * N + n], (half_t)(float)(zero + 1u)};
}

// xp[m][k'] = perm'[k'] >= 0 ? x[m][perm'[k']] : 0; rows of x are K long, rows of xp KP
__global__ __launch_bounds__(256) void gptq_gather_x_padded_kernel(const half_t* __restrict__ x,
                                                                   const int* __restrict__ perm,
                                                                   half_t* __restrict__ xp, int K, int KP) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (i < (KP >> 1)) {
    const int2 p = reinterpret_cast<const int2*>(perm)[i];
    const half_t zero = (half_t)0.0f;
    // (an index beyond the row of x, from operands prepared for another K, reads nothing: it gathers a zero)
    reinterpret_cast<half2_t*>(xp + m * KP)[i] =
        half2_t{(unsigned)p.x < (unsigned)K ? x[m * K + p.x] : zero, (unsigned)p.y < (unsigned)K ? x[m * K + p.y] : zero};
  }
}

// ---- small-batch policy: format A's stream with the (scale, zero point) pair of the lane's group ----
struct GptqSkinnyPolicy {
  static constexpr int kPieces = 1;
  static constexpr bool kScaleDma = true;
  static constexpr bool kCanScaleBlock = false;
  struct Args {
    const uint32_t* W;
    const half2_t* SZ;
    int groups;    // per row
    int ratio;     // 32-code groups per scale group
    uint32_t inv;  // ceil(2^32 / ratio), unused when ratio == 1
  };
  struct Lane {
    const char* w;
    const char* sz;
    int ratio;
    uint32_t inv;
  };
  using Scale = half2_t;  // (scale, zero point)
  __device__ __forceinline__ static void init(Lane& l, const Args& a, int n, int K, int) {
    l.w = reinterpret_cast<const char*>(a.W + (int64_t)n * (K >> 3));
    l.sz = reinterpret_cast<const char*>(a.SZ + (int64_t)n * a.groups);
    l.ratio = a.ratio;
    l.inv = a.inv;
  }
  __device__ __forceinline__ static const char* w_addr(const Lane& l, int k0, int) { return l.w + (k0 >> 1); }
  __device__ __forceinline__ static const char* s_addr(const Lane& l, int k0) {
    const uint32_t g32 = (uint32_t)k0 >> 5;
    return l.sz + (l.ratio == 1 ? g32 : __umulhi(g32, l.inv)) * 4;
  }
  __device__ __forceinline__ static const char* s_pair_addr(const Lane& l, int k0) { return s_addr(l, k0); }
  static bool pair_aligned(const Args&) { return true; }
  __device__ __forceinline__ static Scale pick_scale(const Lane&, half2_t pair, int) { return pair; }
  __device__ __forceinline__ static Scale const_scale(const Lane&) { return Scale{}; }
  __device__ __forceinline__ static Scale null_scale() { return Scale{(half_t)0.0f, (half_t)0.0f}; }
  __device__ __forceinline__ static void dequant(const uint4_t* pieces, Scale sz, half8_t out[4]) {
    const half2_t s2 = {sz.x, sz.x};
    const half_t o = sz.y + (half_t)1024.0f;
    const half2_t off = {o, o};
    const uint32_t words[4] = {pieces[0].x, pieces[0].y, pieces[0].z, pieces[0].w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      half2_t d[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t b = (words[t] >> (8 * j)) & 0xFFu;  // codes 2j, 2j+1
        const uint32_t u = (b << 12) | b;
        d[j] = (as_half2(and_or(u, 0x000F000Fu, 0x64006400u)) - off) * s2;
      }
      out[t] = half8_t{d[0].x, d[0].y, d[1].x, d[1].y, d[2].x, d[2].y, d[3].x, d[3].y};
    }
  }
};

// ---- MFMA GEMM policy: the stream of format A with a (scale, zero point) pair per group ------
// A K-step (64 rows) lies inside one group (group size % 64 == 0), so both lane halves read the
// same 4 staged bytes.  1024 + code - (1024 + zp) is exact, the multiply rounds once: the
// reference's fp16 weight, bit for bit.
struct GptqLdsPolicy {
  static constexpr int kColBytes = 32;
  static constexpr int kScaleBytes = 4;
  static constexpr int kStepStride = 32;
  struct Args {
    const uint32_t* W;
    const half2_t* SZ;
    int groups;          // per row
    int steps_per_group; // group size / 64
    uint32_t inv;        // ceil(2^32 / steps_per_group), unused when steps_per_group == 1
  };
  struct Frag {
    uint4_t w;
  };
  struct Scale {
    half2_t s2;   // scale, twice
    half2_t off;  // 1024 + zero point, twice
  };
  __device__ __forceinline__ static const char* b_src(const Args& a, int n0, int q, int N, int K) {
    const int n = q >> 1, h = q & 1;
    return reinterpret_cast<const char*>(a.W + (int64_t)min(n0 + n, N - 1) * (K >> 3)) + h * 16;
  }
  __device__ __forceinline__ static const char* s_src(const Args& a, int n, int) {
    return reinterpret_cast<const char*>(a.SZ + (int64_t)n * a.groups);
  }
  // ks / steps_per_group by multiplication: exact for ks * steps_per_group < 2^32
  __device__ __forceinline__ static int64_t s_offset(const Args& a, int ks) {
    const uint32_t g = a.steps_per_group == 1 ? (uint32_t)ks : __umulhi((uint32_t)ks, a.inv);
    return (int64_t)g * 4;
  }
  __device__ __forceinline__ static Scale read_scale(const unsigned char* p, int) {
    const half2_t sz = *reinterpret_cast<const half2_t*>(p);
    const half_t o = sz.y + (half_t)1024.0f;
    return Scale{half2_t{sz.x, sz.x}, half2_t{o, o}};
  }
  __device__ __forceinline__ static Scale const_scale(const Args&, int) { return Scale{}; }
  __device__ __forceinline__ static void read(Frag& f, const unsigned char* bslot, int n_local, int lh) {
    f.w = *reinterpret_cast<const uint4_t*>(bslot + (n_local * 2 + lh) * 16);
  }
  __device__ __forceinline__ static uint32_t pair_bits(const Frag& f, int kk, int j) {
    const uint32_t word = kk == 0 ? f.w.x : kk == 1 ? f.w.y : kk == 2 ? f.w.z : f.w.w;
    return q4_pair_bits_natural(word, j);
  }
  __device__ __forceinline__ static half2_t pair_finish(uint32_t bits, const Scale& sc) { return (as_half2(bits) - sc.off) * sc.s2; }
  __device__ __forceinline__ static half2_t pair(const Frag& f, int kk, int j, const Scale& sc) {
    return pair_finish(pair_bits(f, kk, j), sc);
  }
};

}  // namespace wq

extern "C" int wq_gptq_dequantize(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                                  const int32_t* g_idx, uint16_t* out, int64_t K, int64_t N, int64_t G,
                                  wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(K >= 0 && N >= 0 && G >= 0, "wq_gptq_dequantize: negative dimension");
  WQ_REQUIRE(K % 8 == 0 && N % 8 == 0, "wq_gptq_dequantize: K=%lld and N=%lld must be multiples of 8",
             (long long)K, (long long)N);
  if (K == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(G > 0, "wq_gptq_dequantize: no groups");
  WQ_REQUIRE(qweight && qzeros && scales && g_idx && out, "wq_gptq_dequantize: null pointer");
  WQ_REQUIRE(N < (1ll << 30) && K / 8 < 65536, "wq_gptq_dequantize: too large");
  WQ_LAUNCH("wq_gptq_dequantize", gptq_dequant_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)(K / 8)),
            dim3(256), 0, (hipStream_t)stream, qweight, qzeros, (const half_t*)scales, g_idx, (half_t*)out, (int)K,
            (int)N, (int)G);
  return WQ_OK;
}

extern "C" int wq_gptq_prepare(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                               const int32_t* g_idx, uint32_t* W_nk, uint16_t* SZ, int32_t* perm,
                               int32_t* status_scratch, int* needs_perm, int64_t K, int64_t N, int64_t G,
                               wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(K >= 0 && N >= 0 && G >= 0, "wq_gptq_prepare: negative dimension");
  if (needs_perm) *needs_perm = 0;
  if (K == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(G > 0 && K % G == 0, "wq_gptq_prepare: K=%lld is not a multiple of the %lld groups", (long long)K,
             (long long)G);
  const int64_t gs = K / G;
  WQ_REQUIRE(gs % 32 == 0, "wq_gptq_prepare: group size %lld must be a multiple of 32", (long long)gs);
  WQ_REQUIRE(N % 8 == 0, "wq_gptq_prepare: N=%lld must be a multiple of 8", (long long)N);
  WQ_REQUIRE(qweight && qzeros && scales && g_idx && W_nk && SZ && perm && status_scratch,
             "wq_gptq_prepare: null pointer");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 24) && G < 65536, "wq_gptq_prepare: too large");
  // the status word is cleared by a copy of a zero (a fill kernel would do as well); the
  // call synchronises anyway, it is a load-time step
  const int32_t zero = 0;
  WQ_HIP(hipMemcpyAsync(status_scratch, &zero, 4, hipMemcpyHostToDevice, stream));
  WQ_LAUNCH("wq_gptq_prepare", gptq_perm_kernel, dim3((unsigned)((G + 63) / 64)), dim3(64), 0, stream, g_idx,
            perm, status_scratch, (int)K, (int)G, (int)gs);
  int32_t status = 0;
  WQ_HIP(hipMemcpyAsync(&status, status_scratch, 4, hipMemcpyDeviceToHost, stream));
  WQ_HIP(hipStreamSynchronize(stream));
  if (status & 1)
    return fail(WQ_EUNSUPPORTED,
                "wq_gptq_prepare: g_idx must assign exactly K/G = %lld rows to each of the %lld groups",
                (long long)gs, (long long)G);
  if (needs_perm) *needs_perm = (status & 2) ? 1 : 0;
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K / 8 + 63) / 64));
  WQ_LAUNCH("wq_gptq_prepare", gptq_repack_kernel, grid, dim3(256), 0, stream, qweight, perm, W_nk, (int)(K / 8),
            (int)N);
  WQ_LAUNCH("wq_gptq_prepare", gptq_sz_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)G), dim3(256), 0, stream,
            qzeros, (const half_t*)scales, (half2_t*)SZ, (int)N, (int)G);
  return WQ_OK;
}

extern "C" int64_t wq_gptq_padded_k_bound(int64_t K, int64_t G) {
  if (K <= 0 || G <= 0) return 0;
  return (K + 31 * G + 63) / 64 * 64;
}

extern "C" int wq_gptq_prepare_padded(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                                      const int32_t* g_idx, uint32_t* W_nk, uint16_t* SZ, int32_t* perm,
                                      int64_t capacity, int64_t* K_padded, int64_t K, int64_t N, int64_t G,
                                      wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(K >= 0 && N >= 0 && G >= 0 && K_padded, "wq_gptq_prepare_padded: negative dimension or null K_padded");
  *K_padded = 0;
  if (K == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(G > 0 && K % 8 == 0 && N % 8 == 0, "wq_gptq_prepare_padded: K=%lld and N=%lld must be multiples of 8",
             (long long)K, (long long)N);
  WQ_REQUIRE(qweight && qzeros && scales && g_idx && W_nk && SZ && perm, "wq_gptq_prepare_padded: null pointer");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 24) && G < 65536, "wq_gptq_prepare_padded: too large");
  // a load-time step: the row -> group map is sorted on the host
  std::vector<int32_t> gi((size_t)K);
  WQ_HIP(hipMemcpyAsync(gi.data(), g_idx, (size_t)K * 4, hipMemcpyDeviceToHost, stream));
  WQ_HIP(hipStreamSynchronize(stream));
  std::vector<int64_t> count((size_t)G, 0);
  for (int64_t k = 0; k < K; ++k) {
    WQ_REQUIRE(gi[k] >= 0 && gi[k] < G, "wq_gptq_prepare_padded: g_idx[%lld] = %d is outside [0, %lld)", (long long)k,
               gi[k], (long long)G);
    ++count[gi[k]];
  }
  std::vector<int64_t> start((size_t)G + 1, 0);
  for (int64_t g = 0; g < G; ++g) start[g + 1] = start[g] + (count[g] + 31) / 32 * 32;
  const int64_t KP = (start[G] + 63) / 64 * 64;  // the small-batch kernel walks K in steps of 64
  WQ_REQUIRE(KP <= capacity, "wq_gptq_prepare_padded: the padded layer has %lld rows, the buffers hold %lld "
             "(wq_gptq_padded_k_bound gives the most it can be)", (long long)KP, (long long)capacity);
  std::vector<int32_t> hperm((size_t)KP, -1), sub2grp((size_t)(KP / 32), 0);
  std::vector<int64_t> fill(start.begin(), start.end() - 1);
  for (int64_t k = 0; k < K; ++k) hperm[fill[gi[k]]++] = (int32_t)k;
  for (int64_t g = 0; g < G; ++g)
    for (int64_t sub = start[g] / 32; sub < start[g + 1] / 32; ++sub) sub2grp[sub] = (int32_t)g;
  // the sub-group -> group map is only needed by the kernel below: a temporary device allocation
  int32_t* d_map = nullptr;
  WQ_HIP(hipMalloc(&d_map, sub2grp.size() * 4));
  hipError_t e = hipMemcpyAsync(perm, hperm.data(), (size_t)KP * 4, hipMemcpyHostToDevice, stream);
  if (e == hipSuccess) e = hipMemcpyAsync(d_map, sub2grp.data(), sub2grp.size() * 4, hipMemcpyHostToDevice, stream);
  if (e == hipSuccess) {
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((KP / 8 + 63) / 64));
    hipLaunchKernelGGL(gptq_repack_padded_kernel, grid, dim3(256), 0, stream, qweight, (const int*)perm, W_nk,
                       (int)(KP / 8), (int)N);
    hipLaunchKernelGGL(gptq_sz_mapped_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)(KP / 32)), dim3(256), 0,
                       stream, qzeros, (const half_t*)scales, (const int*)d_map, (half2_t*)SZ, (int)N, (int)(KP / 32));
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);  // the host vectors and d_map are in use until here
  (void)hipFree(d_map);
  if (e != hipSuccess) return fail(WQ_EDEVICE, "wq_gptq_prepare_padded: %s", hipGetErrorString(e));
  *K_padded = KP;
  return WQ_OK;
}

extern "C" size_t wq_gptq_padded_workspace_bytes(int64_t M, int64_t K_padded) {
  return (M > 0 && K_padded > 0) ? (size_t)M * (size_t)K_padded * 2 : 0;
}

extern "C" size_t wq_gptq_workspace_bytes(int64_t M, int64_t K, int has_perm) {
  return (has_perm && M > 0 && K > 0) ? (size_t)M * (size_t)K * 2 : 0;
}

namespace wq {
static int gptq_linear_impl(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                            const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                            int64_t K, int64_t G, void* workspace, size_t workspace_bytes, hipStream_t stream);
}

extern "C" int wq_gptq_linear(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                              const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                              int64_t K, int64_t G, void* workspace, size_t workspace_bytes, wq_stream_t stream) {
  return wq::gptq_linear_impl(W_nk, SZ, perm, x, bias, residual, y, M, N, K, G, workspace, workspace_bytes,
                              (hipStream_t)stream);
}

extern "C" int wq_gptq_linear_padded(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                                     const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M,
                                     int64_t N, int64_t K, int64_t K_padded, void* workspace, size_t workspace_bytes,
                                     wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && K_padded >= 0, "wq_gptq_linear_padded: negative dimension");
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0 && K_padded >= K && K_padded % 64 == 0 && K_padded <= 32768,
             "wq_gptq_linear_padded: K_padded=%lld must be a multiple of 64, at least K=%lld and at most 32768",
             (long long)K_padded, (long long)K);
  WQ_REQUIRE(W_nk && SZ && perm && x && y, "wq_gptq_linear_padded: null pointer");
  WQ_REQUIRE(aligned16(perm) && M < (1ll << 16), "wq_gptq_linear_padded: perm must be 16-byte aligned, M < 65536");
  const size_t need = wq_gptq_padded_workspace_bytes(M, K_padded);
  WQ_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
             "wq_gptq_linear_padded: needs a 16-byte aligned workspace of M*K_padded*2 = %zu bytes (got %zu)", need,
             workspace_bytes);
  WQ_LAUNCH("wq_gptq_linear_padded", gptq_gather_x_padded_kernel, dim3((unsigned)((K_padded / 2 + 255) / 256), (unsigned)M),
            dim3(256), 0, stream, (const half_t*)x, perm, (half_t*)workspace, (int)K, (int)K_padded);
  return gptq_linear_impl(W_nk, SZ, nullptr, (const uint16_t*)workspace, bias, residual, y, M, N, K_padded,
                          K_padded / 32, nullptr, 0, stream);
}

// ---- the same linear for callers that cannot allocate: the gathered activations live in a
// ---- file-scope device array instead of a caller workspace
namespace wq {

constexpr size_t kGptqScratchBytes = WQ_GPTQ_NOALLOC_MAX_BYTES;
// One copy per GPU, held until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress; kernels receive the address looked up below.
static __device__ __align__(256) unsigned char scratch[kGptqScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, looked up once per device.
static int gptq_scratch_for_current_device(void** out) {
  int dev = -1;
  WQ_HIP(hipGetDevice(&dev));
  WQ_REQUIRE(dev >= 0 && dev < kMaxDevices, "wq_gptq_linear_noalloc: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    WQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    WQ_REQUIRE(p && aligned16(p), "wq_gptq_linear_noalloc: no device address for the scratch array");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return WQ_OK;
}

}  // namespace wq

extern "C" int wq_gptq_linear_noalloc(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm,
                                      const uint16_t* x, const uint16_t* bias, const uint16_t* residual,
                                      uint16_t* y, int64_t M, int64_t N, int64_t K, int64_t G,
                                      wq_stream_t stream) {
  using namespace wq;
  void* ws = nullptr;
  size_t ws_bytes = 0;
  // (also for M = 0: the way to have the address looked up ahead of a stream capture)
  if (perm)
    if (int rc = gptq_scratch_for_current_device(&ws)) return rc;
  if (perm && M > 0 && N > 0 && K > 0) {
    WQ_REQUIRE(M < (1ll << 30) && K <= 32768, "wq_gptq_linear_noalloc: M=%lld K=%lld outside the supported range",
               (long long)M, (long long)K);
    const size_t need = (size_t)M * (size_t)K * 2;
    WQ_REQUIRE(need <= kGptqScratchBytes,
               "wq_gptq_linear_noalloc: the gathered activations need M*K*2 = %zu bytes, the built-in scratch "
               "buffer holds %zu; use wq_gptq_linear with a workspace",
               need, kGptqScratchBytes);
    ws_bytes = kGptqScratchBytes;
  }
  return gptq_linear_impl(W_nk, SZ, perm, x, bias, residual, y, M, N, K, G, ws, ws_bytes, (hipStream_t)stream);
}

static int wq::gptq_linear_impl(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                                const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                                int64_t K, int64_t G, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using namespace wq;
  WQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && G >= 0, "wq_gptq_linear: negative dimension");
  if (M == 0 || N == 0) return WQ_OK;
  WQ_REQUIRE(K > 0 && G > 0 && K % G == 0, "wq_gptq_linear: K=%lld is not a positive multiple of the %lld groups",
             (long long)K, (long long)G);
  const int64_t gs = K / G;
  WQ_REQUIRE(gs % 32 == 0, "wq_gptq_linear: group size %lld must be a multiple of 32", (long long)gs);
  WQ_REQUIRE(W_nk && SZ && x && y, "wq_gptq_linear: null pointer");
  WQ_REQUIRE(aligned16(W_nk) && aligned16(x) && aligned16(perm) && (reinterpret_cast<uintptr_t>(SZ) & 3u) == 0,
             "wq_gptq_linear: W_nk, x and perm must be 16-byte aligned, SZ 4-byte aligned");
  WQ_REQUIRE(N < (1ll << 30) && K <= 32768 && M < (1ll << 30),
             "wq_gptq_linear: N=%lld K=%lld outside the supported range (K <= 32768)", (long long)N, (long long)K);
  // a row order: gather the activations once, in front of whichever kernel runs
  if (perm) {
    const size_t need = (size_t)M * (size_t)K * 2;
    WQ_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
               "wq_gptq_linear: a row order needs a 16-byte aligned workspace of M*K*2 = %zu bytes (got %zu)", need,
               workspace_bytes);
    if (M <= 64) {  // few rows: spread each over many workgroups
      WQ_LAUNCH("wq_gptq_linear", gptq_gather_x_direct_kernel, dim3((unsigned)((K / 2 + 255) / 256), (unsigned)M),
                dim3(256), 0, stream, (const half_t*)x, perm, (half_t*)workspace, (int)K);
    } else {
      auto kern = gptq_gather_x_kernel;
      const size_t lds = (size_t)K * 2;
      if (lds > 48 * 1024) {
        static DynamicLdsLimit limit;
        WQ_HIP(limit.ensure(reinterpret_cast<const void*>(kern), (int)lds));
      }
      WQ_LAUNCH("wq_gptq_linear", kern, dim3((unsigned)M), dim3(256), lds, stream, (const half_t*)x, perm,
                (half_t*)workspace, (int)K);
    }
    x = (const uint16_t*)workspace;
  }
  const int ratio = (int)(gs / 32);
  const uint32_t inv32 = ratio > 1 ? (uint32_t)(((1ull << 32) + ratio - 1) / ratio) : 0u;
  const Q4G32Epilogue ep{(const half_t*)bias, (const half_t*)residual, (int)N};
  // (two rows of more than 8192 columns go to the small-batch kernel, as in wq_q4g32_linear)
  if (M <= 2 && !(M == 2 && K > 8192 && K % 64 == 0))
    return gemv_dispatch<true>("wq_gptq_linear", W_nk, SZ, GemvZp{ratio, (int)G}, x, bias, residual, y, M, N, K, stream);
  if (M <= WQ_SMALL_BATCH_MAX_M && K % 64 == 0) {
    const GptqSkinnyPolicy::Args pargs{W_nk, (const half2_t*)SZ, (int)G, ratio, inv32};
    return launch_skinny_auto<GptqSkinnyPolicy, Q4G32Epilogue>("wq_gptq_linear", pargs, x, y, ep, M, N, K, stream);
  }
  // up to 128 rows of a small matrix: two passes of the small-batch kernel, as in wq_q4g32_linear (the tiled
  // GEMM would have too few tiles for 256 CUs: N = K = 4096, M = 128: 35.6 us)
  if (M <= 2 * WQ_SMALL_BATCH_MAX_M && K % 64 == 0 && N <= 8192) {
    const GptqSkinnyPolicy::Args pargs{W_nk, (const half2_t*)SZ, (int)G, ratio, inv32};
    const int64_t m0 = WQ_SMALL_BATCH_MAX_M;
    if (int rc = launch_skinny_auto<GptqSkinnyPolicy, Q4G32Epilogue>("wq_gptq_linear", pargs, x, y, ep, m0, N, K, stream)) return rc;
    const Q4G32Epilogue ep2{(const half_t*)bias, residual ? (const half_t*)residual + m0 * N : nullptr, (int)N};
    return launch_skinny_auto<GptqSkinnyPolicy, Q4G32Epilogue>("wq_gptq_linear", pargs, x + m0 * K, y + m0 * N, ep2, M - m0, N, K, stream);
  }
  if (gs % 64 != 0)  // a K-step of the GEMM would straddle two groups: repeat the streaming kernel
    return gemv_dispatch<true>("wq_gptq_linear", W_nk, SZ, GemvZp{ratio, (int)G}, x, bias, residual, y, M, N, K, stream);
  const int spg = (int)(gs / 64);
  const GptqLdsPolicy::Args largs{W_nk, (const half2_t*)SZ, (int)G, spg,
                                  spg > 1 ? (uint32_t)(((1ull << 32) + spg - 1) / spg) : 0u};
  // tile shape as for q4f16_1 (N = K = 4096, M = 512 with 256 x 256 tiles: 47 us, with 256 x 128: 33 us)
  switch (choose_q4_lds_cfg(M, N, cu_count())) {
    case 17: return launch_gemm_lds<GptqLdsPolicy, Q4G32Epilogue, 4, 1, 1, 4, 2>("wq_gptq_linear", largs, x, y, ep, M, N, K, stream);
    case 18: return launch_gemm_lds<GptqLdsPolicy, Q4G32Epilogue, 8, 1, 1, 4, 1>("wq_gptq_linear", largs, x, y, ep, M, N, K, stream);
    case 13: return launch_gemm_lds<GptqLdsPolicy, Q4G32Epilogue, 4, 2, 2, 2, 2>("wq_gptq_linear", largs, x, y, ep, M, N, K, stream);
    default: return launch_gemm_lds<GptqLdsPolicy, Q4G32Epilogue, 8, 2, 1, 4, 1>("wq_gptq_linear", largs, x, y, ep, M, N, K, stream);
  }
}
