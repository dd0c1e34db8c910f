// Quantizers on the device: fp16 weights [N, K] -> the packed formats the linear
// kernels read, so that checkpoints can be prepared without a trip through the host.
//   format B (per channel / group 64): the reference fixtures' `encode`
//     (tests/python/relax/test_codegen_cutlass.py:1392-1457, 1631-1676, 2044-2109);
//     its output feeds wq_ft_preprocess_weight.
//   format A (q4f16_1): the inverse of the decode in tests/python/dlight/test_gpu_gemv.py:198;
//     the reference tree holds no encoder for it, the definition is stated below.
// All arithmetic is float32 with IEEE division and round-half-away-from-zero, as the
// llvm lowering of T.round does (src/target/llvm/intrin_rule_llvm.cc:84-86).
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

// ---- format B, pass 1 (per channel only): scale[n] = max(max_k |A[n,k]|, 1e-4) * c ----
__global__ __launch_bounds__(256) void intb_row_scale_kernel(const half_t* __restrict__ A, float* __restrict__ scale32,
                                                            half_t* __restrict__ scales, int N, int K, float c) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const half_t* row = A + (int64_t)n * K;
  float mx = -65504.0f;
  for (int k = lane * 8; k < K; k += 512) {  // K % 64 == 0: whole 16-byte pieces
    const half8_t v = *reinterpret_cast<const half8_t*>(row + k);
#pragma unroll
    for (int i = 0; i < 8; ++i) mx = fmaxf(mx, fabsf((float)v[i]));
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  if (lane == 0) {
    const float s = fmaxf(mx, 0.0001f) * c;
    scale32[n] = s;
    scales[n] = (half_t)s;
  }
}

// ---- format B, pass 2: quantize and transpose one 64 (n) x 64 (k) tile ----
// GROUPED: the scale is the tile's own row maximum (group 64 along K), written to
// scales[(k0/64)*N + n]; else it comes from pass 1.
template <int NBIT, bool GROUPED>
__global__ __launch_bounds__(256) void intb_encode_tile_kernel(const half_t* __restrict__ A,
                                                              const float* __restrict__ scale32,
                                                              half_t* __restrict__ scales, int8_t* __restrict__ out,
                                                              int N, int K, float c) {
  __shared__ float tile[64][65];
  __shared__ float srow[64];
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int tid = threadIdx.x;
  {  // coalesced load: thread -> (row tid/4, 16 k at (tid%4)*16)
    const int r = tid >> 2, kc = (tid & 3) * 16;
    const half_t* src = A + (int64_t)(n0 + r) * K + k0 + kc;
    const half8_t v0 = *reinterpret_cast<const half8_t*>(src);
    const half8_t v1 = *reinterpret_cast<const half8_t*>(src + 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      tile[r][kc + i] = (float)v0[i];
      tile[r][kc + 8 + i] = (float)v1[i];
    }
  }
  __syncthreads();
  if (tid < 64) {
    float s;
    if (GROUPED) {
      float mx = -65504.0f;
      for (int k = 0; k < 64; ++k) mx = fmaxf(mx, fabsf(tile[tid][k]));
      s = fmaxf(mx, 0.0001f) * c;
      scales[(int64_t)blockIdx.y * N + n0 + tid] = (half_t)s;
    } else {
      s = scale32[n0 + tid];
    }
    srow[tid] = s;
  }
  __syncthreads();
  const float lo = NBIT == 4 ? -8.0f : -128.0f, hi = NBIT == 4 ? 7.0f : 127.0f;
  // thread -> (k = tid/4, 16 n at (tid%4)*16)
  const int k = tid >> 2, nc = (tid & 3) * 16;
  int q[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float r = roundf(tile[nc + i][k] / srow[nc + i]);
    r = fminf(fmaxf(r, lo), hi);
    q[i] = (int)r;
  }
  if (NBIT == 8) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      w[j] = (uint32_t)(q[4 * j] & 255) | ((uint32_t)(q[4 * j + 1] & 255) << 8) |
             ((uint32_t)(q[4 * j + 2] & 255) << 16) | ((uint32_t)(q[4 * j + 3] & 255) << 24);
    *reinterpret_cast<uint4_t*>(out + (int64_t)(k0 + k) * N + n0 + nc) = uint4_t{w[0], w[1], w[2], w[3]};
  } else {
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < 16; ++i) w[i >> 3] |= (uint32_t)(q[i] & 15) << (4 * (i & 7));  // low nibble = even n
    *reinterpret_cast<uint2_t*>(out + (int64_t)(k0 + k) * (N / 2) + (n0 + nc) / 2) = uint2_t{w[0], w[1]};
  }
}

// ---- format A: one lane per group of 32 ----
//   m = max |a| over the group, scale = fp16(max(m, 1e-4) / 7),
//   code = clip(round(a / f32(scale)) + 7, 0, 14)
__global__ __launch_bounds__(256) void q4g32_encode_kernel(const half_t* __restrict__ A, uint32_t* __restrict__ W,
                                                          half_t* __restrict__ S, int64_t groups) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= groups) return;
  const half8_t* src = reinterpret_cast<const half8_t*>(A + g * 32);
  half8_t v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = src[j];
  float mx = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) mx = fmaxf(mx, fabsf((float)v[j][i]));
  const half_t sh = (half_t)(fmaxf(mx, 0.0001f) / 7.0f);
  const float scale = (float)sh;
  uint32_t w[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float r = roundf((float)v[j][i] / scale) + 7.0f;
      r = fminf(fmaxf(r, 0.0f), 14.0f);
      word |= (uint32_t)(int)r << (4 * i);
    }
    w[j] = word;
  }
  *reinterpret_cast<uint4_t*>(W + g * 4) = uint4_t{w[0], w[1], w[2], w[3]};
  S[g] = sh;
}

}  // namespace wq

extern "C" int wq_intb_encode(const uint16_t* A, int8_t* w_out, uint16_t* scales, float* scale_scratch,
                              int64_t N, int64_t K, int64_t group_size, int weight_nbit, wq_stream_t stream_) {
  using namespace wq;
  hipStream_t stream = (hipStream_t)stream_;
  WQ_REQUIRE(weight_nbit == 8 || weight_nbit == 4, "wq_intb_encode: weight_nbit must be 8 or 4, got %d", weight_nbit);
  WQ_REQUIRE(N >= 0 && K >= 0 && N % 64 == 0 && K % 64 == 0,
             "wq_intb_encode: N=%lld and K=%lld must be multiples of 64", (long long)N, (long long)K);
  WQ_REQUIRE(group_size <= 0 || group_size == 64 || group_size == K,
             "wq_intb_encode: group_size must be 64 or <= 0 / K (per channel), got %lld", (long long)group_size);
  if (N == 0 || K == 0) return WQ_OK;
  const bool grouped = group_size == 64 && group_size != K;
  WQ_REQUIRE(A && w_out && scales && (grouped || scale_scratch),
             "wq_intb_encode: null pointer (per-channel mode needs N floats of scratch)");
  WQ_REQUIRE(aligned16(A) && aligned16(w_out), "wq_intb_encode: A and w_out must be 16-byte aligned");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 30) && K / 64 < 65536, "wq_intb_encode: too large");
  const float c = weight_nbit == 4 ? 0.125f : 0.0078125f;
  const half_t* a = (const half_t*)A;
  if (!grouped)
    WQ_LAUNCH("wq_intb_encode(scale)", intb_row_scale_kernel, dim3((unsigned)((N + 3) / 4)), dim3(256), 0, stream,
              a, scale_scratch, (half_t*)scales, (int)N, (int)K, c);
  const dim3 grid((unsigned)(N / 64), (unsigned)(K / 64));
#define WQ_ENC(NB, G)                                                                                        \
  WQ_LAUNCH("wq_intb_encode", (intb_encode_tile_kernel<NB, G>), grid, dim3(256), 0, stream, a, scale_scratch, \
            (half_t*)scales, w_out, (int)N, (int)K, c)
  if (weight_nbit == 8) {
    if (grouped) WQ_ENC(8, true); else WQ_ENC(8, false);
  } else {
    if (grouped) WQ_ENC(4, true); else WQ_ENC(4, false);
  }
#undef WQ_ENC
  return WQ_OK;
}

extern "C" int wq_q4g32_encode(const uint16_t* A, uint32_t* W, uint16_t* S, int64_t N, int64_t K,
                               wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(N >= 0 && K >= 0 && K % 32 == 0, "wq_q4g32_encode: K=%lld must be a multiple of 32", (long long)K);
  if (N == 0 || K == 0) return WQ_OK;
  WQ_REQUIRE(A && W && S, "wq_q4g32_encode: null pointer");
  WQ_REQUIRE(aligned16(A) && aligned16(W), "wq_q4g32_encode: A and W must be 16-byte aligned");
  const int64_t groups = N * (K / 32);
  WQ_REQUIRE((groups + 255) / 256 < (1ll << 31), "wq_q4g32_encode: too large");
  WQ_LAUNCH("wq_q4g32_encode", q4g32_encode_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0,
            (hipStream_t)stream, (const half_t*)A, W, (half_t*)S, groups);
  return WQ_OK;
}
