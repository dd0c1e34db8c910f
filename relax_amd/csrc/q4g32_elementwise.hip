// Format A element-wise entry points: code unpack and weight dequantization.
// They exist so that the integer unpack and the fp16 dequantization used inside
// the fused GEMV / GEMM kernels can be compared bit for bit with a CPU oracle:
// both call the same device functions (q4_word_minus7 / q4_word_dequant).
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

// One thread per uint32 word: 8 codes -> 8 bytes.
__global__ __launch_bounds__(256) void q4_unpack_kernel(const uint32_t* __restrict__ W,
                                                        uint2_t* __restrict__ q, int64_t nwords) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nwords) return;
  uint32_t w = W[i];
  // codes 0,2,4,6 sit in the low nibbles of the four bytes, 1,3,5,7 in the high nibbles
  uint32_t even = w & 0x0F0F0F0Fu;         // bytes: c0 c2 c4 c6
  uint32_t odd = (w >> 4) & 0x0F0F0F0Fu;   // bytes: c1 c3 c5 c7
  uint2_t o;
  o.x = __builtin_amdgcn_perm(odd, even, 0x05010400u);  // c0 c1 c2 c3
  o.y = __builtin_amdgcn_perm(odd, even, 0x07030602u);  // c4 c5 c6 c7
  q[i] = o;
}

// One thread per 16 bytes of W (4 words = one scale group = 32 weights = 64 bytes out).
__global__ __launch_bounds__(256) void q4g32_dequant_kernel(const uint4_t* __restrict__ W,
                                                            const half_t* __restrict__ S,
                                                            uint4_t* __restrict__ out,
                                                            int64_t ngroups) {
  int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= ngroups) return;
  uint4_t w4 = W[g];
  half_t s = S[g];
  half2_t s2 = {s, s};
  uint32_t ws[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    half2_t d[4];
    q4_word_dequant(ws[c], s2, d);  // d[i] = (w_i, w_{i+4})
    uint32_t u[4] = {as_u32(d[0]), as_u32(d[1]), as_u32(d[2]), as_u32(d[3])};
    // back to natural order: (w0,w1) (w2,w3) (w4,w5) (w6,w7)
    uint4_t o;
    o.x = __builtin_amdgcn_perm(u[1], u[0], 0x05040100u);
    o.y = __builtin_amdgcn_perm(u[3], u[2], 0x05040100u);
    o.z = __builtin_amdgcn_perm(u[1], u[0], 0x07060302u);
    o.w = __builtin_amdgcn_perm(u[3], u[2], 0x07060302u);
    out[g * 4 + c] = o;
  }
}

}  // namespace wq

extern "C" int wq_q4_unpack(const uint32_t* W, uint8_t* q, int64_t N, int64_t K,
                            wq_stream_t stream) {
  WQ_REQUIRE(N >= 0 && K >= 0 && K % 8 == 0, "wq_q4_unpack: K=%lld must be a multiple of 8",
             (long long)K);
  int64_t nwords = N * (K / 8);
  if (nwords == 0) return WQ_OK;
  WQ_REQUIRE(W && q, "wq_q4_unpack: null pointer");
  WQ_REQUIRE(((uintptr_t)q & 7u) == 0, "wq_q4_unpack: output must be 8-byte aligned");
  int64_t blocks = (nwords + 255) / 256;
  WQ_REQUIRE(blocks < (1ll << 31), "wq_q4_unpack: tensor too large");
  WQ_LAUNCH("wq_q4_unpack", wq::q4_unpack_kernel, dim3((unsigned)blocks), dim3(256), 0,
            (hipStream_t)stream, W, (wq::uint2_t*)q, nwords);
  return WQ_OK;
}

extern "C" int wq_q4g32_dequantize(const uint32_t* W, const uint16_t* S, uint16_t* out, int64_t N,
                                   int64_t K, wq_stream_t stream) {
  WQ_REQUIRE(N >= 0 && K >= 0 && K % 32 == 0,
             "wq_q4g32_dequantize: K=%lld must be a multiple of the group size 32", (long long)K);
  int64_t ngroups = N * (K / 32);
  if (ngroups == 0) return WQ_OK;
  WQ_REQUIRE(W && S && out, "wq_q4g32_dequantize: null pointer");
  WQ_REQUIRE(wq::aligned16(W) && wq::aligned16(out),
             "wq_q4g32_dequantize: W and out must be 16-byte aligned");
  int64_t blocks = (ngroups + 255) / 256;
  WQ_REQUIRE(blocks < (1ll << 31), "wq_q4g32_dequantize: tensor too large");
  WQ_LAUNCH("wq_q4g32_dequantize", wq::q4g32_dequant_kernel, dim3((unsigned)blocks), dim3(256), 0,
            (hipStream_t)stream, (const wq::uint4_t*)W, (const wq::half_t*)S, (wq::uint4_t*)out,
            ngroups);
  return WQ_OK;
}
