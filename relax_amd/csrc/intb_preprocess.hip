// Weight reordering for the fp16 x int8/int4 GEMM: the MI355X-native counterpart of
// cutlass.ft_preprocess_weight (src/runtime/contrib/cutlass/weight_preprocess.cc:38-59),
// which forwards to fastertransformer::preprocess_weights of the external
// tlc-pack/cutlass_fpA_intB_gemm library.  The stored format is kept byte for byte
// (layout family sm 75..89) so that weights prepared by either side are
// interchangeable; the kernels in intb_kernels.hip read it directly.
//
// Closed form of the result (rows = K, cols = N elements), as 32-bit words:
//   int8: word d  ->  pair = d / (2*K/4), tile = (d % (2*K/4)) / 32,
//         c = 2*pair + (d%32)/16, v = d%16;   byte i of the word is source element
//         (k = 64*tile + 16*(v/4) + 2*(v%4) + {0, 8, 1, 9}[i],  n = c), plus 128.
//   int4: word d  ->  quad = d / (4*K/8), tile = (d % (4*K/8)) / 32,
//         c = 4*quad + (d%32)/8, v = d%8;     nibble i of the word is source element
//         (k = 64*tile + 32*(v/4) + 2*(v%4) + {0, 8, 16, 24, 1, 9, 17, 25}[i],  n = c), plus 8.
// i.e. 2 (int8) / 4 (int4) columns are interleaved per 64-row tile, and inside a
// word the two elements a packed fp16 pair needs (k, k+1) sit in byte 0/2 (int8) or
// in nibble i / i+4 (int4).
//
// The device version moves one 64 x 64 element tile through LDS per workgroup:
// coalesced 16-byte reads of the row-major source, 128-byte contiguous writes of
// the interleaved result.  The reference does this step on the host (device ->
// host copy, CPU permutation, host -> device copy); the host entry point keeps
// that behaviour for callers that hold host memory.
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

__host__ __device__ __forceinline__ int ft_src_k8(int v, int i) {
  // v: word index inside the 64-row tile (0..15), i: byte in word
  const int off[4] = {0, 8, 1, 9};
  return 16 * (v >> 2) + 2 * (v & 3) + off[i];
}
__host__ __device__ __forceinline__ int ft_src_k4(int v, int i) {
  // v: word index inside the 64-row tile (0..7), i: nibble in word
  const int off[8] = {0, 8, 16, 24, 1, 9, 17, 25};
  return 32 * (v >> 2) + 2 * (v & 3) + off[i];
}

constexpr int kTileStride8 = 80;  // bytes per LDS row (64 + pad, 16-byte multiple)
constexpr int kTileStride4 = 48;  // 32 + pad

__global__ __launch_bounds__(256) void ft_preprocess_int8_kernel(const uint8_t* __restrict__ in,
                                                                 uint32_t* __restrict__ out, int K,
                                                                 int N) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[64 * kTileStride8];
  const int64_t expert = (int64_t)blockIdx.z * K * N;
  const int c0 = blockIdx.x * 64, tile_k = blockIdx.y, k0 = tile_k * 64;
  const int t = threadIdx.x;
  {
    const int row = t >> 2, cc = t & 3;
    const uint4_t v =
        *reinterpret_cast<const uint4_t*>(in + expert + (int64_t)(k0 + row) * N + c0 + 16 * cc);
    *reinterpret_cast<uint4_t*>(&tile[row * kTileStride8 + 16 * cc]) = v;
  }
  __syncthreads();
  uint32_t* dst = out + expert / 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int widx = t + 256 * j;       // 0..1023: 32 column pairs x 32 words
    const int pair = widx >> 5, within = widx & 31;
    const int c = 2 * pair + (within >> 4), v = within & 15;
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t b = (uint32_t)(tile[ft_src_k8(v, i) * kTileStride8 + c] + 128u) & 0xffu;
      word |= b << (8 * i);
    }
    dst[((int64_t)(c0 / 2 + pair) * (K / 64) + tile_k) * 32 + within] = word;
  }
}

__global__ __launch_bounds__(256) void ft_preprocess_int4_kernel(const uint8_t* __restrict__ in,
                                                                 uint32_t* __restrict__ out, int K,
                                                                 int N) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[64 * kTileStride4];
  const int64_t expert = (int64_t)blockIdx.z * K * (N / 2);
  const int c0 = blockIdx.x * 64, tile_k = blockIdx.y, k0 = tile_k * 64;
  const int t = threadIdx.x;
  if (t < 128) {
    const int row = t >> 1, cc = t & 1;
    const uint4_t v = *reinterpret_cast<const uint4_t*>(in + expert + (int64_t)(k0 + row) * (N / 2) +
                                                        c0 / 2 + 16 * cc);
    *reinterpret_cast<uint4_t*>(&tile[row * kTileStride4 + 16 * cc]) = v;
  }
  __syncthreads();
  uint32_t* dst = out + expert / 4;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int widx = t + 256 * j;       // 0..511: 16 column quads x 32 words
    const int quad = widx >> 5, within = widx & 31;
    const int c = 4 * quad + (within >> 3), v = within & 7;
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t byte = tile[ft_src_k4(v, i) * kTileStride4 + (c >> 1)];
      const uint32_t nib = ((byte >> (4 * (c & 1))) + 8u) & 15u;
      word |= nib << (4 * i);
    }
    dst[((int64_t)(c0 / 4 + quad) * (K / 64) + tile_k) * 32 + within] = word;
  }
}

static int check_preprocess_args(const char* who, const void* out, const void* in,
                                 int64_t num_experts, int64_t rows, int64_t cols, int sm) {
  if (sm < 75 || sm >= 90)
    return fail(WQ_EUNSUPPORTED,
                "%s: sm=%d selects a layout family that is not implemented (75 <= sm < 90 only)",
                who, sm);
  WQ_REQUIRE(num_experts >= 0 && rows >= 0 && cols >= 0, "%s: negative dimension", who);
  WQ_REQUIRE(rows % 64 == 0 && cols % 64 == 0,
             "%s: rows=%lld and cols=%lld must be multiples of 64", who, (long long)rows,
             (long long)cols);
  if (num_experts * rows * cols == 0) return 1;  // nothing to do
  WQ_REQUIRE(out && in, "%s: null pointer", who);
  WQ_REQUIRE(out != in, "%s: in-place reordering is not supported", who);
  return WQ_OK;
}

}  // namespace wq

extern "C" int wq_ft_preprocess_weight_host(int8_t* out_, const int8_t* in_, int64_t num_experts,
                                            int64_t rows, int64_t cols, int is_int4, int sm) {
  using namespace wq;
  int rc = check_preprocess_args("wq_ft_preprocess_weight_host", out_, in_, num_experts, rows, cols, sm);
  if (rc != WQ_OK) return rc > 0 ? WQ_OK : rc;
  const int64_t K = rows, N = cols;
  const int64_t expert_bytes = is_int4 ? K * N / 2 : K * N;
  for (int64_t e = 0; e < num_experts; ++e) {
    const uint8_t* in = reinterpret_cast<const uint8_t*>(in_) + e * expert_bytes;
    uint32_t* out = reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(out_) + e * expert_bytes);
    const int64_t nwords = expert_bytes / 4;
    if (!is_int4) {
      const int64_t per_pair = 2 * (K / 4);
      for (int64_t d = 0; d < nwords; ++d) {
        const int64_t pair = d / per_pair, rem = d % per_pair, tile = rem / 32;
        const int within = (int)(rem % 32);
        const int64_t c = 2 * pair + within / 16;
        const int v = within % 16;
        uint32_t word = 0;
        for (int i = 0; i < 4; ++i) {
          const int64_t k = 64 * tile + ft_src_k8(v, i);
          word |= ((uint32_t)(in[k * N + c] + 128u) & 0xffu) << (8 * i);
        }
        out[d] = word;
      }
    } else {
      const int64_t per_quad = 4 * (K / 8);
      for (int64_t d = 0; d < nwords; ++d) {
        const int64_t quad = d / per_quad, rem = d % per_quad, tile = rem / 32;
        const int within = (int)(rem % 32);
        const int64_t c = 4 * quad + within / 8;
        const int v = within % 8;
        uint32_t word = 0;
        for (int i = 0; i < 8; ++i) {
          const int64_t k = 64 * tile + ft_src_k4(v, i);
          const uint32_t byte = in[k * (N / 2) + c / 2];
          word |= (((byte >> (4 * (c & 1))) + 8u) & 15u) << (4 * i);
        }
        out[d] = word;
      }
    }
  }
  return WQ_OK;
}

extern "C" int wq_ft_preprocess_weight(int8_t* out, const int8_t* in, int64_t num_experts,
                                       int64_t rows, int64_t cols, int is_int4, int sm,
                                       wq_stream_t stream) {
  using namespace wq;
  int rc = check_preprocess_args("wq_ft_preprocess_weight", out, in, num_experts, rows, cols, sm);
  if (rc != WQ_OK) return rc > 0 ? WQ_OK : rc;
  WQ_REQUIRE(aligned16(in) && aligned16(out), "wq_ft_preprocess_weight: buffers must be 16-byte aligned");
  WQ_REQUIRE(cols / 64 < (1ll << 31) && rows / 64 < 65536 && num_experts < 65536,
             "wq_ft_preprocess_weight: tensor too large");
  const dim3 grid((unsigned)(cols / 64), (unsigned)(rows / 64), (unsigned)num_experts);
  if (is_int4) {
    WQ_LAUNCH("wq_ft_preprocess_weight", ft_preprocess_int4_kernel, grid, dim3(256), 0,
              (hipStream_t)stream, (const uint8_t*)in, (uint32_t*)out, (int)rows, (int)cols);
  } else {
    WQ_LAUNCH("wq_ft_preprocess_weight", ft_preprocess_int8_kernel, grid, dim3(256), 0,
              (hipStream_t)stream, (const uint8_t*)in, (uint32_t*)out, (int)rows, (int)cols);
  }
  return WQ_OK;
}
