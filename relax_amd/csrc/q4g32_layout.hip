// KN-layout q4f16_1 checkpoints -> the NK layout every kernel of this library reads.
//
// The reference also schedules the same quantization scheme with the weight stored
// K-major (tests/python/dlight/test_gpu_reduction.py:102-120, test_gpu_gemv.py:813-830):
//   W uint32 [K/8, N], S fp16 [K/32, N],  w[k,n] = (((W[k/8][n] >> 4*(k%8)) & 15) - 7) * S[k/32][n].
// A word holds 8 consecutive k of ONE column in both layouts, so the conversion is a plain
// transpose of 32-bit words (and of the fp16 scales): done once when a checkpoint is loaded,
// after which the NK kernels apply unchanged.  64x64 tiles through LDS: coalesced reads
// along n, coalesced writes along k.
#include "wq_device.h"
#include "wq_host.h"

namespace wq {

template <typename T>
__global__ __launch_bounds__(256) void transpose_tile_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                            int rows, int cols) {
  __shared__ T tile[64][65];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = r0 + ty * 16 + i, c = c0 + tx;
    if (r < rows && c < cols) tile[ty * 16 + i][tx] = in[(int64_t)r * cols + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = c0 + ty * 16 + i, r = r0 + tx;  // out[c][r]
    if (r < rows && c < cols) out[(int64_t)c * rows + r] = tile[tx][ty * 16 + i];
  }
}

template <typename T>
static int transpose(const char* who, const T* in, T* out, int64_t rows, int64_t cols, hipStream_t stream) {
  if (rows == 0 || cols == 0) return WQ_OK;
  const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  WQ_REQUIRE(grid.y < 65536, "%s: too many rows", who);
  WQ_LAUNCH(who, transpose_tile_kernel<T>, grid, dim3(256), 0, stream, in, out, (int)rows, (int)cols);
  return WQ_OK;
}

}  // namespace wq

extern "C" int wq_q4g32_kn_to_nk(const uint32_t* W_kn, const uint16_t* S_kn, uint32_t* W_nk, uint16_t* S_nk,
                                 int64_t N, int64_t K, wq_stream_t stream) {
  using namespace wq;
  WQ_REQUIRE(N >= 0 && K >= 0 && K % 32 == 0, "wq_q4g32_kn_to_nk: K=%lld must be a multiple of 32", (long long)K);
  if (N == 0 || K == 0) return WQ_OK;
  WQ_REQUIRE(W_kn && S_kn && W_nk && S_nk, "wq_q4g32_kn_to_nk: null pointer");
  WQ_REQUIRE((const void*)W_kn != (const void*)W_nk && (const void*)S_kn != (const void*)S_nk,
             "wq_q4g32_kn_to_nk: cannot convert in place");
  WQ_REQUIRE(N < (1ll << 30) && K < (1ll << 24), "wq_q4g32_kn_to_nk: too large");
  if (int rc = transpose<uint32_t>("wq_q4g32_kn_to_nk", W_kn, W_nk, K / 8, N, (hipStream_t)stream)) return rc;
  return transpose<uint16_t>("wq_q4g32_kn_to_nk", S_kn, S_nk, K / 32, N, (hipStream_t)stream);
}
