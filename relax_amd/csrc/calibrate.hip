// Two microbenchmark kernels that give the measured ceilings the library's kernels are
// compared with, next to the vendor peak figures: MFMA issue only (no memory traffic)
// and a pure streaming read (no arithmetic worth mentioning, no write).
#include "../../include/relax_amd_wq_testing.h"
#include <hip/hip_runtime.h>

#include "wq_device.h"

namespace wq {

// Eight independent accumulators per wavefront, one wavefront per SIMD: every
// v_mfma_f32_32x32x16_f16 can issue as soon as the previous one has left the pipe.
__global__ __launch_bounds__(256) void calibrate_mfma_kernel(float* out, int iters, float seed) {
  float16_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  half8_t a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (half_t)(threadIdx.x * 0.001f + seed);
    b[i] = (half_t)(seed * 0.5f);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Every wavefront reads 8 KB contiguous with eight 16-byte loads per lane in flight and
// ends; the grid covers the buffer once.
__global__ __launch_bounds__(256) void calibrate_read_kernel(const uint4_t* __restrict__ src, int64_t n16,
                                                            uint32_t* out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t base = ((int64_t)blockIdx.x * 4 + wave) * 512 + lane;
  uint4_t v[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int64_t i = base + u * 64;
    v[u] = i < n16 ? __builtin_nontemporal_load(&src[i]) : uint4_t{0, 0, 0, 0};
  }
  uint4_t acc = {0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < 8; ++u) acc ^= v[u];
  // data-dependent and practically never true: keeps the loads alive without a store per lane
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u) out[0] = acc.x;
}

}  // namespace wq

// This file is a library of its own (librelax_amd_wq_calibrate.so): it reports errors through its
// return value only (WQ_EINVAL, WQ_EDEVICE) and shares no state with the product library.
static int launch_status() { return hipGetLastError() == hipSuccess ? WQ_OK : WQ_EDEVICE; }

extern "C" int wq_calibrate_mfma_f16(void* scratch, int64_t scratch_bytes, int iters, double* flops,
                                     wq_stream_t stream) {
  using namespace wq;
  int dev = 0, blocks = 0;  // one workgroup of four wavefronts per CU
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&blocks, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return WQ_EDEVICE;
  if (!scratch || scratch_bytes < (int64_t)blocks * 256 * 4 || iters <= 0) return WQ_EINVAL;
  hipLaunchKernelGGL(calibrate_mfma_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (float*)scratch, iters,
                     1.0f);
  if (flops) *flops = (double)blocks * 4 * iters * 8 * (2.0 * 32 * 32 * 16);
  return launch_status();
}

extern "C" int wq_calibrate_read(const void* src, int64_t bytes, void* scratch, wq_stream_t stream) {
  using namespace wq;
  if (!src || !scratch || bytes < 0 || bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(src) & 15u))
    return WQ_EINVAL;
  if (bytes == 0) return WQ_OK;
  const int64_t blocks = (bytes / 16 + 2047) / 2048;
  if (blocks >= (1ll << 31)) return WQ_EINVAL;
  hipLaunchKernelGGL(calibrate_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const uint4_t*)src, bytes / 16, (uint32_t*)scratch);
  return launch_status();
}
