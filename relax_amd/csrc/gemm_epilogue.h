// Row-wise epilogue shared by the MFMA GEMM kernels.
//
// After v_mfma_f32_32x32x16_f16 accumulator register r of lane (j, h) is element
// (row 8*(r/4) + 4*h + r%4, col j) of its 32x32 sub-tile: a lane holds single columns, so
// direct stores would be 2-byte accesses in 64-byte runs.  Instead each wavefront transposes
// the fp32 accumulators through its own piece of LDS, one row sub-tile at a time, and then
// handles 8 consecutive columns of a row per lane: the epilogue's arithmetic is unchanged, its
// bias / residual reads and the store are 16 bytes wide.
//
// An Epilogue provides
//   half_t  operator()(float acc, int m, int n)                 one element
//   bool    wide_ok(int N, const half_t* y)                     16-byte accesses are possible
//   half8_t apply8(const float (&v)[8], int m, int n)           columns n .. n+7 of row m, n % 8 == 0
#ifndef RELAX_AMD_CSRC_GEMM_EPILOGUE_H_
#define RELAX_AMD_CSRC_GEMM_EPILOGUE_H_

#include "wq_device.h"

namespace wq {

// One row sub-tile (32 rows) per pass: a wavefront stages TN * 4 KB.
template <int TME, int TN>
struct RowwiseEpilogueCfg {
  static constexpr int RT = 1;
  static constexpr int kPitch = TN * 128;                 // bytes per staged row (fp32)
  static constexpr int kBytesPerWave = RT * 32 * kPitch;
};

// acc[i][t]: sub-tile (i, t) of a wavefront's TME x TN sub-tiles whose first element is
// (m_base, n_base).  `stage`: this wavefront's kBytesPerWave bytes of LDS that nobody else
// touches.  The caller has checked epilogue.wide_ok().
template <class Epilogue, int TME, int TN>
__device__ __forceinline__ void store_tile_rowwise(const float16_t (&acc)[TME][TN], const Epilogue& epilogue,
                                                   half_t* __restrict__ Y, int M, int N, int m_base,
                                                   int n_base, unsigned char* stage, int lane) {
  using Cfg = RowwiseEpilogueCfg<TME, TN>;
  constexpr int RT = Cfg::RT, kPitch = Cfg::kPitch;
  const int lj = lane & 31, lh = lane >> 5;
#pragma unroll
  for (int i0 = 0; i0 < TME; i0 += RT) {
#pragma unroll
    for (int ii = 0; ii < RT; ++ii) {
      if (i0 + ii < TME) {
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = ii * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            *reinterpret_cast<float*>(stage + row * kPitch + (t * 32 + lj) * 4) = acc[i0 + ii < TME ? i0 + ii : 0][t][r];
          }
      }
    }
    // LDS operations of one wavefront execute in order: no barrier between write and read
    constexpr int kGroupsPerRow = TN * 4;  // groups of 8 columns
    constexpr int kIters = RT * 32 * kGroupsPerRow / 64;
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      const int c = it * 64 + lane;
      const int row = c / kGroupsPerRow, cc = c % kGroupsPerRow;
      const float4_t v0 = *reinterpret_cast<const float4_t*>(stage + row * kPitch + cc * 32);
      const float4_t v1 = *reinterpret_cast<const float4_t*>(stage + row * kPitch + cc * 32 + 16);
      const int m = m_base + i0 * 32 + row;
      const int n = n_base + cc * 8;
      if (row < (TME - i0) * 32 && m < M && n < N) {
        const float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
        *reinterpret_cast<half8_t*>(Y + (int64_t)m * N + n) = epilogue.apply8(v, m, n);
      }
    }
  }
}

}  // namespace wq
#endif  // RELAX_AMD_CSRC_GEMM_EPILOGUE_H_
