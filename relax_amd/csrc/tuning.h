// Work-split overrides for tests and measurement, and the once-per-device kernel set-up.
#ifndef RELAX_AMD_CSRC_TUNING_H_
#define RELAX_AMD_CSRC_TUNING_H_

#include <hip/hip_runtime.h>

#include <atomic>

namespace wq {

// Overrides of the automatic work split, 0 = choose from the shape.  They belong to the CALLING
// THREAD (the tests set one, call an entry point and reset it): other threads of the process
// keep the automatic choice.  Declared for callers in include/relax_amd_wq_testing.h.
struct Tuning {
  int gemm_cfg = 0;          // tile configuration of the MFMA GEMMs
  int gemm_tail_split = 1;   // split the tiles of the last, partial round (on by default)
  int gemv_rows = 0, gemv_gpl = 0, gemv_blocks_per_cu = 0;
  int skinny_nw = 0, skinny_stages = 0, skinny_waves = 0;
  int intb_k_split = 0;      // Format B decode GEMV: wavefronts that share a column group and split K (1, 2, 4, 8)
};
Tuning& tuning();

// hipFuncAttributeMaxDynamicSharedMemorySize is a property of (kernel, device): it is raised when a
// launch first needs more than has been set on that device, not on every launch.  One object per
// kernel instantiation (a function-local static of the launcher).
struct DynamicLdsLimit {
  static constexpr int kMaxDevices = 16;
  std::atomic<int> bytes[kMaxDevices] = {};
  hipError_t ensure(const void* kernel, int need) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
      return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, need);
    if (bytes[dev].load(std::memory_order_acquire) >= need) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, need);
    if (e == hipSuccess) bytes[dev].store(need, std::memory_order_release);
    return e;
  }
};

}  // namespace wq
#endif  // RELAX_AMD_CSRC_TUNING_H_
