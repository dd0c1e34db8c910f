// Host-side helpers shared by the entry points: error reporting and argument checks.
#ifndef RELAX_AMD_CSRC_WQ_HOST_H_
#define RELAX_AMD_CSRC_WQ_HOST_H_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/relax_amd_wq.h"

namespace wq {

// Stores a printf-style message for wq_last_error() on this thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Number of compute units of the current device (cached).
int cu_count();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace wq

#define WQ_REQUIRE(cond, ...)                                  \
  do {                                                         \
    if (!(cond)) return ::wq::fail(WQ_EINVAL, __VA_ARGS__);    \
  } while (0)

// Launches `kernel` and reports a failed launch (bad grid, missing code object)
// without synchronising.  The thread's sticky error is cleared first so that an
// error left behind by an unrelated earlier HIP call is not blamed on this launch.
#define WQ_LAUNCH(what, kernel, grid, block, lds, stream, ...)                              \
  do {                                                                                     \
    (void)hipGetLastError();                                                               \
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                     \
    hipError_t e_ = hipGetLastError();                                                     \
    if (e_ != hipSuccess)                                                                  \
      return ::wq::fail(WQ_EDEVICE, "%s: launch failed: %s", what, hipGetErrorString(e_)); \
  } while (0)

#define WQ_HIP(call)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      return ::wq::fail(WQ_EDEVICE, "%s failed: %s", #call, hipGetErrorString(e_));         \
  } while (0)

#endif  // RELAX_AMD_CSRC_WQ_HOST_H_
