// Error reporting and small host utilities of the C ABI.
#include <cstring>

#include "wq_host.h"

namespace wq {

static thread_local char g_last_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

}  // namespace wq

extern "C" const char* wq_last_error(void) { return wq::g_last_error; }
extern "C" int wq_abi_version(void) { return 1; }
extern "C" const char* wq_target_arch(void) { return "gfx950"; }

extern "C" int wq_activation_from_string(const char* s) {
  if (!s) return -1;
  if (!strcmp(s, "identity")) return WQ_ACT_IDENTITY;
  if (!strcmp(s, "relu")) return WQ_ACT_RELU;
  if (!strcmp(s, "silu")) return WQ_ACT_SILU;
  if (!strcmp(s, "gelu")) return WQ_ACT_GELU;
  return -1;
}
extern "C" int wq_binary_op_from_string(const char* s) {
  if (!s) return -1;
  if (!strcmp(s, "plus")) return WQ_BIN_PLUS;
  if (!strcmp(s, "multiply")) return WQ_BIN_MULTIPLY;
  return -1;
}
extern "C" int wq_unary_op_from_string(const char* s) {
  if (!s) return -1;
  if (!strcmp(s, "identity")) return WQ_UN_IDENTITY;
  if (!strcmp(s, "relu")) return WQ_UN_RELU;
  return -1;
}
