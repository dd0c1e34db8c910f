/*
 * A tiny stand-in for the handful of TVM runtime C-API entry points the PackedFunc
 * layer looks up with dlsym (TVMFuncCreateFromCFunc, TVMFuncRegisterGlobal,
 * TVMFuncGetGlobal, TVMFuncCall, TVMCFuncSetReturn, TVMAPISetLastError,
 * TVMArrayAlloc, TVMArrayFree).  Test double only: it lets the CPU tests check that the library
 * registers its global names when a runtime is present and that a registry call
 * round-trips arguments and a returned NDArray.  Host (kDLCPU) arrays only.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/relax_amd_tvm_abi.h"

#define MAXF 256
typedef struct {
  TVMPackedCFunc fn;
  void* resource;
} Func;
static Func g_funcs[MAXF];
static char g_names[MAXF][96];
static Func* g_named[MAXF];
static int g_nfuncs = 0, g_nnames = 0;
static char g_last_error[512];
static int g_live_arrays = 0;

typedef struct {
  TVMValue value;
  int tcode;
} Ret;

void TVMAPISetLastError(const char* msg) {
  strncpy(g_last_error, msg ? msg : "", sizeof(g_last_error) - 1);
}
const char* TVMGetLastError(void) { return g_last_error; }

int TVMFuncCreateFromCFunc(TVMPackedCFunc func, void* resource_handle, TVMPackedCFuncFinalizer fin,
                           TVMFunctionHandle* out) {
  (void)fin;
  if (g_nfuncs >= MAXF) return -1;
  g_funcs[g_nfuncs].fn = func;
  g_funcs[g_nfuncs].resource = resource_handle;
  *out = &g_funcs[g_nfuncs++];
  return 0;
}
int TVMFuncRegisterGlobal(const char* name, TVMFunctionHandle f, int override) {
  for (int i = 0; i < g_nnames; ++i)
    if (!strcmp(g_names[i], name)) {
      if (!override) return -1;  /* "already registered" */
      g_named[i] = (Func*)f;
      return 0;
    }
  if (g_nnames >= MAXF) return -1;
  strncpy(g_names[g_nnames], name, 95);
  g_named[g_nnames++] = (Func*)f;
  return 0;
}
int TVMFuncGetGlobal(const char* name, TVMFunctionHandle* out) {
  *out = NULL;
  for (int i = 0; i < g_nnames; ++i)
    if (!strcmp(g_names[i], name)) *out = g_named[i];
  return 0;
}
int TVMCFuncSetReturn(TVMRetValueHandle ret, TVMValue* value, int* type_code, int num_ret) {
  if (num_ret != 1) return -1;
  ((Ret*)ret)->value = *value;
  ((Ret*)ret)->tcode = *type_code;
  return 0;
}
int TVMFuncCall(TVMFunctionHandle func, TVMValue* args, int* type_codes, int num_args,
                TVMValue* ret_val, int* ret_type_code) {
  Func* f = (Func*)func;
  Ret r;
  r.value.v_handle = NULL;
  r.tcode = kTVMNullptr;
  int rc = f->fn(args, type_codes, num_args, &r, f->resource);
  *ret_val = r.value;
  *ret_type_code = r.tcode;
  return rc;
}
int TVMArrayAlloc(const tvm_index_t* shape, int ndim, int dtype_code, int dtype_bits, int dtype_lanes,
                  int device_type, int device_id, TVMArrayHandle* out) {
  if (device_type != kDLCPU) return -1;
  DLTensor* t = (DLTensor*)calloc(1, sizeof(DLTensor));
  int64_t n = 1;
  t->shape = (int64_t*)malloc(sizeof(int64_t) * (size_t)(ndim > 0 ? ndim : 1));
  for (int i = 0; i < ndim; ++i) {
    t->shape[i] = shape[i];
    n *= shape[i];
  }
  t->ndim = ndim;
  t->dtype.code = (uint8_t)dtype_code;
  t->dtype.bits = (uint8_t)dtype_bits;
  t->dtype.lanes = (uint16_t)dtype_lanes;
  t->device.device_type = (DLDeviceType)device_type;
  t->device.device_id = device_id;
  t->data = malloc((size_t)(n * dtype_bits / 8 + 64));
  ++g_live_arrays;
  *out = t;
  return 0;
}
int TVMArrayFree(TVMArrayHandle h) {
  DLTensor* t = (DLTensor*)h;
  free(t->data);
  free(t->shape);
  free(t);
  --g_live_arrays;
  return 0;
}
int fake_live_arrays(void) { return g_live_arrays; }
/* a function of the host's own, to check that the library does not replace it */
static int host_own_fn(TVMValue* a, int* c, int n, TVMRetValueHandle r, void* res) {
  (void)a; (void)c; (void)n; (void)r; (void)res;
  return 0;
}
int fake_register_host_function(const char* name) {
  TVMFunctionHandle f;
  if (TVMFuncCreateFromCFunc(host_own_fn, NULL, NULL, &f) != 0) return -1;
  return TVMFuncRegisterGlobal(name, f, 0);
}
int fake_is_host_function(const char* name) {
  TVMFunctionHandle f = NULL;
  TVMFuncGetGlobal(name, &f);
  return f && ((Func*)f)->fn == host_own_fn;
}
int fake_num_registered(void) { return g_nnames; }
const char* fake_registered_name(int i) { return g_names[i]; }
