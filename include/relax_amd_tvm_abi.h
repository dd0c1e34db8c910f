/*
 * relax_amd_tvm_abi.h — the slice of the TVM runtime C ABI that the PackedFunc
 * layer of this library speaks, restated from the reference's public headers so
 * that the library builds without a TVM checkout and still loads into a real
 * libtvm_runtime unchanged.
 *
 *   TVMValue, type codes .......... include/tvm/runtime/c_runtime_api.h:174-215
 *   device type codes ............. include/tvm/runtime/c_runtime_api.h:131-144 (kDLROCM == 10)
 *   DLTensor ...................... dlpack (3rdparty/dlpack, an empty submodule in the reference
 *                                   tree; layout per the published dlpack.h, v0.7/0.8)
 *   exported-symbol signature ..... include/tvm/runtime/c_backend_api.h:49-51 (TVMBackendPackedCFunc)
 *   registry functions ............ include/tvm/runtime/c_runtime_api.h:245,385,399,424-425,455-478,509
 *
 * If the real <dlpack/dlpack.h> / <tvm/runtime/c_runtime_api.h> were included
 * first, their definitions are used instead.
 */
#ifndef RELAX_AMD_TVM_ABI_H_
#define RELAX_AMD_TVM_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef DLPACK_DLPACK_H_
#define DLPACK_DLPACK_H_
typedef enum { kDLCPU = 1, kDLCUDA = 2, kDLCUDAHost = 3, kDLROCM = 10, kDLROCMHost = 11 } DLDeviceType;
typedef struct {
  DLDeviceType device_type;
  int32_t device_id;
} DLDevice;
typedef enum { kDLInt = 0U, kDLUInt = 1U, kDLFloat = 2U, kDLOpaqueHandle = 3U, kDLBfloat = 4U } DLDataTypeCode;
typedef struct {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
} DLDataType;
typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides; /* NULL = compact row-major */
  uint64_t byte_offset;
} DLTensor;
#endif /* DLPACK_DLPACK_H_ */

#ifndef TVM_RUNTIME_C_RUNTIME_API_H_
typedef int64_t tvm_index_t;
typedef union {
  int64_t v_int64;
  double v_float64;
  void* v_handle;
  const char* v_str;
  DLDataType v_type;
  DLDevice v_device;
} TVMValue;
/* argument type codes */
enum {
  kTVMArgInt = 0,
  kTVMArgFloat = 2,
  kTVMOpaqueHandle = 3,
  kTVMNullptr = 4,
  kTVMDLTensorHandle = 7,
  kTVMObjectHandle = 8,
  kTVMStr = 11,
  kTVMNDArrayHandle = 13
};
typedef void* TVMFunctionHandle;
typedef void* TVMRetValueHandle;
typedef DLTensor* TVMArrayHandle;
typedef int (*TVMPackedCFunc)(TVMValue* args, int* type_codes, int num_args, TVMRetValueHandle ret,
                              void* resource_handle);
typedef void (*TVMPackedCFuncFinalizer)(void* resource_handle);
#endif

/* Signature of every PackedFunc symbol this library exports
 * (TVMBackendPackedCFunc; the BYOC C codegen emits its 5-argument prefix,
 * src/relay/backend/contrib/codegen_c/codegen_c.h:101-112).  0 = ok, -1 = error. */
typedef int (*WqTVMBackendPackedCFunc)(TVMValue* args, int* type_codes, int num_args,
                                       TVMValue* out_ret_value, int* out_ret_tcode,
                                       void* resource_handle);

#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_TVM_ABI_H_ */
