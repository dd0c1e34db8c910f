// PackedFunc layer: the symbols a Relax VM resolves by name (imported module
// first, then the global registry: src/runtime/relax_vm/vm.cc:669-681) and calls
// with TVMValue / type-code arrays.  Each one validates its DLTensors and
// forwards plain pointers to the C ABI of relax_amd_wq.h.
#include <dlfcn.h>

#include <cstring>
#include <string>
#include <vector>

#include "../../include/relax_amd_tvm.h"
#include "wq_host.h"

namespace wq {
namespace {

// ---- optional services of a host TVM runtime, looked up once with dlsym ----
struct HostRuntime {
  void (*set_last_error)(const char*) = nullptr;
  int (*func_create)(TVMPackedCFunc, void*, TVMPackedCFuncFinalizer, TVMFunctionHandle*) = nullptr;
  int (*func_register)(const char*, TVMFunctionHandle, int) = nullptr;
  int (*func_get_global)(const char*, TVMFunctionHandle*) = nullptr;
  int (*func_call)(TVMFunctionHandle, TVMValue*, int*, int, TVMValue*, int*) = nullptr;
  int (*set_return)(TVMRetValueHandle, TVMValue*, int*, int) = nullptr;
  int (*array_alloc)(const tvm_index_t*, int, int, int, int, int, int, TVMArrayHandle*) = nullptr;
  int (*array_free)(TVMArrayHandle) = nullptr;
  bool present = false;
};

HostRuntime& host() {
  static HostRuntime h = [] {
    HostRuntime r;
    auto sym = [](const char* n) { return dlsym(RTLD_DEFAULT, n); };
    r.set_last_error = reinterpret_cast<decltype(r.set_last_error)>(sym("TVMAPISetLastError"));
    r.func_create = reinterpret_cast<decltype(r.func_create)>(sym("TVMFuncCreateFromCFunc"));
    r.func_register = reinterpret_cast<decltype(r.func_register)>(sym("TVMFuncRegisterGlobal"));
    r.func_get_global = reinterpret_cast<decltype(r.func_get_global)>(sym("TVMFuncGetGlobal"));
    r.func_call = reinterpret_cast<decltype(r.func_call)>(sym("TVMFuncCall"));
    r.set_return = reinterpret_cast<decltype(r.set_return)>(sym("TVMCFuncSetReturn"));
    r.array_alloc = reinterpret_cast<decltype(r.array_alloc)>(sym("TVMArrayAlloc"));
    r.array_free = reinterpret_cast<decltype(r.array_free)>(sym("TVMArrayFree"));
    r.present = r.func_create && r.func_register;
    return r;
  }();
  return h;
}

wq_stream_getter_t g_stream_getter = nullptr;
thread_local bool t_stream_override_on = false;
thread_local void* t_stream_override = nullptr;

// The stream a PackedFunc call enqueues on.
void* current_stream() {
  if (t_stream_override_on) return t_stream_override;  // set by the instruction-list executor
  if (g_stream_getter) return g_stream_getter();
  HostRuntime& h = host();
  if (h.func_get_global && h.func_call) {
    static TVMFunctionHandle getter = [&h]() -> TVMFunctionHandle {
      TVMFunctionHandle f = nullptr;
      if (h.func_get_global("runtime.get_rocm_stream", &f) != 0) return nullptr;
      return f;
    }();
    if (getter) {
      TVMValue ret;
      int tcode = kTVMNullptr;
      ret.v_handle = nullptr;
      if (h.func_call(getter, nullptr, nullptr, 0, &ret, &tcode) == 0 && tcode != kTVMNullptr)
        return ret.v_handle;
    }
  }
  return nullptr;  // the null stream
}

// Reports an error the way a PackedFunc must: message to the runtime, -1 to the caller.
int packed_fail() {
  HostRuntime& h = host();
  if (h.set_last_error) h.set_last_error(wq_last_error());
  return -1;
}

struct Tensor {
  const DLTensor* t = nullptr;
  void* ptr = nullptr;  // data + byte_offset
  int64_t numel = 1;
};

bool is_compact(const DLTensor* t) {
  if (!t->strides) return true;
  int64_t expect = 1;
  for (int i = t->ndim - 1; i >= 0; --i) {
    if (t->shape[i] != 1 && t->strides[i] != expect) return false;
    expect *= t->shape[i];
  }
  return true;
}

// Fetches argument i as a tensor of the given dtype; returns false with the error set.
bool get_tensor(const char* who, TVMValue* args, int* tcodes, int num_args, int i, int code, int bits,
                const char* what, Tensor* out, bool allow_host = false) {
  if (i >= num_args) {
    fail(WQ_EINVAL, "%s: missing argument %d (%s)", who, i, what);
    return false;
  }
  if (tcodes[i] != kTVMDLTensorHandle && tcodes[i] != kTVMNDArrayHandle) {
    fail(WQ_EINVAL, "%s: argument %d (%s) is not a tensor (type code %d)", who, i, what, tcodes[i]);
    return false;
  }
  const DLTensor* t = static_cast<const DLTensor*>(args[i].v_handle);
  if (!t) {
    fail(WQ_EINVAL, "%s: argument %d (%s) is null", who, i, what);
    return false;
  }
  if (t->dtype.code != code || t->dtype.bits != bits || t->dtype.lanes != 1) {
    fail(WQ_EINVAL, "%s: %s has dtype (code %d, %d bits, %d lanes), expected (code %d, %d bits)", who,
         what, t->dtype.code, t->dtype.bits, t->dtype.lanes, code, bits);
    return false;
  }
  const bool on_gpu = t->device.device_type == kDLROCM;
  const bool on_host = t->device.device_type == kDLCPU || t->device.device_type == kDLROCMHost;
  if (!(on_gpu || (allow_host && on_host))) {
    fail(WQ_EINVAL, "%s: %s lives on device type %d; expected a ROCm device tensor", who, what,
         (int)t->device.device_type);
    return false;
  }
  if (!is_compact(t)) {
    fail(WQ_EINVAL, "%s: %s must be compact (row-major, no strides)", who, what);
    return false;
  }
  out->t = t;
  out->ptr = static_cast<char*>(t->data) + t->byte_offset;
  out->numel = 1;
  for (int d = 0; d < t->ndim; ++d) out->numel *= t->shape[d];
  return true;
}

bool get_int(const char* who, TVMValue* args, int* tcodes, int num_args, int i, const char* what,
             int64_t* out) {
  if (i >= num_args || tcodes[i] != kTVMArgInt) {
    fail(WQ_EINVAL, "%s: argument %d (%s) must be an integer", who, i, what);
    return false;
  }
  *out = args[i].v_int64;
  return true;
}

int64_t leading(const DLTensor* t) {  // product of all dims but the last
  int64_t m = 1;
  for (int d = 0; d + 1 < t->ndim; ++d) m *= t->shape[d];
  return m;
}

// ------------------------------------------------------------------ format A
int q4_matmul(const char* who, TVMValue* args, int* tcodes, int n, bool has_bias, bool has_res) {
  Tensor W, S, x, bias, res, y;
  int i = 0;
  if (n != 4 + (int)has_bias + (int)has_res) {
    fail(WQ_EINVAL, "%s: expected %d arguments, got %d", who, 4 + (int)has_bias + (int)has_res, n);
    return packed_fail();
  }
  if (!get_tensor(who, args, tcodes, n, i++, kDLUInt, 32, "W", &W)) return packed_fail();
  if (!get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "S", &S)) return packed_fail();
  if (!get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "x", &x)) return packed_fail();
  if (has_bias && !get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "bias", &bias)) return packed_fail();
  if (has_res && !get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "residual", &res)) return packed_fail();
  if (!get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "out", &y)) return packed_fail();
  if (W.t->ndim != 2 || S.t->ndim != 2 || x.t->ndim < 1 || y.t->ndim < 1) {
    fail(WQ_EINVAL, "%s: W and S must be matrices", who);
    return packed_fail();
  }
  const int64_t N = W.t->shape[0], K = W.t->shape[1] * 8;
  const int64_t M = x.t->ndim ? leading(x.t) : 0;
  if (S.t->shape[0] != N || S.t->shape[1] * 32 != K || x.t->shape[x.t->ndim - 1] != K ||
      y.numel != M * N || y.t->shape[y.t->ndim - 1] != N || (has_bias && bias.numel != N) ||
      (has_res && res.numel != M * N)) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (N=%lld K=%lld M=%lld)", who, (long long)N,
         (long long)K, (long long)M);
    return packed_fail();
  }
  const int rc = wq_q4g32_linear((const uint32_t*)W.ptr, (const uint16_t*)S.ptr, (const uint16_t*)x.ptr,
                                 (const uint16_t*)bias.ptr, (const uint16_t*)res.ptr, (uint16_t*)y.ptr,
                                 M, N, K, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// ------------------------------------------------------------------ format B
// op_type follows python/tvm/contrib/cutlass/build.py:742-775: activation is looked up
// between "matmul_" and "residual_", the residual postfix gives binary / unary op.
struct DecodeMatmulOp {
  bool has_bias, has_residual;
  int activation, binary_op, unary_op;
};

DecodeMatmulOp parse_op_type(const std::string& op) {
  DecodeMatmulOp r{};
  r.has_bias = op.find("bias") != std::string::npos;
  const size_t rpos = op.find("residual_");
  r.has_residual = rpos != std::string::npos;
  const size_t mpos = op.find("matmul");
  const std::string head = op.substr(mpos, r.has_residual ? rpos - mpos : std::string::npos);
  r.activation = WQ_ACT_IDENTITY;
  for (const char* a : {"relu", "silu", "gelu"})
    if (head.find(a) != std::string::npos) {
      r.activation = wq_activation_from_string(a);
      break;
    }
  r.binary_op = WQ_BIN_NONE;
  r.unary_op = WQ_UN_IDENTITY;
  if (r.has_residual) {
    const std::string post = op.substr(rpos + strlen("residual_"));
    r.binary_op = post.rfind("multiply", 0) == 0 ? WQ_BIN_MULTIPLY : WQ_BIN_PLUS;
    r.unary_op = post.find("relu") != std::string::npos ? WQ_UN_RELU : WQ_UN_IDENTITY;
  }
  return r;
}

int decode_matmul(const char* op_type, TVMValue* args, int* tcodes, int n) {
  const DecodeMatmulOp op = parse_op_type(op_type);
  const char* who = op_type;
  const int expect = 4 + (int)op.has_bias + (int)op.has_residual;
  if (n != expect) {
    fail(WQ_EINVAL, "%s: expected %d arguments (x, w, scales%s%s, out), got %d", who, expect,
         op.has_bias ? ", bias" : "", op.has_residual ? ", residual" : "", n);
    return packed_fail();
  }
  Tensor x, w, s, bias, res, out;
  int i = 0;
  if (!get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "x", &x)) return packed_fail();
  if (!get_tensor(who, args, tcodes, n, i++, kDLInt, 8, "w_encoded", &w)) return packed_fail();
  if (!get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "scales", &s)) return packed_fail();
  if (op.has_bias && !get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "bias", &bias)) return packed_fail();
  if (op.has_residual && !get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "residual", &res)) return packed_fail();
  if (!get_tensor(who, args, tcodes, n, i++, kDLFloat, 16, "out", &out)) return packed_fail();
  if (w.t->ndim != 2 || x.t->ndim < 1 || out.t->ndim < 1 || s.t->ndim < 1 || s.t->ndim > 2) {
    fail(WQ_EINVAL, "%s: unexpected ranks", who);
    return packed_fail();
  }
  const int64_t k = w.t->shape[0];
  const int64_t N = out.t->shape[out.t->ndim - 1];
  int nbit;
  if (N == w.t->shape[1]) {
    nbit = 8;
  } else if (N == 2 * w.t->shape[1]) {
    nbit = 4;
  } else {
    fail(WQ_EINVAL, "%s: output width %lld matches neither int8 nor int4 weight of width %lld", who,
         (long long)N, (long long)w.t->shape[1]);
    return packed_fail();
  }
  // group size: 64 when the scales are a matrix with more than one row, else per column
  const int64_t group = (s.t->ndim == 2 && s.t->shape[0] != 1) ? 64 : -1;
  const int64_t m = leading(x.t);
  if (x.t->shape[x.t->ndim - 1] != k || out.numel != m * N ||
      s.numel != (group > 0 ? (k / 64) * N : N) || (op.has_residual && res.numel != m * N)) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (m=%lld n=%lld k=%lld)", who, (long long)m,
         (long long)N, (long long)k);
    return packed_fail();
  }
  int64_t bias_stride = 0;
  if (op.has_bias) {
    if (bias.t->ndim < 1 || bias.t->shape[bias.t->ndim - 1] != N ||
        (bias.numel != N && bias.numel != m * N)) {
      fail(WQ_EINVAL, "%s: bias must have n or m*n elements with last dim n", who);
      return packed_fail();
    }
    if (bias.numel != N) bias_stride = N;
  }
  void* stream = current_stream();
  int rc;
  if (op.has_residual) {
    if (bias_stride) {
      fail(WQ_EINVAL, "%s: the residual form takes a bias that only varies along n", who);
      return packed_fail();
    }
    rc = wq_fpA_intB_gemm_residual((const uint16_t*)x.ptr, (const int8_t*)w.ptr, (const uint16_t*)s.ptr,
                                   (const uint16_t*)bias.ptr, (const uint16_t*)res.ptr,
                                   (uint16_t*)out.ptr, op.activation, op.binary_op, op.unary_op, m, N,
                                   k, group, nbit, nullptr, 0, stream);
  } else {
    rc = wq_fpA_intB_gemm((const uint16_t*)x.ptr, (const int8_t*)w.ptr, (const uint16_t*)s.ptr,
                          (const uint16_t*)bias.ptr, (uint16_t*)out.ptr, op.activation, m, N, k, group,
                          bias_stride, nbit, nullptr, 0, stream);
  }
  return rc == WQ_OK ? 0 : packed_fail();
}

// ---------------------------------------------------------- weight reordering
int preprocess_into(const char* who, const Tensor& in, int64_t sm, int64_t is_int4, void* out_ptr) {
  const DLTensor* t = in.t;
  if (t->ndim != 2 && t->ndim != 3) {
    fail(WQ_EINVAL, "%s: packed_weight must be [K, N] or [E, K, N]", who);
    return -1;
  }
  const bool is_2d = t->ndim == 2;
  const int64_t experts = is_2d ? 1 : t->shape[0];
  const int64_t rows = t->shape[is_2d ? 0 : 1];
  int64_t cols = t->shape[is_2d ? 1 : 2];
  if (is_int4) cols *= 2;  // "cols" counts unpacked elements (weight_preprocess.cc:48-50)
  int rc;
  if (t->device.device_type == kDLROCM)
    rc = wq_ft_preprocess_weight((int8_t*)out_ptr, (const int8_t*)in.ptr, experts, rows, cols,
                                 (int)is_int4, (int)sm, current_stream());
  else
    rc = wq_ft_preprocess_weight_host((int8_t*)out_ptr, (const int8_t*)in.ptr, experts, rows, cols,
                                      (int)is_int4, (int)sm);
  return rc == WQ_OK ? 0 : -1;
}

}  // namespace
}  // namespace wq

using namespace wq;

extern "C" {

WQ_PACKED(cutlass_ft_preprocess_weight) {
  (void)resource_handle;
  const char* who = "cutlass.ft_preprocess_weight";
  Tensor in;
  int64_t sm = 0, is_int4 = 0;
  if (num_args != 3) {
    fail(WQ_EINVAL, "%s: expected (packed_weight, sm, is_int4)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLInt, 8, "packed_weight", &in, true) ||
      !get_int(who, args, type_codes, num_args, 1, "sm", &sm) ||
      !get_int(who, args, type_codes, num_args, 2, "is_int4", &is_int4))
    return packed_fail();
  HostRuntime& h = host();
  if (!h.array_alloc) {
    fail(WQ_EUNSUPPORTED,
         "%s: no TVM runtime in this process to allocate the result; call "
         "relax_amd.ft_preprocess_weight_dps(packed_weight, sm, is_int4, out) instead",
         who);
    return packed_fail();
  }
  TVMArrayHandle out = nullptr;
  const DLTensor* t = in.t;
  if (h.array_alloc(t->shape, t->ndim, t->dtype.code, t->dtype.bits, t->dtype.lanes,
                    (int)t->device.device_type, t->device.device_id, &out) != 0 || !out) {
    fail(WQ_EDEVICE, "%s: TVMArrayAlloc failed", who);
    return packed_fail();
  }
  if (preprocess_into(who, in, sm, is_int4, static_cast<char*>(out->data) + out->byte_offset) != 0) {
    if (h.array_free) (void)h.array_free(out);  // the result never reaches the caller: give it back
    return packed_fail();
  }
  // ownership of the new array moves to the caller (packed_func.h:975-982)
  out_ret_value->v_handle = out;
  *out_ret_tcode = kTVMNDArrayHandle;
  return 0;
}

WQ_PACKED(relax_amd_ft_preprocess_weight_dps) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.ft_preprocess_weight_dps";
  Tensor in, out;
  int64_t sm = 0, is_int4 = 0;
  if (num_args != 4) {
    fail(WQ_EINVAL, "%s: expected (packed_weight, sm, is_int4, out)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLInt, 8, "packed_weight", &in, true) ||
      !get_int(who, args, type_codes, num_args, 1, "sm", &sm) ||
      !get_int(who, args, type_codes, num_args, 2, "is_int4", &is_int4) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLInt, 8, "out", &out, true))
    return packed_fail();
  if (out.numel != in.numel || out.t->device.device_type != in.t->device.device_type) {
    fail(WQ_EINVAL, "%s: out must match packed_weight in size and device", who);
    return packed_fail();
  }
  return preprocess_into(who, in, sm, is_int4, out.ptr) == 0 ? 0 : packed_fail();
}

WQ_PACKED(relax_amd_q4f16_1_matmul) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  return q4_matmul("relax_amd.q4f16_1_matmul", args, type_codes, num_args, false, false);
}
WQ_PACKED(relax_amd_q4f16_1_matmul_bias) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  return q4_matmul("relax_amd.q4f16_1_matmul_bias", args, type_codes, num_args, true, false);
}
WQ_PACKED(relax_amd_q4f16_1_matmul_bias_residual) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  return q4_matmul("relax_amd.q4f16_1_matmul_bias_residual", args, type_codes, num_args, true, true);
}
// (W, S, x fp16 [.., K], out fp16 [.., N]): the matmul with the reference's fp16 accumulation
// (tests/python/dlight/test_gpu_reduction.py:44-51, test_gpu_low_batch_gemv.py:50-57): a decode / low-batch entry
WQ_PACKED(relax_amd_q4f16_1_matmul_f16acc) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_matmul_f16acc";
  Tensor W, S, x, y;
  if (num_args != 4) {
    fail(WQ_EINVAL, "%s: expected (W, S, x, out)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W", &W) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "S", &S) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLFloat, 16, "x", &x) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 16, "out", &y))
    return packed_fail();
  if (W.t->ndim != 2 || S.t->ndim != 2 || x.t->ndim < 1 || y.t->ndim < 1) {
    fail(WQ_EINVAL, "%s: W and S must be matrices", who);
    return packed_fail();
  }
  const int64_t N = W.t->shape[0], K = W.t->shape[1] * 8;
  const int64_t M = leading(x.t);
  if (S.t->shape[0] != N || S.t->shape[1] * 32 != K || x.t->shape[x.t->ndim - 1] != K || y.numel != M * N ||
      y.t->shape[y.t->ndim - 1] != N) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (N=%lld K=%lld M=%lld)", who, (long long)N, (long long)K, (long long)M);
    return packed_fail();
  }
  const int rc = wq_q4g32_gemv_f16acc((const uint32_t*)W.ptr, (const uint16_t*)S.ptr, (const uint16_t*)x.ptr,
                                      (uint16_t*)y.ptr, M, N, K, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}
WQ_PACKED(relax_amd_q4f16_1_decode) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_decode";
  Tensor W, S, out;
  if (num_args != 3) {
    fail(WQ_EINVAL, "%s: expected (W, S, out)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W", &W) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "S", &S) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLFloat, 16, "out", &out))
    return packed_fail();
  if (W.t->ndim != 2 || S.t->ndim != 2 || S.t->shape[0] != W.t->shape[0] ||
      S.t->shape[1] * 4 != W.t->shape[1] || out.numel != W.numel * 8) {
    fail(WQ_EINVAL, "%s: inconsistent shapes", who);
    return packed_fail();
  }
  const int rc = wq_q4g32_dequantize((const uint32_t*)W.ptr, (const uint16_t*)S.ptr, (uint16_t*)out.ptr,
                                     W.t->shape[0], W.t->shape[1] * 8, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (W_kn uint32 [K/8, N], S_kn fp16 [K/32, N], x fp16 [.., K], out fp16 [.., N][, workspace uint8]): the decode
// linear over a K-major checkpoint in place (buffer order of tests/python/dlight/test_gpu_reduction.py:102-107:
// weights, scales, activations, result), up to WQ_KN_GEMV_MAX_M rows.
WQ_PACKED(relax_amd_q4f16_1_kn_matmul) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_kn_matmul";
  Tensor W, S, x, out, ws;
  if (num_args != 4 && num_args != 5) {
    fail(WQ_EINVAL, "%s: expected (W_kn, S_kn, x, out[, workspace])", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W_kn", &W) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "S_kn", &S) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLFloat, 16, "x", &x) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 16, "out", &out) ||
      (num_args == 5 && !get_tensor(who, args, type_codes, num_args, 4, kDLUInt, 8, "workspace", &ws)))
    return packed_fail();
  if (W.t->ndim != 2 || S.t->ndim != 2 || x.t->ndim < 1 || S.t->shape[1] != W.t->shape[1] ||
      S.t->shape[0] * 4 != W.t->shape[0] || x.t->shape[x.t->ndim - 1] != W.t->shape[0] * 8) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (W_kn [K/8,N], S_kn [K/32,N], x [..,K])", who);
    return packed_fail();
  }
  const int64_t N = W.t->shape[1], K = W.t->shape[0] * 8, m = leading(x.t);
  if (out.numel != m * N) {
    fail(WQ_EINVAL, "%s: out must have %lld x %lld elements", who, (long long)m, (long long)N);
    return packed_fail();
  }
  const int rc = wq_q4g32_kn_gemv((const uint32_t*)W.ptr, (const uint16_t*)S.ptr, (const uint16_t*)x.ptr, nullptr, nullptr,
                                  (uint16_t*)out.ptr, m, N, K, ws.ptr, num_args == 5 ? (size_t)ws.numel : 0,
                                  current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (A fp16 [N, K]) -> (W uint32 [N, K/8], S fp16 [N, K/32]): the q4f16_1 quantizer.
WQ_PACKED(relax_amd_q4f16_1_encode) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_encode";
  Tensor A, W, S;
  if (num_args != 3) {
    fail(WQ_EINVAL, "%s: expected (A, W_out, S_out)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLFloat, 16, "A", &A) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLUInt, 32, "W_out", &W) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLFloat, 16, "S_out", &S))
    return packed_fail();
  if (A.t->ndim != 2 || W.t->ndim != 2 || S.t->ndim != 2 || W.t->shape[0] != A.t->shape[0] ||
      S.t->shape[0] != A.t->shape[0] || W.t->shape[1] * 8 != A.t->shape[1] || S.t->shape[1] * 32 != A.t->shape[1]) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (A [N,K], W [N,K/8], S [N,K/32])", who);
    return packed_fail();
  }
  const int rc = wq_q4g32_encode((const uint16_t*)A.ptr, (uint32_t*)W.ptr, (uint16_t*)S.ptr, A.t->shape[0],
                                 A.t->shape[1], current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (W uint32 [K/8, N], S fp16 [K/32, N]) -> (W uint32 [N, K/8], S fp16 [N, K/32]): K-major checkpoints.
WQ_PACKED(relax_amd_q4f16_1_kn_to_nk) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_kn_to_nk";
  Tensor Wi, Si, Wo, So;
  if (num_args != 4) {
    fail(WQ_EINVAL, "%s: expected (W_kn, S_kn, W_out, S_out)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W_kn", &Wi) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "S_kn", &Si) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLUInt, 32, "W_out", &Wo) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 16, "S_out", &So))
    return packed_fail();
  if (Wi.t->ndim != 2 || Si.t->ndim != 2 || Wo.t->ndim != 2 || So.t->ndim != 2 ||
      Si.t->shape[1] != Wi.t->shape[1] || Si.t->shape[0] * 4 != Wi.t->shape[0] ||
      Wo.t->shape[0] != Wi.t->shape[1] || Wo.t->shape[1] != Wi.t->shape[0] ||
      So.t->shape[0] != Si.t->shape[1] || So.t->shape[1] != Si.t->shape[0]) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (W_kn [K/8,N], S_kn [K/32,N], W_out [N,K/8], S_out [N,K/32])", who);
    return packed_fail();
  }
  const int rc = wq_q4g32_kn_to_nk((const uint32_t*)Wi.ptr, (const uint16_t*)Si.ptr, (uint32_t*)Wo.ptr,
                                   (uint16_t*)So.ptr, Wi.t->shape[1], Wi.t->shape[0] * 8, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// ---- q4f16_1 packed along N (tests/python/dlight/test_gpu_matmul.py:352-401) ----
// (W uint32 [K, N/8], S fp16 [K, N/32], W_out uint32 [N, K/8], ST_out fp16 [N/32, K]): the load-time rearrangement
WQ_PACKED(relax_amd_q4f16_1_ngroup_prepare) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_ngroup_prepare";
  Tensor Wi, Si, Wo, So;
  if (num_args != 4) {
    fail(WQ_EINVAL, "%s: expected (W, S, W_out, ST_out)", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W", &Wi) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "S", &Si) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLUInt, 32, "W_out", &Wo) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 16, "ST_out", &So))
    return packed_fail();
  if (Wi.t->ndim != 2 || Si.t->ndim != 2 || Wo.t->ndim != 2 || So.t->ndim != 2 || Si.t->shape[0] != Wi.t->shape[0] ||
      Si.t->shape[1] * 4 != Wi.t->shape[1] || Wo.t->shape[0] != Wi.t->shape[1] * 8 || Wo.t->shape[1] * 8 != Wi.t->shape[0] ||
      So.t->shape[0] != Si.t->shape[1] || So.t->shape[1] != Si.t->shape[0]) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (W [K,N/8], S [K,N/32], W_out [N,K/8], ST_out [N/32,K])", who);
    return packed_fail();
  }
  const int rc = wq_q4n32_prepare((const uint32_t*)Wi.ptr, (const uint16_t*)Si.ptr, (uint32_t*)Wo.ptr, (uint16_t*)So.ptr,
                                  Wi.t->shape[0], Wi.t->shape[1] * 8, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (W_nk, ST, x fp16 [.., K], bias fp16 [N] | null, residual fp16 [.., N] | null, out fp16 [.., N]): the matmul and the
// epilogue chain of the fixture (:378-401) over the prepared operands, buffer order as there.
WQ_PACKED(relax_amd_q4f16_1_ngroup_matmul_bias_residual) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.q4f16_1_ngroup_matmul_bias_residual";
  Tensor W, ST, x, bias, res, y;
  if (num_args != 6) {
    fail(WQ_EINVAL, "%s: expected (W_nk, ST, x, bias|null, residual|null, out)", who);
    return packed_fail();
  }
  const bool has_bias = type_codes[3] != kTVMNullptr, has_res = type_codes[4] != kTVMNullptr;
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W_nk", &W) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "ST", &ST) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLFloat, 16, "x", &x) ||
      (has_bias && !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 16, "bias", &bias)) ||
      (has_res && !get_tensor(who, args, type_codes, num_args, 4, kDLFloat, 16, "residual", &res)) ||
      !get_tensor(who, args, type_codes, num_args, 5, kDLFloat, 16, "out", &y))
    return packed_fail();
  if (W.t->ndim != 2 || ST.t->ndim != 2 || x.t->ndim < 1 || y.t->ndim < 1) {
    fail(WQ_EINVAL, "%s: W_nk and ST must be matrices", who);
    return packed_fail();
  }
  const int64_t N = W.t->shape[0], K = W.t->shape[1] * 8;
  const int64_t M = leading(x.t);
  if (ST.t->shape[0] * 32 != N || ST.t->shape[1] != K || x.t->shape[x.t->ndim - 1] != K || y.numel != M * N ||
      y.t->shape[y.t->ndim - 1] != N || (has_bias && bias.numel != N) || (has_res && res.numel != M * N)) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (N=%lld K=%lld M=%lld)", who, (long long)N, (long long)K, (long long)M);
    return packed_fail();
  }
  const int rc = wq_q4n32_linear((const uint32_t*)W.ptr, (const uint16_t*)ST.ptr, (const uint16_t*)x.ptr,
                                 (const uint16_t*)bias.ptr, (const uint16_t*)res.ptr, (uint16_t*)y.ptr, M, N, K,
                                 current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// ---- AutoGPTQ layers (tests/python/dlight/test_gpu_gemv.py:636-665) ----
// g_idx is uint32 in the reference's PrimFunc and int32 in AutoGPTQ checkpoints: same bytes.
static bool get_index_tensor(const char* who, TVMValue* args, int* tcodes, int n, int i, const char* what, Tensor* t) {
  const DLTensor* d = i < n && (tcodes[i] == kTVMDLTensorHandle || tcodes[i] == kTVMNDArrayHandle)
                          ? static_cast<const DLTensor*>(args[i].v_handle)
                          : nullptr;
  const int code = (d && d->dtype.code == kDLUInt) ? kDLUInt : kDLInt;
  return get_tensor(who, args, tcodes, n, i, code, 32, what, t);
}

static bool gptq_checkpoint_args(const char* who, TVMValue* args, int* tcodes, int n, Tensor* qw, Tensor* qz,
                                 Tensor* sc, Tensor* gi, int64_t* K, int64_t* N, int64_t* G) {
  if (!get_tensor(who, args, tcodes, n, 0, kDLUInt, 32, "qweight", qw) ||
      !get_tensor(who, args, tcodes, n, 1, kDLUInt, 32, "qzeros", qz) ||
      !get_tensor(who, args, tcodes, n, 2, kDLFloat, 16, "scales", sc) ||
      !get_index_tensor(who, args, tcodes, n, 3, "g_idx", gi))
    return false;
  if (qw->t->ndim != 2 || qz->t->ndim != 2 || sc->t->ndim != 2 || gi->t->ndim != 1) {
    fail(WQ_EINVAL, "%s: expected qweight [K/8,N], qzeros [G,N/8], scales [G,N], g_idx [K]", who);
    return false;
  }
  *K = qw->t->shape[0] * 8;
  *N = qw->t->shape[1];
  *G = sc->t->shape[0];
  if (sc->t->shape[1] != *N || qz->t->shape[0] != *G || qz->t->shape[1] * 8 != *N || gi->t->shape[0] != *K) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (K=%lld N=%lld G=%lld)", who, (long long)*K, (long long)*N,
         (long long)*G);
    return false;
  }
  return true;
}

// (qweight, qzeros, scales, g_idx, out fp16 [K, N]): the decode block alone.
WQ_PACKED(relax_amd_autogptq_decode) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.autogptq_decode";
  Tensor qw, qz, sc, gi, out;
  int64_t K, N, G;
  if (num_args != 5) {
    fail(WQ_EINVAL, "%s: expected (qweight, qzeros, scales, g_idx, out)", who);
    return packed_fail();
  }
  if (!gptq_checkpoint_args(who, args, type_codes, num_args, &qw, &qz, &sc, &gi, &K, &N, &G) ||
      !get_tensor(who, args, type_codes, num_args, 4, kDLFloat, 16, "out", &out))
    return packed_fail();
  if (out.numel != K * N) {
    fail(WQ_EINVAL, "%s: out must have K*N elements", who);
    return packed_fail();
  }
  const int rc = wq_gptq_dequantize((const uint32_t*)qw.ptr, (const uint32_t*)qz.ptr, (const uint16_t*)sc.ptr,
                                    (const int32_t*)gi.ptr, (uint16_t*)out.ptr, K, N, G, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (qweight, qzeros, scales, g_idx, W_out uint32 [N,K/8], SZ_out fp16 [N,G,2], perm_out int32 [K],
//  scratch int32 [1]) -> int: 1 if the matmul must be given perm_out, 0 if the rows were already in group order.
WQ_PACKED(relax_amd_autogptq_prepare) {
  (void)resource_handle;
  const char* who = "relax_amd.autogptq_prepare";
  Tensor qw, qz, sc, gi, Wo, SZ, perm, scratch;
  int64_t K, N, G;
  if (num_args != 8) {
    fail(WQ_EINVAL, "%s: expected (qweight, qzeros, scales, g_idx, W_out, SZ_out, perm_out, scratch)", who);
    return packed_fail();
  }
  if (!gptq_checkpoint_args(who, args, type_codes, num_args, &qw, &qz, &sc, &gi, &K, &N, &G) ||
      !get_tensor(who, args, type_codes, num_args, 4, kDLUInt, 32, "W_out", &Wo) ||
      !get_tensor(who, args, type_codes, num_args, 5, kDLFloat, 16, "SZ_out", &SZ) ||
      !get_tensor(who, args, type_codes, num_args, 6, kDLInt, 32, "perm_out", &perm) ||
      !get_tensor(who, args, type_codes, num_args, 7, kDLInt, 32, "scratch", &scratch))
    return packed_fail();
  if (Wo.numel != N * (K / 8) || SZ.numel != N * G * 2 || perm.numel != K || scratch.numel < 1) {
    fail(WQ_EINVAL, "%s: outputs must be W_out [N,K/8], SZ_out [N,G,2], perm_out [K], scratch [1]", who);
    return packed_fail();
  }
  int needs = 0;
  const int rc = wq_gptq_prepare((const uint32_t*)qw.ptr, (const uint32_t*)qz.ptr, (const uint16_t*)sc.ptr,
                                 (const int32_t*)gi.ptr, (uint32_t*)Wo.ptr, (uint16_t*)SZ.ptr, (int32_t*)perm.ptr,
                                 (int32_t*)scratch.ptr, &needs, K, N, G, current_stream());
  if (rc != WQ_OK) return packed_fail();
  if (out_ret_value && out_ret_tcode) {
    out_ret_value->v_int64 = needs;
    *out_ret_tcode = kTVMArgInt;
  }
  return 0;
}

// (W_nk, SZ, perm | null, x, residual | null, out [, workspace uint8]): the matmul and the add of the
// reference's PrimFunc over the prepared operands, argument order as there (weights, x, residual, out).
WQ_PACKED(relax_amd_autogptq_matmul) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.autogptq_matmul";
  Tensor W, SZ, perm, x, res, out, ws;
  if (num_args != 6 && num_args != 7) {
    fail(WQ_EINVAL, "%s: expected (W_nk, SZ, perm|null, x, residual|null, out[, workspace])", who);
    return packed_fail();
  }
  const bool has_perm = type_codes[2] != kTVMNullptr, has_res = type_codes[4] != kTVMNullptr;
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W_nk", &W) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "SZ", &SZ) ||
      (has_perm && !get_tensor(who, args, type_codes, num_args, 2, kDLInt, 32, "perm", &perm)) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 16, "x", &x) ||
      (has_res && !get_tensor(who, args, type_codes, num_args, 4, kDLFloat, 16, "residual", &res)) ||
      !get_tensor(who, args, type_codes, num_args, 5, kDLFloat, 16, "out", &out) ||
      (num_args == 7 && !get_tensor(who, args, type_codes, num_args, 6, kDLUInt, 8, "workspace", &ws)))
    return packed_fail();
  if (W.t->ndim != 2 || SZ.t->ndim != 3 || SZ.t->shape[2] != 2 || SZ.t->shape[0] != W.t->shape[0] || x.t->ndim < 1) {
    fail(WQ_EINVAL, "%s: expected W_nk [N,K/8] and SZ [N,G,2]", who);
    return packed_fail();
  }
  const int64_t N = W.t->shape[0], K = W.t->shape[1] * 8, G = SZ.t->shape[1];
  const int64_t m = leading(x.t);
  if (x.t->shape[x.t->ndim - 1] != K || out.numel != m * N || (has_perm && perm.numel != K) ||
      (has_res && res.numel != m * N)) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (m=%lld n=%lld k=%lld)", who, (long long)m, (long long)N, (long long)K);
    return packed_fail();
  }
  const int rc = wq_gptq_linear((const uint32_t*)W.ptr, (const uint16_t*)SZ.ptr, (const int32_t*)perm.ptr,
                                (const uint16_t*)x.ptr, nullptr, (const uint16_t*)res.ptr, (uint16_t*)out.ptr, m, N, K,
                                G, ws.ptr, num_args == 7 ? (size_t)ws.numel : 0, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (qweight, qzeros, scales, g_idx, W_out uint32 [N * capacity/8], SZ_out fp16 [N * capacity/32 * 2],
//  perm_out int32 [capacity]) -> int: K_padded.  Any g_idx (groups of unequal size, in any order: the
// PrimFunc indexes scales[g_idx[k], n] without restriction); capacity = perm_out's length, at least
// wq_gptq_padded_k_bound(K, G).  The outputs are filled compactly for K_padded: W [N, K_padded/8] and so on.
WQ_PACKED(relax_amd_autogptq_prepare_padded) {
  (void)resource_handle;
  const char* who = "relax_amd.autogptq_prepare_padded";
  Tensor qw, qz, sc, gi, Wo, SZ, perm;
  int64_t K, N, G;
  if (num_args != 7) {
    fail(WQ_EINVAL, "%s: expected (qweight, qzeros, scales, g_idx, W_out, SZ_out, perm_out)", who);
    return packed_fail();
  }
  if (!gptq_checkpoint_args(who, args, type_codes, num_args, &qw, &qz, &sc, &gi, &K, &N, &G) ||
      !get_tensor(who, args, type_codes, num_args, 4, kDLUInt, 32, "W_out", &Wo) ||
      !get_tensor(who, args, type_codes, num_args, 5, kDLFloat, 16, "SZ_out", &SZ) ||
      !get_tensor(who, args, type_codes, num_args, 6, kDLInt, 32, "perm_out", &perm))
    return packed_fail();
  const int64_t capacity = perm.numel;
  if (capacity % 32 != 0 || Wo.numel < N * (capacity / 8) || SZ.numel < N * (capacity / 32) * 2) {
    fail(WQ_EINVAL, "%s: outputs must hold W [N, capacity/8], SZ [N, capacity/32, 2] for capacity = len(perm_out), a multiple of 32", who);
    return packed_fail();
  }
  int64_t k_padded = 0;
  const int rc = wq_gptq_prepare_padded((const uint32_t*)qw.ptr, (const uint32_t*)qz.ptr, (const uint16_t*)sc.ptr,
                                        (const int32_t*)gi.ptr, (uint32_t*)Wo.ptr, (uint16_t*)SZ.ptr,
                                        (int32_t*)perm.ptr, capacity, &k_padded, K, N, G, current_stream());
  if (rc != WQ_OK) return packed_fail();
  if (out_ret_value && out_ret_tcode) {
    out_ret_value->v_int64 = k_padded;
    *out_ret_tcode = kTVMArgInt;
  }
  return 0;
}

// (W_nk, SZ, perm, K_padded, x fp16 [.., K], residual | null, out fp16 [.., N], workspace uint8): the matmul and
// the add over operands prepared by relax_amd.autogptq_prepare_padded (N follows from out, K from x).
WQ_PACKED(relax_amd_autogptq_matmul_padded) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.autogptq_matmul_padded";
  Tensor W, SZ, perm, x, res, out, ws;
  int64_t k_padded = 0;
  if (num_args != 8) {
    fail(WQ_EINVAL, "%s: expected (W_nk, SZ, perm, K_padded, x, residual|null, out, workspace)", who);
    return packed_fail();
  }
  const bool has_res = type_codes[5] != kTVMNullptr;
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLUInt, 32, "W_nk", &W) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLFloat, 16, "SZ", &SZ) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLInt, 32, "perm", &perm) ||
      !get_int(who, args, type_codes, num_args, 3, "K_padded", &k_padded) ||
      !get_tensor(who, args, type_codes, num_args, 4, kDLFloat, 16, "x", &x) ||
      (has_res && !get_tensor(who, args, type_codes, num_args, 5, kDLFloat, 16, "residual", &res)) ||
      !get_tensor(who, args, type_codes, num_args, 6, kDLFloat, 16, "out", &out) ||
      !get_tensor(who, args, type_codes, num_args, 7, kDLUInt, 8, "workspace", &ws))
    return packed_fail();
  if (x.t->ndim < 1 || out.t->ndim < 1) {
    fail(WQ_EINVAL, "%s: x and out need at least one dimension", who);
    return packed_fail();
  }
  const int64_t K = x.t->shape[x.t->ndim - 1], N = out.t->shape[out.t->ndim - 1];
  const int64_t m = leading(x.t);
  if (k_padded <= 0 || k_padded % 32 != 0 || perm.numel < k_padded || W.numel < N * (k_padded / 8) ||
      SZ.numel < N * (k_padded / 32) * 2 || out.numel != m * N || (has_res && res.numel != m * N)) {
    fail(WQ_EINVAL, "%s: inconsistent shapes (m=%lld n=%lld k=%lld k_padded=%lld)", who, (long long)m, (long long)N,
         (long long)K, (long long)k_padded);
    return packed_fail();
  }
  const int rc = wq_gptq_linear_padded((const uint32_t*)W.ptr, (const uint16_t*)SZ.ptr, (const int32_t*)perm.ptr,
                                       (const uint16_t*)x.ptr, nullptr, (const uint16_t*)res.ptr, (uint16_t*)out.ptr, m,
                                       N, K, k_padded, ws.ptr, (size_t)ws.numel, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

// (A fp16 [N, K]) -> (w int8 [K, N] | [K, N/2], scales fp16 [N] | [K/64, N], scratch fp32 [N]): the
// reference fixtures' `encode`; int4 and the group size follow from the output shapes.
WQ_PACKED(relax_amd_fpA_intB_encode) {
  (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;
  const char* who = "relax_amd.fpA_intB_encode";
  Tensor A, Wq, Sc, Tmp;
  if (num_args != 4) {
    fail(WQ_EINVAL, "%s: expected (A, w_out, scales_out, scratch_f32[N])", who);
    return packed_fail();
  }
  if (!get_tensor(who, args, type_codes, num_args, 0, kDLFloat, 16, "A", &A) ||
      !get_tensor(who, args, type_codes, num_args, 1, kDLInt, 8, "w_out", &Wq) ||
      !get_tensor(who, args, type_codes, num_args, 2, kDLFloat, 16, "scales_out", &Sc) ||
      !get_tensor(who, args, type_codes, num_args, 3, kDLFloat, 32, "scratch", &Tmp))
    return packed_fail();
  if (A.t->ndim != 2 || Wq.t->ndim != 2 || Wq.t->shape[0] != A.t->shape[1]) {
    fail(WQ_EINVAL, "%s: A must be [N,K] and w_out [K,N] or [K,N/2]", who);
    return packed_fail();
  }
  const int64_t N = A.t->shape[0], K = A.t->shape[1];
  int nbit;
  if (Wq.t->shape[1] == N) nbit = 8;
  else if (Wq.t->shape[1] * 2 == N) nbit = 4;
  else {
    fail(WQ_EINVAL, "%s: w_out has %lld columns for N = %lld", who, (long long)Wq.t->shape[1], (long long)N);
    return packed_fail();
  }
  int64_t group;
  if (Sc.numel == N) group = -1;
  else if (Sc.numel == (K / 64) * N) group = 64;
  else {
    fail(WQ_EINVAL, "%s: scales_out must have N or (K/64)*N elements", who);
    return packed_fail();
  }
  if (Tmp.numel < N) {
    fail(WQ_EINVAL, "%s: scratch must hold N floats", who);
    return packed_fail();
  }
  const int rc = wq_intb_encode((const uint16_t*)A.ptr, (int8_t*)Wq.ptr, (uint16_t*)Sc.ptr, (float*)Tmp.ptr, N, K,
                                group, nbit, current_stream());
  return rc == WQ_OK ? 0 : packed_fail();
}

#define WQ_DECODE_MATMUL(sym, op)                                       \
  WQ_PACKED(sym) {                                                      \
    (void)resource_handle; (void)out_ret_value; (void)out_ret_tcode;    \
    return decode_matmul(op, args, type_codes, num_args);               \
  }
#define WQ_DECODE_MATMUL_LIST(X)                                                                     \
  X(relax_amd_decode_matmul, "decode_matmul")                                                        \
  X(relax_amd_decode_matmul_bias, "decode_matmul_bias")                                              \
  X(relax_amd_decode_matmul_cast, "decode_matmul_cast")                                              \
  X(relax_amd_decode_matmul_cast_bias, "decode_matmul_cast_bias")                                    \
  X(relax_amd_decode_matmul_bias_gelu, "decode_matmul_bias_gelu")                                    \
  X(relax_amd_decode_matmul_cast_bias_gelu, "decode_matmul_cast_bias_gelu")                          \
  X(relax_amd_decode_matmul_bias_residual_add, "decode_matmul_bias_residual_add")                    \
  X(relax_amd_decode_matmul_bias_residual_multiply, "decode_matmul_bias_residual_multiply")          \
  X(relax_amd_decode_matmul_bias_residual_add_relu, "decode_matmul_bias_residual_add_relu")          \
  X(relax_amd_decode_matmul_bias_residual_multiply_relu, "decode_matmul_bias_residual_multiply_relu") \
  X(relax_amd_decode_matmul_cast_bias_residual_add, "decode_matmul_cast_bias_residual_add")          \
  X(relax_amd_decode_matmul_cast_bias_residual_multiply, "decode_matmul_cast_bias_residual_multiply") \
  X(relax_amd_decode_matmul_cast_bias_residual_add_relu, "decode_matmul_cast_bias_residual_add_relu") \
  X(relax_amd_decode_matmul_cast_bias_residual_multiply_relu,                                        \
    "decode_matmul_cast_bias_residual_multiply_relu")                                                \
  X(relax_amd_decode_matmul_bias_gelu_residual_add, "decode_matmul_bias_gelu_residual_add")          \
  X(relax_amd_decode_matmul_bias_gelu_residual_multiply, "decode_matmul_bias_gelu_residual_multiply") \
  X(relax_amd_decode_matmul_bias_gelu_residual_add_relu, "decode_matmul_bias_gelu_residual_add_relu") \
  X(relax_amd_decode_matmul_bias_gelu_residual_multiply_relu,                                        \
    "decode_matmul_bias_gelu_residual_multiply_relu")                                                \
  X(relax_amd_decode_matmul_cast_bias_gelu_residual_add, "decode_matmul_cast_bias_gelu_residual_add") \
  X(relax_amd_decode_matmul_cast_bias_gelu_residual_multiply,                                        \
    "decode_matmul_cast_bias_gelu_residual_multiply")                                                \
  X(relax_amd_decode_matmul_cast_bias_gelu_residual_add_relu,                                        \
    "decode_matmul_cast_bias_gelu_residual_add_relu")                                                \
  X(relax_amd_decode_matmul_cast_bias_gelu_residual_multiply_relu,                                   \
    "decode_matmul_cast_bias_gelu_residual_multiply_relu")

WQ_DECODE_MATMUL_LIST(WQ_DECODE_MATMUL)

}  // extern "C"

namespace {

struct Entry {
  std::string name;    // dotted global-registry name
  const char* symbol;  // exported C symbol
  WqTVMBackendPackedCFunc fn;
};

const std::vector<Entry>& table() {
  static const std::vector<Entry> t = [] {
    std::vector<Entry> v;
    v.push_back({"cutlass.ft_preprocess_weight", "cutlass_ft_preprocess_weight", cutlass_ft_preprocess_weight});
    v.push_back({"relax_amd.ft_preprocess_weight_dps", "relax_amd_ft_preprocess_weight_dps",
                 relax_amd_ft_preprocess_weight_dps});
    v.push_back({"relax_amd.q4f16_1_matmul", "relax_amd_q4f16_1_matmul", relax_amd_q4f16_1_matmul});
    v.push_back({"relax_amd.q4f16_1_matmul_bias", "relax_amd_q4f16_1_matmul_bias", relax_amd_q4f16_1_matmul_bias});
    v.push_back({"relax_amd.q4f16_1_matmul_bias_residual", "relax_amd_q4f16_1_matmul_bias_residual",
                 relax_amd_q4f16_1_matmul_bias_residual});
    v.push_back({"relax_amd.q4f16_1_decode", "relax_amd_q4f16_1_decode", relax_amd_q4f16_1_decode});
    v.push_back({"relax_amd.q4f16_1_encode", "relax_amd_q4f16_1_encode", relax_amd_q4f16_1_encode});
    v.push_back({"relax_amd.q4f16_1_kn_to_nk", "relax_amd_q4f16_1_kn_to_nk", relax_amd_q4f16_1_kn_to_nk});
    v.push_back({"relax_amd.q4f16_1_kn_matmul", "relax_amd_q4f16_1_kn_matmul", relax_amd_q4f16_1_kn_matmul});
    v.push_back({"relax_amd.q4f16_1_matmul_f16acc", "relax_amd_q4f16_1_matmul_f16acc", relax_amd_q4f16_1_matmul_f16acc});
    v.push_back({"relax_amd.q4f16_1_ngroup_prepare", "relax_amd_q4f16_1_ngroup_prepare", relax_amd_q4f16_1_ngroup_prepare});
    v.push_back({"relax_amd.q4f16_1_ngroup_matmul_bias_residual", "relax_amd_q4f16_1_ngroup_matmul_bias_residual",
                 relax_amd_q4f16_1_ngroup_matmul_bias_residual});
    v.push_back({"relax_amd.fpA_intB_encode", "relax_amd_fpA_intB_encode", relax_amd_fpA_intB_encode});
    v.push_back({"relax_amd.autogptq_decode", "relax_amd_autogptq_decode", relax_amd_autogptq_decode});
    v.push_back({"relax_amd.autogptq_prepare", "relax_amd_autogptq_prepare", relax_amd_autogptq_prepare});
    v.push_back({"relax_amd.autogptq_matmul", "relax_amd_autogptq_matmul", relax_amd_autogptq_matmul});
    v.push_back({"relax_amd.autogptq_prepare_padded", "relax_amd_autogptq_prepare_padded", relax_amd_autogptq_prepare_padded});
    v.push_back({"relax_amd.autogptq_matmul_padded", "relax_amd_autogptq_matmul_padded", relax_amd_autogptq_matmul_padded});
#define WQ_ENTRY(sym, op) v.push_back({std::string("relax_amd.") + op, #sym, sym});
    WQ_DECODE_MATMUL_LIST(WQ_ENTRY)
#undef WQ_ENTRY
    return v;
  }();
  return t;
}

// Adapter from the registry's TVMPackedCFunc (return through TVMCFuncSetReturn) to the
// exported-symbol signature (return through out pointers).
int registry_trampoline(TVMValue* args, int* type_codes, int num_args, TVMRetValueHandle ret,
                        void* resource_handle) {
  const Entry* e = static_cast<const Entry*>(resource_handle);
  TVMValue rv;
  rv.v_handle = nullptr;
  int rcode = kTVMNullptr;
  const int rc = e->fn(args, type_codes, num_args, &rv, &rcode, nullptr);
  if (rc != 0) return rc;
  if (rcode != kTVMNullptr) {
    wq::HostRuntime& h = wq::host();
    if (!h.set_return) return -1;
    return h.set_return(ret, &rv, &rcode, 1);
  }
  return 0;
}

}  // namespace

namespace wq {
// Used by the instruction-list executor (dps_program.cc).
void set_stream_override(bool on, void* stream) {
  t_stream_override_on = on;
  t_stream_override = stream;
}
// Looks a PackedFunc of this library up by its dotted global name or its C symbol.
WqTVMBackendPackedCFunc find_packed_function(const char* name) {
  for (const Entry& e : table())
    if (e.name == name || std::strcmp(e.symbol, name) == 0) return e.fn;
  return nullptr;
}
}  // namespace wq

extern "C" int wq_tvm_num_functions(void) { return (int)table().size(); }
extern "C" const char* wq_tvm_function_name(int i) {
  return i >= 0 && i < (int)table().size() ? table()[i].name.c_str() : nullptr;
}
extern "C" const char* wq_tvm_function_symbol(int i) {
  return i >= 0 && i < (int)table().size() ? table()[i].symbol : nullptr;
}
extern "C" void wq_tvm_set_stream_getter(wq_stream_getter_t getter) { wq::g_stream_getter = getter; }

extern "C" int wq_tvm_register_globals(void) {
  wq::HostRuntime& h = wq::host();
  if (!h.present) return 0;
  int n = 0;
  for (const Entry& e : table()) {
    TVMFunctionHandle f = nullptr;
    // Names of this library ("relax_amd.*") are replaced on a second call; a name that belongs
    // to the host ("cutlass.ft_preprocess_weight" of a TVM built with CUTLASS) is left alone
    // when the host already has it.
    const bool ours = e.name.rfind("relax_amd.", 0) == 0;
    if (!ours && h.func_get_global) {
      TVMFunctionHandle have = nullptr;
      if (h.func_get_global(e.name.c_str(), &have) == 0 && have) continue;
    }
    if (h.func_create(registry_trampoline, const_cast<Entry*>(&e), nullptr, &f) != 0) return -1;
    if (h.func_register(e.name.c_str(), f, /*override=*/ours ? 1 : 0) != 0) return -1;
    ++n;
  }
  return n;
}

// Registers with a TVM runtime that is already in the process when the library is loaded.
__attribute__((constructor)) static void wq_tvm_autoregister() { (void)wq_tvm_register_globals(); }
