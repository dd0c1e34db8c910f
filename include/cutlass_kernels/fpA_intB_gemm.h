/*
 * cutlass_kernels/fpA_intB_gemm.h — source-compatible front end for host code that was
 * written against the external mixed-input GEMM library of the reference.
 *
 * The host code the reference emits for a decode_matmul composite
 * (python/tvm/contrib/cutlass/gemm_operation.py:415-477, header selected at
 * python/tvm/contrib/cutlass/gen_tensor_op.py:523-561) includes this path and calls
 *
 *   fastertransformer::gemm_fp16_int_bias_act<WeightType, QuantOp>(A, B, scales, bias, C,
 *       activation, m, n, k, group_size, bias_stride, workspace, workspace_bytes, stream);
 *   fastertransformer::gemm_fp16_int_bias_act_residual<WeightType, QuantOp>(A, B, scales, bias,
 *       residual, C, activation, binary_op, unary_op, m, n, k, group_size,
 *       workspace, workspace_bytes, stream);
 *
 * with WeightType = uint8_t | cutlass::uint4b_t and QuantOp =
 * cutlass::WeightOnlyQuantOp::{PER_COLUMN_SCALE_ONLY, FINEGRAINED_SCALE_ONLY}.
 * Putting this repository's include/ directory on the include path and linking
 * librelax_amd_wq.so makes that code run on MI355X; the only edit is the stream
 * type (hipStream_t, obtained from "runtime.get_rocm_stream").  Only the type and
 * function names the emitted code uses are provided — this is not a CUTLASS header.
 *
 * Errors throw std::runtime_error (the generated wrapper turns C++ exceptions into
 * a TVM error, include/tvm/runtime/packed_func.h:1234-1237).
 */
#ifndef RELAX_AMD_CUTLASS_KERNELS_FPA_INTB_GEMM_H_
#define RELAX_AMD_CUTLASS_KERNELS_FPA_INTB_GEMM_H_

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "../relax_amd_wq.h"

namespace cutlass {
struct half_t {
  uint16_t storage;
};
struct uint4b_t {
  uint8_t storage;  // two codes per byte
};
enum class WeightOnlyQuantOp { UNDEFINED, PER_COLUMN_SCALE_ONLY, FINEGRAINED_SCALE_ONLY };
}  // namespace cutlass

namespace fastertransformer {

namespace detail {
template <typename WeightType>
constexpr int weight_nbit() {
  static_assert(std::is_same<WeightType, uint8_t>::value || std::is_same<WeightType, cutlass::uint4b_t>::value,
                "WeightType must be uint8_t or cutlass::uint4b_t");
  return std::is_same<WeightType, uint8_t>::value ? 8 : 4;
}
inline void check(int rc) {
  if (rc != WQ_OK) throw std::runtime_error(wq_last_error());
}
inline int64_t group_arg(cutlass::WeightOnlyQuantOp op, int group_size) {
  return op == cutlass::WeightOnlyQuantOp::FINEGRAINED_SCALE_ONLY ? group_size : -1;
}
}  // namespace detail

template <typename WeightType, cutlass::WeightOnlyQuantOp QuantOp>
void gemm_fp16_int_bias_act(cutlass::half_t* A, WeightType* B, cutlass::half_t* weight_scales,
                            cutlass::half_t* bias, cutlass::half_t* C, const std::string& activation,
                            int m, int n, int k, int group_size, int bias_stride, char* workspace_ptr,
                            size_t workspace_bytes, wq_stream_t stream) {
  const int act = wq_activation_from_string(activation.c_str());
  if (act < 0) throw std::runtime_error("gemm_fp16_int_bias_act: unknown activation " + activation);
  detail::check(wq_fpA_intB_gemm(reinterpret_cast<const uint16_t*>(A), reinterpret_cast<const int8_t*>(B),
                                 reinterpret_cast<const uint16_t*>(weight_scales),
                                 reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(C), act,
                                 m, n, k, detail::group_arg(QuantOp, group_size), bias_stride,
                                 detail::weight_nbit<WeightType>(), workspace_ptr, workspace_bytes, stream));
}

template <typename WeightType, cutlass::WeightOnlyQuantOp QuantOp>
void gemm_fp16_int_bias_act_residual(cutlass::half_t* A, WeightType* B, cutlass::half_t* weight_scales,
                                     cutlass::half_t* bias, cutlass::half_t* residual, cutlass::half_t* C,
                                     const std::string& activation, const std::string& binary_op,
                                     const std::string& unary_op, int m, int n, int k, int group_size,
                                     char* workspace_ptr, size_t workspace_bytes, wq_stream_t stream) {
  const int act = wq_activation_from_string(activation.c_str());
  const int bin = wq_binary_op_from_string(binary_op.c_str());
  const int un = wq_unary_op_from_string(unary_op.c_str());
  if (act < 0 || bin < 0 || un < 0)
    throw std::runtime_error("gemm_fp16_int_bias_act_residual: unknown epilogue " + activation + "/" +
                             binary_op + "/" + unary_op);
  detail::check(wq_fpA_intB_gemm_residual(
      reinterpret_cast<const uint16_t*>(A), reinterpret_cast<const int8_t*>(B),
      reinterpret_cast<const uint16_t*>(weight_scales), reinterpret_cast<const uint16_t*>(bias),
      reinterpret_cast<const uint16_t*>(residual), reinterpret_cast<uint16_t*>(C), act, bin, un, m, n, k,
      detail::group_arg(QuantOp, group_size), detail::weight_nbit<WeightType>(), workspace_ptr,
      workspace_bytes, stream));
}

}  // namespace fastertransformer
#endif  // RELAX_AMD_CUTLASS_KERNELS_FPA_INTB_GEMM_H_
