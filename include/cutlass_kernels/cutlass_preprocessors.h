/*
 * cutlass_kernels/cutlass_preprocessors.h — source-compatible declaration of
 *   fastertransformer::preprocess_weights(out, in, num_experts, rows, cols, is_int4, arch)
 * as called by src/runtime/contrib/cutlass/weight_preprocess.cc:53 of the reference.
 * With this repository's include/ directory on the include path that file compiles
 * unchanged and links against librelax_amd_wq.so.  Host memory in, host memory out;
 * `cols` counts unpacked elements; arch must select the sm 75..89 layout family.
 */
#ifndef RELAX_AMD_CUTLASS_KERNELS_CUTLASS_PREPROCESSORS_H_
#define RELAX_AMD_CUTLASS_KERNELS_CUTLASS_PREPROCESSORS_H_

#include <cstddef>
#include <cstdint>
#include <stdexcept>

#include "../relax_amd_wq.h"

namespace fastertransformer {

inline void preprocess_weights(int8_t* preprocessed_quantized_weight, const int8_t* row_major_quantized_weight,
                               size_t num_experts, size_t rows, size_t cols, bool is_int4, int arch) {
  const int rc = wq_ft_preprocess_weight_host(preprocessed_quantized_weight, row_major_quantized_weight,
                                              (int64_t)num_experts, (int64_t)rows, (int64_t)cols,
                                              is_int4 ? 1 : 0, arch);
  if (rc != WQ_OK) throw std::runtime_error(wq_last_error());
}

}  // namespace fastertransformer
#endif  // RELAX_AMD_CUTLASS_KERNELS_CUTLASS_PREPROCESSORS_H_
