// Compiles against the source-compatible headers exactly as host code written for
// the reference's external library would, and exercises the host-only part
// (weight reordering) so that it can run without a GPU.  Usage: ft_api_host <in> <out> <rows> <cols> <is_int4>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "cutlass_kernels/cutlass_preprocessors.h"
#include "cutlass_kernels/fpA_intB_gemm.h"

// Instantiating the templates the emitted code uses proves they compile and link.
using fastertransformer::gemm_fp16_int_bias_act;
using fastertransformer::gemm_fp16_int_bias_act_residual;
constexpr auto kPerCol = cutlass::WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY;
constexpr auto kFine = cutlass::WeightOnlyQuantOp::FINEGRAINED_SCALE_ONLY;
auto* f1 = &gemm_fp16_int_bias_act<uint8_t, kPerCol>;
auto* f2 = &gemm_fp16_int_bias_act<cutlass::uint4b_t, kFine>;
auto* f3 = &gemm_fp16_int_bias_act_residual<cutlass::uint4b_t, kPerCol>;

int main(int argc, char** argv) {
  if (argc != 6) return 2;
  const size_t rows = atol(argv[3]), cols = atol(argv[4]);
  const bool is_int4 = atoi(argv[5]) != 0;
  const size_t bytes = rows * cols / (is_int4 ? 2 : 1);
  std::vector<int8_t> in(bytes), out(bytes);
  FILE* f = fopen(argv[1], "rb");
  if (!f || fread(in.data(), 1, bytes, f) != bytes) return 3;
  fclose(f);
  try {
    fastertransformer::preprocess_weights(out.data(), in.data(), 1, rows, cols, is_int4, 80);
  } catch (const std::exception& e) {
    fprintf(stderr, "error: %s\n", e.what());
    return 4;
  }
  f = fopen(argv[2], "wb");
  fwrite(out.data(), 1, bytes, f);
  fclose(f);
  // an unsupported arch must surface as an exception, not as a crash
  try {
    fastertransformer::preprocess_weights(out.data(), in.data(), 1, rows, cols, is_int4, 70);
    return 5;
  } catch (const std::exception&) {
  }
  printf("ok %p %p %p\n", (void*)f1, (void*)f2, (void*)f3);
  return 0;
}
