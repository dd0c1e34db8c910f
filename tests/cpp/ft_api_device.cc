// Host code of the shape the reference emits for a decode_matmul composite
// (python/tvm/contrib/cutlass/gemm_operation.py:415-477), compiled against the
// source-compatible headers and run on device buffers: the argument lists are the
// emitted ones word for word, `nullptr, 0, stream` included.
//
// Usage: ft_api_device <case> <dir> <m> <n> <k>
//   case int8_percol : gemm_fp16_int_bias_act<uint8_t, PER_COLUMN_SCALE_ONLY>, bias, "gelu", bias_stride 0
//   case int4_fine   : gemm_fp16_int_bias_act_residual<cutlass::uint4b_t, FINEGRAINED_SCALE_ONLY>,
//                      bias, residual, "identity", "plus", "relu", group_size 64
//   case int8_nobias : gemm_fp16_int_bias_act<uint8_t, PER_COLUMN_SCALE_ONLY> with bias = nullptr
// Reads <dir>/{A,B,scales,bias,residual}.bin (raw bytes; B is the preprocessed weight) and
// writes <dir>/C.bin (fp16 [m, n]).
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "cutlass_kernels/fpA_intB_gemm.h"

namespace {

struct DLTensorLike {  // the two fields the emitted code reads
  void* data;
  int64_t* shape;
};

bool read_file(const std::string& path, std::vector<char>* out) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return false;
  fseek(f, 0, SEEK_END);
  const long n = ftell(f);
  fseek(f, 0, SEEK_SET);
  out->resize((size_t)n);
  const bool ok = fread(out->data(), 1, (size_t)n, f) == (size_t)n;
  fclose(f);
  return ok;
}

void* to_device(const std::vector<char>& h) {
  void* d = nullptr;
  if (hipMalloc(&d, h.size() ? h.size() : 1) != hipSuccess) return nullptr;
  if (hipMemcpy(d, h.data(), h.size(), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc != 6) return 2;
  const std::string which = argv[1], dir = argv[2];
  const int M = atoi(argv[3]), N = atoi(argv[4]), K = atoi(argv[5]);
  const bool int4 = which == "int4_fine";
  std::vector<char> hA, hB, hS, hBias, hRes;
  if (!read_file(dir + "/A.bin", &hA) || !read_file(dir + "/B.bin", &hB) || !read_file(dir + "/scales.bin", &hS))
    return 3;
  const bool has_bias = read_file(dir + "/bias.bin", &hBias);
  const bool has_res = read_file(dir + "/residual.bin", &hRes);
  if (hipSetDevice(0) != hipSuccess) return 4;
  hipStream_t stream_h = nullptr;
  if (hipStreamCreate(&stream_h) != hipSuccess) return 4;
  int64_t b_shape[2] = {K, int4 ? N / 2 : N};
  DLTensorLike tA{to_device(hA), nullptr}, tB{to_device(hB), b_shape}, tS{to_device(hS), nullptr};
  DLTensorLike tBias{has_bias ? to_device(hBias) : nullptr, nullptr};
  DLTensorLike tRes{has_res ? to_device(hRes) : nullptr, nullptr};
  void* dC = nullptr;
  if (hipMalloc(&dC, (size_t)M * N * 2) != hipSuccess) return 4;
  DLTensorLike tOut{dC, nullptr};
  DLTensorLike *x = &tA, *w = &tB, *scales = &tS, *bias = &tBias, *residual = &tRes, *out0 = &tOut;
  if (!x->data || !w->data || !scales->data) return 4;

  try {
    // ---- what the reference emits, with hipStream_t for cudaStream_t ----
    using namespace fastertransformer;
    int m = M;
    int k = w->shape[0];
    wq_stream_t stream = static_cast<wq_stream_t>(stream_h);
    if (which == "int8_percol") {
      constexpr auto QuantOp = cutlass::WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY;
      int n = w->shape[1] * 1;
      gemm_fp16_int_bias_act<uint8_t, QuantOp>(static_cast<cutlass::half_t*>(x->data),
                static_cast<uint8_t*>(w->data),
                static_cast<cutlass::half_t*>(scales->data),
                static_cast<cutlass::half_t*>(bias->data),
                static_cast<cutlass::half_t*>(out0->data),
                "gelu",
                m, n, k, k, 0, nullptr, 0, stream);
    } else if (which == "int8_nobias") {
      constexpr auto QuantOp = cutlass::WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY;
      int n = w->shape[1] * 1;
      gemm_fp16_int_bias_act<uint8_t, QuantOp>(static_cast<cutlass::half_t*>(x->data),
                static_cast<uint8_t*>(w->data),
                static_cast<cutlass::half_t*>(scales->data),
                nullptr,
                static_cast<cutlass::half_t*>(out0->data),
                "identity",
                m, n, k, k, 0, nullptr, 0, stream);
    } else if (which == "int4_fine") {
      constexpr auto QuantOp = cutlass::WeightOnlyQuantOp::FINEGRAINED_SCALE_ONLY;
      int n = w->shape[1] * 2;
      gemm_fp16_int_bias_act_residual<cutlass::uint4b_t, QuantOp>(static_cast<cutlass::half_t*>(x->data),
                static_cast<cutlass::uint4b_t*>(w->data),
                static_cast<cutlass::half_t*>(scales->data),
                static_cast<cutlass::half_t*>(bias->data),
                static_cast<cutlass::half_t*>(residual->data),
                static_cast<cutlass::half_t*>(out0->data), "identity", "plus", "relu",
                m, n, k, 64, nullptr, 0, stream);
    } else {
      return 2;
    }
    // an unknown activation string must surface as an exception
    bool threw = false;
    try {
      gemm_fp16_int_bias_act<uint8_t, cutlass::WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY>(
          static_cast<cutlass::half_t*>(x->data), static_cast<uint8_t*>(w->data),
          static_cast<cutlass::half_t*>(scales->data), nullptr, static_cast<cutlass::half_t*>(out0->data),
          "tanh", m, N, k, k, 0, nullptr, 0, stream);
    } catch (const std::exception&) {
      threw = true;
    }
    if (!threw) return 6;
  } catch (const std::exception& e) {
    fprintf(stderr, "error: %s\n", e.what());
    return 5;
  }
  if (hipStreamSynchronize(stream_h) != hipSuccess) return 7;
  std::vector<char> hC((size_t)M * N * 2);
  if (hipMemcpy(hC.data(), dC, hC.size(), hipMemcpyDeviceToHost) != hipSuccess) return 7;
  FILE* f = fopen((dir + "/C.bin").c_str(), "wb");
  if (!f || fwrite(hC.data(), 1, hC.size(), f) != hC.size()) return 8;
  fclose(f);
  printf("ok %s m=%d n=%d k=%d\n", which.c_str(), M, N, K);
  return 0;
}
