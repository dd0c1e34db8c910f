/*
 * relax_amd_tvm.h — PackedFunc symbols exported by librelax_amd_wq.so.
 *
 * Every function has the TVMBackendPackedCFunc signature
 * (include/tvm/runtime/c_backend_api.h:49-51) and the destination-passing
 * convention of R.call_dps_packed (src/relax/op/op.cc:556-595,
 * src/relax/transform/call_tir_rewrite.cc:62-168): inputs first, then the
 * pre-allocated output; tensors arrive as DLTensor* / NDArray handles
 * (type code 7 or 13), ints and bools as type code 0.  Kernels are
 * enqueued on the runtime's current stream (global "runtime.get_rocm_stream",
 * src/runtime/rocm/rocm_device_api.cc:263-265) or on the null stream when no
 * TVM runtime is loaded.  Errors: message through TVMAPISetLastError (when the
 * runtime is present) and wq_last_error(), return -1.
 *
 * When the library is loaded into a process that already holds libtvm_runtime
 * (or when wq_tvm_register_globals() is called later) the functions are also
 * registered in TVM's global registry under the dotted names given below.
 */
#ifndef RELAX_AMD_TVM_H_
#define RELAX_AMD_TVM_H_

#include "relax_amd_tvm_abi.h"

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

#define WQ_PACKED(name)                                                                      \
  int name(TVMValue* args, int* type_codes, int num_args, TVMValue* out_ret_value,           \
           int* out_ret_tcode, void* resource_handle)

/* "cutlass.ft_preprocess_weight"(NDArray packed_weight, int sm, bool is_int4) -> NDArray
 * Same name and arguments as src/runtime/contrib/cutlass/weight_preprocess.cc:38-59.
 * The result is allocated with the host runtime's TVMArrayAlloc; device weights are
 * reordered on the device, host (kDLCPU) weights on the host. */
WQ_PACKED(cutlass_ft_preprocess_weight);
/* "relax_amd.ft_preprocess_weight_dps"(packed_weight, sm, is_int4, out): destination-passing
 * twin for callers without a TVM allocator. */
WQ_PACKED(relax_amd_ft_preprocess_weight_dps);

/* Format A (q4f16_1).  Buffer order of the reference's PrimFuncs
 * (tests/python/dlight/test_gpu_gemv.py:189, test_gpu_matmul.py:352; of the latter the argument order and the
 * epilogue chain :378-401 only: its weights are packed along N, W[k, n/8], which the q4f16_1_ngroup pair below takes):
 * "relax_amd.q4f16_1_matmul"(W u32[N,K/8], S f16[N,K/32], x f16[..,K], out f16[..,N])
 * "relax_amd.q4f16_1_matmul_bias"(W, S, x, bias f16[N], out)
 * "relax_amd.q4f16_1_matmul_bias_residual"(W, S, x, bias f16[N], residual f16[..,N], out) */
WQ_PACKED(relax_amd_q4f16_1_matmul);
WQ_PACKED(relax_amd_q4f16_1_matmul_bias);
WQ_PACKED(relax_amd_q4f16_1_matmul_bias_residual);
/* "relax_amd.q4f16_1_matmul_f16acc"(W, S, x f16[..,K], out f16[..,N]): the matmul with the fp16 accumulation of the
 * decode fixtures (tests/python/dlight/test_gpu_reduction.py:44-51, test_gpu_low_batch_gemv.py:50-57); a decode /
 * low-batch entry (wq_q4g32_gemv_f16acc), no epilogue. */
WQ_PACKED(relax_amd_q4f16_1_matmul_f16acc);
/* "relax_amd.q4f16_1_decode"(W, S, out f16[N,K]): the decode block alone. */
WQ_PACKED(relax_amd_q4f16_1_decode);
/* Weight preparation, destination-passing:
 *   relax_amd.q4f16_1_encode    (A fp16 [N,K], W_out uint32 [N,K/8], S_out fp16 [N,K/32])
 *   relax_amd.q4f16_1_kn_to_nk  (W_kn uint32 [K/8,N], S_kn fp16 [K/32,N], W_out [N,K/8], S_out [N,K/32])
 *   relax_amd.fpA_intB_encode   (A fp16 [N,K], w_out int8 [K,N] | [K,N/2], scales_out fp16 [N] | [K/64,N],
 *                                scratch fp32 [N]) — the fixtures' encode
 *                                (tests/python/relax/test_codegen_cutlass.py:1392-1457, 1631-1676, 2044-2109) */
WQ_PACKED(relax_amd_q4f16_1_encode);
WQ_PACKED(relax_amd_q4f16_1_kn_to_nk);
/* q4f16_1 packed along N, the operands of tests/python/dlight/test_gpu_matmul.py:352-401 (W u32[K,N/8], S f16[K,N/32]):
 * "relax_amd.q4f16_1_ngroup_prepare"(W, S, W_out u32[N,K/8], ST_out f16[N/32,K]): load-time rearrangement;
 * "relax_amd.q4f16_1_ngroup_matmul_bias_residual"(W_nk, ST, x f16[..,K], bias f16[N] | null, residual f16[..,N] | null,
 * out f16[..,N]): the matmul and the fixture's epilogue chain, buffer order as there. */
WQ_PACKED(relax_amd_q4f16_1_ngroup_prepare);
WQ_PACKED(relax_amd_q4f16_1_ngroup_matmul_bias_residual);
/* "relax_amd.q4f16_1_kn_matmul"(W_kn u32[K/8,N], S_kn f16[K/32,N], x f16[..,K], out f16[..,N][, workspace u8]):
 * the decode linear over a K-major checkpoint in place (tests/python/dlight/test_gpu_reduction.py:102-165), up to
 * WQ_KN_GEMV_MAX_M rows; workspace >= wq_q4g32_kn_gemv_workspace_bytes(M, N, K) bytes where that is not 0. */
WQ_PACKED(relax_amd_q4f16_1_kn_matmul);
WQ_PACKED(relax_amd_fpA_intB_encode);

/* AutoGPTQ layers (tests/python/dlight/test_gpu_gemv.py:636-665: qweight u32[K/8,N], qzeros u32[G,N/8],
 * scales f16[G,N], g_idx u32|i32[K]).  The reference leaves this PrimFunc unscheduled (:667-672).
 *   relax_amd.autogptq_decode   (qweight, qzeros, scales, g_idx, out f16[K,N])        the decode block
 *   relax_amd.autogptq_prepare  (qweight, qzeros, scales, g_idx, W_out u32[N,K/8], SZ_out f16[N,G,2],
 *                                perm_out i32[K], scratch i32[1]) -> int               load time; 1 = pass
 *                                perm_out to the matmul, 0 = rows already in group order
 *   relax_amd.autogptq_matmul   (W_nk, SZ, perm | null, x f16[..,K], residual | null, out f16[..,N]
 *                                [, workspace u8 >= M*K*2 bytes, needed with perm])    matmul + T_add
 * autogptq_prepare wants groups of equal size; the PrimFunc reads scales[g_idx[k], n] for ANY g_idx (:645-648),
 * which the padded pair serves (each group's rows padded to a multiple of 32):
 *   relax_amd.autogptq_prepare_padded (qweight, qzeros, scales, g_idx, W_out u32[N*cap/8], SZ_out f16[N*cap/32*2],
 *                                perm_out i32[cap]) -> int K_padded        load time; cap = len(perm_out)
 *                                >= wq_gptq_padded_k_bound(K, G); outputs compact for K_padded
 *   relax_amd.autogptq_matmul_padded  (W_nk, SZ, perm, K_padded, x f16[..,K], residual | null, out f16[..,N],
 *                                workspace u8 >= wq_gptq_padded_workspace_bytes(M, K_padded)) */
WQ_PACKED(relax_amd_autogptq_decode);
WQ_PACKED(relax_amd_autogptq_prepare);
WQ_PACKED(relax_amd_autogptq_matmul);
WQ_PACKED(relax_amd_autogptq_prepare_padded);
WQ_PACKED(relax_amd_autogptq_matmul_padded);

/* Format B composites, one per pattern name of
 * python/tvm/relax/backend/contrib/cutlass.py:305-312, 344-372.  Arguments are the
 * composite's parameters in their Relax order followed by the output:
 *   (x, w_preprocessed, scales, [bias], [residual], out)
 * weight_nbit, group size, M and the bias stride are derived from the shapes
 * exactly as python/tvm/contrib/cutlass/build.py:701-777 does.  Registered as
 * "relax_amd.<name>", e.g. "relax_amd.decode_matmul_bias_gelu". */
WQ_PACKED(relax_amd_decode_matmul);
WQ_PACKED(relax_amd_decode_matmul_bias);
WQ_PACKED(relax_amd_decode_matmul_cast);
WQ_PACKED(relax_amd_decode_matmul_cast_bias);
WQ_PACKED(relax_amd_decode_matmul_bias_gelu);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_gelu);
WQ_PACKED(relax_amd_decode_matmul_bias_residual_add);
WQ_PACKED(relax_amd_decode_matmul_bias_residual_multiply);
WQ_PACKED(relax_amd_decode_matmul_bias_residual_add_relu);
WQ_PACKED(relax_amd_decode_matmul_bias_residual_multiply_relu);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_residual_add);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_residual_multiply);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_residual_add_relu);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_residual_multiply_relu);
WQ_PACKED(relax_amd_decode_matmul_bias_gelu_residual_add);
WQ_PACKED(relax_amd_decode_matmul_bias_gelu_residual_multiply);
WQ_PACKED(relax_amd_decode_matmul_bias_gelu_residual_add_relu);
WQ_PACKED(relax_amd_decode_matmul_bias_gelu_residual_multiply_relu);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_gelu_residual_add);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_gelu_residual_multiply);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_gelu_residual_add_relu);
WQ_PACKED(relax_amd_decode_matmul_cast_bias_gelu_residual_multiply_relu);

/* Registers every function above in the TVM global registry of the current
 * process (TVMFuncCreateFromCFunc + TVMFuncRegisterGlobal, looked up with
 * dlsym).  Returns the number of names registered, 0 when no TVM runtime is
 * loaded, -1 on error.  Called automatically when the library is loaded.  The
 * "relax_amd.*" names replace an earlier registration of the same name; the host's own
 * name "cutlass.ft_preprocess_weight" is registered only when the host does not have it
 * (a TVM built with its CUTLASS back end keeps its function). */
int wq_tvm_register_globals(void);

/* Number of PackedFunc names and the i-th dotted name / C symbol (for tools and tests). */
int wq_tvm_num_functions(void);
const char* wq_tvm_function_name(int i);
const char* wq_tvm_function_symbol(int i);

/* The stream kernels are enqueued on when called through the PackedFunc layer:
 * NULL selects "ask the TVM runtime, else the null stream"; a non-NULL getter
 * overrides it (used by hosts that manage their own streams). */
typedef void* (*wq_stream_getter_t)(void);
void wq_tvm_set_stream_getter(wq_stream_getter_t getter);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_TVM_H_ */
