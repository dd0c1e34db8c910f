/*
 * relax_amd_wq.h — C ABI of the MI355X (gfx950) weight-only quantized linear library.
 *
 * Plain pointers and sizes only.  All tensor pointers are DEVICE pointers unless
 * a parameter says "host".  fp16 tensors are passed as uint16_t bit patterns.
 * Every launch is asynchronous on `stream` (a hipStream_t; NULL = the default
 * stream); no entry point synchronises, allocates device memory or keeps a
 * pointer after it returns, so all of them may be captured into a HIP graph.
 *
 * Return value: 0 on success, a negative WQ_E* code on failure; the message is
 * available from wq_last_error() on the calling thread.  Nothing calls exit().
 *
 * Paths in the comments are relative to the reference tree (mlc-ai/relax).
 */
#ifndef RELAX_AMD_WQ_H_
#define RELAX_AMD_WQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Every entry point below is exported with default visibility. */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

#define WQ_OK 0
#define WQ_EINVAL (-1)   /* bad shape / pointer / enum */
#define WQ_EDEVICE (-2)  /* a HIP call failed */
#define WQ_EUNSUPPORTED (-3)

typedef void* wq_stream_t; /* hipStream_t */

/* activation / binary_op / unary_op selectors of the mixed-input GEMM epilogue;
 * the strings the reference passes ("identity", "relu", "silu", "gelu",
 * "plus", "multiply": python/tvm/contrib/cutlass/build.py:742-775) map onto these. */
enum { WQ_ACT_IDENTITY = 0, WQ_ACT_RELU = 1, WQ_ACT_SILU = 2, WQ_ACT_GELU = 3 };
enum { WQ_BIN_NONE = 0, WQ_BIN_PLUS = 1, WQ_BIN_MULTIPLY = 2 };
enum { WQ_UN_IDENTITY = 0, WQ_UN_RELU = 1 };

const char* wq_last_error(void);
int wq_abi_version(void);
/* Name of the device architecture the kernels were built for ("gfx950"). */
const char* wq_target_arch(void);

/* ------------------------------------------------------------------------- *
 * Format A — q4f16_1 group quantization.
 *   W  uint32 [N, K/8]   element k of row n = bits 4*(k%8).. of word k/8, code 0..15
 *   S  fp16   [N, K/32]  one scale per 32 consecutive k
 *   w[n,k] = (fp16(q) - 7) * S[n, k/32]      (fp16, one rounding)
 *   y[m,n] = sum_k x[m,k] * w[n,k]           (fp32 accumulate, fp16 out)
 * Replaces the generated kernels of the TIR functions in
 *   tests/python/dlight/test_gpu_reduction.py:33-51, 400-424     (M = 1)
 *   tests/python/dlight/test_gpu_low_batch_gemv.py:30-57         (small batch)
 *   tests/python/dlight/test_gpu_matmul.py:378-401               (prefill: the EPILOGUE chain only, see below)
 * which the reference schedules with python/tvm/dlight/gpu/{gemv,low_batch_gemv,matmul}.py.
 * The weight layout of that prefill fixture itself is a third scheme: its decode block
 * (test_gpu_matmul.py:366-377) reads W[k, n/8] and S[k, n/32], i.e. the codes are packed along N and a scale
 * covers 32 consecutive n of one k (rows of 32 k here, K-major words in wq_q4g32_kn_*); the square 4096 x 4096
 * shape hides the difference.  The entry points below do not take it: wq_q4n32_prepare / wq_q4n32_linear do.
 * Requirements: K % 32 == 0; W, S rows 16-byte aligned (true for K % 32 == 0
 * and 16-byte aligned bases).
 * ------------------------------------------------------------------------- */

/* q[n,k] = code (uint8 [N,K]); test_gpu_gemv.py:198 */
int wq_q4_unpack(const uint32_t* W, uint8_t* q, int64_t N, int64_t K, wq_stream_t stream);

/* out[n,k] = dequantized weight (fp16 [N,K]); the "decode" block, test_gpu_reduction.py:37-42.
 * Uses the same device function as the fused kernels below. */
int wq_q4g32_dequantize(const uint32_t* W, const uint16_t* S, uint16_t* out, int64_t N, int64_t K,
                        wq_stream_t stream);

/* y = x @ dequant(W,S)^T (+ bias[n] in fp32, then fp16, then + residual[m,n] in fp16).
 * x fp16 [M,K], y fp16 [M,N]; bias / residual may be NULL.  Chooses from the shape
 * between the decode GEMV (M <= 2), the small-batch kernel (M <= 64, or two passes
 * of it up to M = 128 on a small matrix) and the MFMA GEMM. */
int wq_q4g32_linear(const uint32_t* W, const uint16_t* S, const uint16_t* x, const uint16_t* bias,
                    const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K,
                    wq_stream_t stream);

/* The kernels behind wq_q4g32_linear, selectable for tests and measurement.
 * wq_q4g32_small_batch (M <= WQ_SMALL_BATCH_MAX_M, K % 64 == 0) streams the weights
 * once for all rows and multiplies on the matrix cores: the counterpart of
 * python/tvm/dlight/gpu/low_batch_gemv.py. */
#define WQ_GEMV_MAX_M 8
#define WQ_SMALL_BATCH_MAX_M 64
int wq_q4g32_small_batch(const uint32_t* W, const uint16_t* S, const uint16_t* x, const uint16_t* bias,
                         const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K,
                         wq_stream_t stream);
int wq_q4g32_gemv(const uint32_t* W, const uint16_t* S, const uint16_t* x, const uint16_t* bias,
                  const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K,
                  wq_stream_t stream);
int wq_q4g32_gemm(const uint32_t* W, const uint16_t* S, const uint16_t* x, const uint16_t* bias,
                  const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K,
                  wq_stream_t stream);

/* q4f16_1 weights packed along N, the scheme of tests/python/dlight/test_gpu_matmul.py:352-401 (which the
 * reference schedules with python/tvm/dlight/gpu/matmul.py):
 *   W uint32 [K, N/8], S fp16 [K, N/32],  w[k, n] = (fp16((W[k, n/8] >> 4 (n % 8)) & 15) - 7) * S[k, n/32]
 *   y[m, n] = residual[m, n] + fp16(sum_k x[m, k] w[k, n] + bias[n])     (:378-401; fp32 accumulation)
 * prepare  a load-time rearrangement (no arithmetic): W_nk uint32 [N, K/8] holds the same codes with 8 consecutive k
 *          of one column per word, ST fp16 [N/32, K] the same scales with those of a group of 32 columns contiguous
 *          along k.  K % 8 == 0, N % 32 == 0.
 * linear   over the prepared operands, any M (the fixture's n is dynamic).  More than WQ_Q4N32_GEMV_MAX_M rows: the
 *          matrix-core GEMM; every weight is the reference's fp16 value bit for bit ((code - 7) is exact, the
 *          product rounds once).  Up to 8 rows, and up to WQ_Q4N32_GEMV_MAX_M where that is the faster way (small
 *          matrices, whose GEMM fills few CUs): a streaming kernel, one pass over the weights per 4 rows of
 *          x (fewer where K > 15000), which rounds x[k] * s[k, n/32] to fp16 instead (the scales of a group of 32 columns belong to the
 *          activations there) and keeps (code - 7) exact.  K % 64 == 0, N % 32 == 0; bias fp16 [N] / residual
 *          fp16 [M, N] may be NULL.
 * The fp16 weight itself, [K, N], is what wq_q4g32_dequantize(W, S, out, K, N) returns for these operands (the
 * decode of format A with the two dimensions exchanged). */
#define WQ_Q4N32_GEMV_MAX_M 64
int wq_q4n32_prepare(const uint32_t* W, const uint16_t* S, uint32_t* W_nk, uint16_t* ST, int64_t K, int64_t N,
                     wq_stream_t stream);
int wq_q4n32_linear(const uint32_t* W_nk, const uint16_t* ST, const uint16_t* x, const uint16_t* bias,
                    const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K, wq_stream_t stream);

/* The decode GEMV with the reference's fp16 accumulation (tests/python/dlight/test_gpu_reduction.py:44-51,
 * test_gpu_gemv.py:199-206: `NT_matmul += x * decode`, everything fp16): every product and every partial
 * sum is rounded to fp16.  The order of the sum is free in the reference (its schedules reorder it) and a
 * tree here, so results agree with a sequential fp16 sum only within fp16 accumulation error.  x fp16 [M, K],
 * y fp16 [M, N]; no epilogue.  Up to 4 rows of x share one pass over the weights (the dynamic batch of
 * tests/python/dlight/test_gpu_low_batch_gemv.py:29-57); every row is summed in the order it has alone, so the
 * result of a row does not depend on M.  wq_q4g32_linear accumulates in fp32 instead. */
int wq_q4g32_gemv_f16acc(const uint32_t* W, const uint16_t* S, const uint16_t* x, uint16_t* y, int64_t M,
                         int64_t N, int64_t K, wq_stream_t stream);

/* A list of decode linears (M = 1 each) as ONE launch: what a decoder layer, or a whole stack
 * of them, asks of python/tvm/dlight/gpu/gemv.py:216-530 one generated kernel at a time.  A grid
 * of persistent workgroups walks the list; the weights of the next linear are already streaming
 * while the current one finishes, and a linear whose x is the y of an earlier linear of the list
 * (found from the addresses) waits on a device-side counter instead of a kernel boundary.
 *   create  validates, finds the dependencies, uploads the descriptor table into `workspace`
 *           (256-byte aligned device memory of wq_q4g32_gemv_list_workspace_bytes(n) bytes, owned
 *           by the caller and left alone until destroy) and synchronises `stream`: a load-time call.
 *           Outputs must not overlap any operand of an earlier linear of the list other than as that
 *           dependency (refused with WQ_EUNSUPPORTED); bias / residual must come from outside the list.
 *   run     one asynchronous launch on `stream`; no allocation, no synchronisation: capturable.
 *           Launches of one list must not overlap in time (they share the counters).
 *   status  synchronises `stream` and reports a wait that ran into the spin limit (WQ_EDEVICE):
 *           this happens only if the grid could not be resident at once, e.g. while another
 *           kernel holds CUs; the results of that launch are undefined.
 *   poll    the same check without synchronising, for a serving loop that must not stall: enqueues an
 *           asynchronous copy of the list's error word into `*host_word` (pinned host memory of the caller,
 *           e.g. from hipHostMalloc) behind the work already on `stream`.  Once the stream has passed that
 *           point the word is 0, or non-zero if a wait of an earlier launch ran out (then call status, which
 *           names the linear and resets the counters).  No allocation: capturable.
 * The kernels rely on two properties of the device that the HIP memory model does not promise.  (1) All
 * workgroups of a launch are resident at once (one per CU; sized from the occupancy the runtime reports): a
 * consumer spins on counters that workgroups on other CUs raise.  A kernel of another stream that holds CUs
 * breaks this; the spin limit turns the resulting dead wait into the error word above instead of a hang.
 * (2) A producer publishes y with device-scope (sc1) write-through stores, waits for them (vmcnt), then raises
 * its counter with a relaxed device-scope atomic; the consumer polls the counter with read-modify-write atomics
 * (performed at the memory side, never served from a stale line), takes a device-scope acquire fence and reads x
 * with sc1 loads.  There is no release fence (the L2 write-back it implies costs 9 - 17 us per linear on this
 * part).  This is the gfx950 cache hierarchy's behaviour, checked by the eager-against-replay bit-equality
 * tests of 32-layer stacks, not a guarantee of the language.
 * NULL from create / non-zero from the others: see wq_last_error(). */
typedef struct wq_q4g32_gemv_desc {
  const uint32_t* W;        /* uint32 [N, K/8] */
  const uint16_t* S;        /* fp16 [N, K/32] */
  const uint16_t* x;        /* fp16 [K] */
  const uint16_t* bias;     /* fp16 [N] or NULL */
  const uint16_t* residual; /* fp16 [N] or NULL */
  uint16_t* y;              /* fp16 [N] */
  int64_t N, K;             /* K % 32 == 0, K <= WQ_GEMV_LIST_MAX_K */
} wq_q4g32_gemv_desc;
typedef struct wq_gemv_list wq_gemv_list_t;
#define WQ_GEMV_LIST_MAX 4096
#define WQ_GEMV_LIST_MAX_K 32768
size_t wq_q4g32_gemv_list_workspace_bytes(int n);
wq_gemv_list_t* wq_q4g32_gemv_list_create(const wq_q4g32_gemv_desc* descs, int n, void* workspace,
                                          size_t workspace_bytes, wq_stream_t stream);
/* The same for M rows of activations per linear, 1 <= M <= WQ_GEMV_LIST_MAX_M (a small decode batch): x is
 * fp16 [M, K], y and residual fp16 [M, N], all contiguous; one launch runs the list on the matrix cores, one pass
 * over the weights for every M (more than 16 rows: each unpacked weight feeds two matrix-core tiles of 16
 * rows, in a kernel whose wavefronts own rows of W and keep their sums in registers over all of K).  M > 1 needs
 * K % 256 == 0 and S 16-byte aligned, M > 16 also N * K < 2^35 per linear (WQ_EUNSUPPORTED otherwise: run such a
 * list linear by linear with wq_q4g32_linear).  A short list (at most 8 independent linears at a time) gives
 * every linear a set of the 8 XCDs sized by its cost; a long one runs on equal groups of workgroups. */
#define WQ_GEMV_LIST_MAX_M 32
wq_gemv_list_t* wq_q4g32_gemv_list_create_batched(const wq_q4g32_gemv_desc* descs, int n, int M, void* workspace,
                                                  size_t workspace_bytes, wq_stream_t stream);
int wq_q4g32_gemv_list_run(wq_gemv_list_t* list, wq_stream_t stream);
int wq_q4g32_gemv_list_status(wq_gemv_list_t* list, wq_stream_t stream);
int wq_q4g32_gemv_list_poll(wq_gemv_list_t* list, int* host_word, wq_stream_t stream);
void wq_q4g32_gemv_list_destroy(wq_gemv_list_t* list);
/* How many linears of the list wait for an earlier one, and how many of those for the linear
 * directly in front of them (those cannot overlap with it; order lists to keep this number low). */
int wq_q4g32_gemv_list_info(const wq_gemv_list_t* list, int* dependencies, int* adjacent);
/* Upper bound of one wait in ticks of the 100 MHz wall clock (default 2 s). */
int wq_q4g32_gemv_list_set_spin_limit(wq_gemv_list_t* list, long long ticks);

/* ------------------------------------------------------------------------- *
 * Format B — fp16 activations x int8 / int4 weights (per-channel or group-64 scales).
 *   packed weight  int8 [K, N]   or  int4 as int8 [K, N/2] (two's complement
 *                  nibbles, low nibble = even n)
 *   w[k,n] = fp16(q) * scale            (tests/python/relax/test_codegen_cutlass.py:1371-1389, 1628, 2041)
 *   C[m,n] = act(sum_k A[m,k] w[k,n] + bias)                  fp32 accumulate, fp16 out
 * ------------------------------------------------------------------------- */

/* cutlass.ft_preprocess_weight (src/runtime/contrib/cutlass/weight_preprocess.cc:38-59):
 * reorders a packed weight into the layout the GEMM kernels read.  `rows` = K,
 * `cols` = N in ELEMENTS (the caller doubles the packed column count for int4,
 * as weight_preprocess.cc:48-50 does).  Output has the same byte size as the
 * input.  sm selects the layout family; only 75 <= sm < 90 is supported.
 * Requires rows % 64 == 0 and cols % 64 == 0.
 * _host works on host memory (what the reference does); the other one runs a
 * device kernel on device memory and never leaves the GPU. */
int wq_ft_preprocess_weight_host(int8_t* out_host, const int8_t* in_host, int64_t num_experts,
                                 int64_t rows, int64_t cols, int is_int4, int sm);
int wq_ft_preprocess_weight(int8_t* out, const int8_t* in, int64_t num_experts, int64_t rows,
                            int64_t cols, int is_int4, int sm, wq_stream_t stream);

/* Dequantized weight fp16 [K,N] from the PREPROCESSED layout (the decode
 * PrimFunc of test_codegen_cutlass.py:1359-1389 composed with the inverse of the
 * reordering).  group_size <= 0: scales [N]; group_size == 64: scales [K/64, N]. */
int wq_intb_dequantize(const int8_t* B, const uint16_t* scales, uint16_t* out, int64_t K, int64_t N,
                       int weight_nbit, int64_t group_size, wq_stream_t stream);

/* fastertransformer::gemm_fp16_int_bias_act<WeightType, QuantOp>(A, B, scales, bias, C,
 *   activation, m, n, k, group_size, bias_stride, workspace, workspace_bytes, stream)
 * — call site python/tvm/contrib/cutlass/gemm_operation.py:441-447.  Same argument
 * order; the two template parameters become weight_nbit (8 | 4) and the sign of
 * group_size (per-column when group_size <= 0 or == k, else fine-grained, 64).
 * B is the preprocessed weight.  bias may be NULL; bias_stride == 0 broadcasts
 * bias[n] over rows, otherwise bias[m*bias_stride + n].  workspace is unused. */
int wq_fpA_intB_gemm(const uint16_t* A, const int8_t* B, const uint16_t* scales,
                     const uint16_t* bias, uint16_t* C, int activation, int64_t m, int64_t n,
                     int64_t k, int64_t group_size, int64_t bias_stride, int weight_nbit,
                     void* workspace, size_t workspace_bytes, wq_stream_t stream);

/* fastertransformer::gemm_fp16_int_bias_act_residual<...>(A, B, scales, bias, residual, C,
 *   activation, binary_op, unary_op, m, n, k, group_size, workspace, workspace_bytes, stream)
 * — call site gemm_operation.py:452-458.  C = unary(binary(act(A w + bias), residual)). */
int wq_fpA_intB_gemm_residual(const uint16_t* A, const int8_t* B, const uint16_t* scales,
                              const uint16_t* bias, const uint16_t* residual, uint16_t* C,
                              int activation, int binary_op, int unary_op, int64_t m, int64_t n,
                              int64_t k, int64_t group_size, int weight_nbit, void* workspace,
                              size_t workspace_bytes, wq_stream_t stream);

/* Maps the reference's epilogue strings onto the enums above; -1 if unknown. */
int wq_activation_from_string(const char* name);
int wq_binary_op_from_string(const char* name);
int wq_unary_op_from_string(const char* name);

/* ------------------------------------------------------------------------- *
 * Quantizers (device): fp16 weights [N, K] -> packed codes + scales.
 * ------------------------------------------------------------------------- */
/* Format B, the reference fixtures' `encode`
 * (tests/python/relax/test_codegen_cutlass.py:1392-1457 int4, 1631-1676 int8, 2044-2109 group 64):
 *   scale = max(max |A|, 1e-4) * (0.125 | 0.0078125) over the row (group_size <= 0 or == K)
 *           or over each 64-k group; q = clip(round(A / scale), lo, hi), round half away
 *           from zero, float32 arithmetic.
 * w_out int8 [K, N] or packed int4 [K, N/2] (un-preprocessed: feed it to
 * wq_ft_preprocess_weight); scales fp16 [N] or [K/64, N].  scale_scratch: N floats of
 * device memory (per-channel mode only; may be NULL for group 64).  N % 64 == K % 64 == 0. */
int wq_intb_encode(const uint16_t* A, int8_t* w_out, uint16_t* scales, float* scale_scratch, int64_t N,
                   int64_t K, int64_t group_size, int weight_nbit, wq_stream_t stream);
/* Format A (q4f16_1): per group of 32 along K, scale = fp16(max(max |A|, 1e-4) / 7),
 * code = clip(round(A / scale) + 7, 0, 14); W uint32 [N, K/8], S fp16 [N, K/32].
 * Inverse of the decode in tests/python/dlight/test_gpu_gemv.py:198; the reference tree
 * has no encoder for this format, so the rounding convention is this library's. */
int wq_q4g32_encode(const uint16_t* A, uint32_t* W, uint16_t* S, int64_t N, int64_t K, wq_stream_t stream);

/* K-major q4f16_1 checkpoints (W uint32 [K/8, N], S fp16 [K/32, N]; the layout of
 * tests/python/dlight/test_gpu_reduction.py:102-120 and test_gpu_gemv.py:813-830) -> the
 * [N, K/8] / [N, K/32] layout the kernels above read.  A word holds 8 consecutive k of one
 * column in both layouts, so this is a transpose of words and scales; run it once at load
 * time.  Not in place. */
int wq_q4g32_kn_to_nk(const uint32_t* W_kn, const uint16_t* S_kn, uint32_t* W_nk, uint16_t* S_nk,
                      int64_t N, int64_t K, wq_stream_t stream);
/* The decode linear over a K-major checkpoint IN PLACE (no transposed copy): y fp16 [M, N] =
 * epilogue(x fp16 [M, K] . w) for M <= WQ_KN_GEMV_MAX_M rows, 4 rows per pass over the weights (what the
 * reference's reduction rule schedules for this layout, test_gpu_reduction.py:102-165; epilogue as
 * wq_q4g32_linear).  N % 4 == 0.  K is cut into slices over workgroups; their partial sums go through
 * `workspace` (wq_q4g32_kn_gemv_workspace_bytes, 16-byte aligned; 0 bytes when one slice covers K).  More rows
 * are refused with WQ_EUNSUPPORTED: convert once with wq_q4g32_kn_to_nk and use wq_q4g32_linear. */
#define WQ_KN_GEMV_MAX_M 16
size_t wq_q4g32_kn_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K);
int wq_q4g32_kn_gemv(const uint32_t* W_kn, const uint16_t* S_kn, const uint16_t* x, const uint16_t* bias,
                     const uint16_t* residual, uint16_t* y, int64_t M, int64_t N, int64_t K, void* workspace,
                     size_t workspace_bytes, wq_stream_t stream);

/* ------------------------------------------------------------------------- *
 * AutoGPTQ checkpoints (tests/python/dlight/test_gpu_gemv.py:636-665):
 *   qweight uint32 [K/8, N]   code of (k, n) in bits 4*(k%8).. of qweight[k/8][n]
 *   qzeros  uint32 [G, N/8]   zero of (g, n) in bits 4*(n%8).. of qzeros[g][n/8]
 *   scales  fp16   [G, N],  g_idx int32 [K] with values in [0, G)
 *   w[k,n] = (fp16(code) - (fp16(zero) + 1)) * scales[g_idx[k], n]          all in fp16
 *   y[m,n] = residual[m,n] + fp16(sum_k x[m,k] * w[k,n])
 * The reference accumulates this sum in fp16 (:653-660) and leaves the function to the
 * unscheduled fallback (:667-672); this library accumulates in fp32 like its other linears.
 * ------------------------------------------------------------------------- */
/* The fp16 weight, bit for bit, straight from the checkpoint layout: out fp16 [K, N].
 * g_idx entries outside [0, G) are clamped. */
int wq_gptq_dequantize(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                       const int32_t* g_idx, uint16_t* out, int64_t K, int64_t N, int64_t G,
                       wq_stream_t stream);
/* Load-time conversion to what wq_gptq_linear reads.  Rows are sorted by group (stable), so
 * every group becomes K/G consecutive rows:
 *   perm  int32  [K]         perm[k'] = original row at sorted position k'
 *   W_nk  uint32 [N, K/8]    codes of the sorted rows, 8 per word along K
 *   SZ    fp16   [N, G, 2]   (scale, zero + 1) per column and group
 * status_scratch: 4 bytes of device memory used during the call.  *needs_perm (host, may be
 * NULL) is set to 1 if the sorted order differs from 0..K-1; otherwise wq_gptq_linear may be
 * given perm = NULL.  Requires K % G == 0, (K/G) % 32 == 0, N % 8 == 0 and a g_idx that
 * gives each group exactly K/G rows (what AutoGPTQ writes, with or without desc_act);
 * anything else returns WQ_EUNSUPPORTED.  Synchronises the stream (it reads the check back). */
int wq_gptq_prepare(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                    const int32_t* g_idx, uint32_t* W_nk, uint16_t* SZ, int32_t* perm,
                    int32_t* status_scratch, int* needs_perm, int64_t K, int64_t N, int64_t G,
                    wq_stream_t stream);
/* The same for ANY g_idx (groups of unequal size, in any order; entries must lie in [0, G)): each group's rows,
 * in ascending k, are padded to a multiple of 32, so the prepared layer has K_padded >= K rows in sub-groups of
 * exactly 32 (K_padded <= wq_gptq_padded_k_bound(K, G), which is what the caller sizes the buffers by:
 * W_nk uint32 [N, capacity/8], SZ fp16 [N, capacity/32, 2], perm int32 [capacity]).  *K_padded receives the
 * row count; perm[k'] is the checkpoint row at position k' or -1 for padding.  A load-time call: sorts on the
 * host, allocates a temporary, synchronises the stream.  Only K % 8 == 0 and N % 8 == 0 are required. */
int64_t wq_gptq_padded_k_bound(int64_t K, int64_t G);
int wq_gptq_prepare_padded(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                           const int32_t* g_idx, uint32_t* W_nk, uint16_t* SZ, int32_t* perm, int64_t capacity,
                           int64_t* K_padded, int64_t K, int64_t N, int64_t G, wq_stream_t stream);
/* The linear over operands prepared by wq_gptq_prepare_padded: x fp16 [M, K] is gathered into the workspace
 * (M * K_padded * 2 bytes, 16-byte aligned; zeros at the padding), then the kernels of wq_gptq_linear run with
 * K_padded rows in groups of 32.  K_padded <= 32768.  K is the row length of x: an entry of perm that is not
 * below K (operands prepared for a wider checkpoint) gathers a zero, it never reads beyond the row. */
size_t wq_gptq_padded_workspace_bytes(int64_t M, int64_t K_padded);
int wq_gptq_linear_padded(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                          const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                          int64_t K, int64_t K_padded, void* workspace, size_t workspace_bytes, wq_stream_t stream);
/* Bytes of workspace wq_gptq_linear needs: M*K*2 for the gathered activations when a row
 * order is given, else 0. */
size_t wq_gptq_workspace_bytes(int64_t M, int64_t K, int has_perm);
/* y fp16 [M, N] = epilogue(x fp16 [M, K] . w) over the prepared operands; bias fp16 [N] and
 * residual fp16 [M, N] may be NULL (epilogue as wq_q4g32_linear).  perm may be NULL (rows
 * already in group order); with a row order the activations are first gathered into the
 * workspace (16-byte aligned, wq_gptq_workspace_bytes).  M <= 2 streams the weights once,
 * M <= WQ_SMALL_BATCH_MAX_M runs the small-batch kernel (K % 64 == 0), larger M the MFMA GEMM
 * (group size % 64 == 0); shapes outside those conditions repeat the streaming kernel. */
int wq_gptq_linear(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                   const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                   int64_t K, int64_t G, void* workspace, size_t workspace_bytes, wq_stream_t stream);

/* A list of prepared AutoGPTQ layers at M = 1 as ONE launch: wq_q4g32_gemv_list_create for the layers of
 * tests/python/dlight/test_gpu_gemv.py:636-665, which the reference's GEMV rule leaves unscheduled (:667-672).
 * Same kernel design, workspace of wq_gptq_gemv_list_workspace_bytes (the plain size of
 * wq_q4g32_gemv_list_workspace_bytes is accepted as well), and the list is run, checked and
 * destroyed with the wq_q4g32_gemv_list_* calls above; arithmetic as wq_gptq_linear at M = 1.  W_nk / SZ from
 * wq_gptq_prepare; perm is the row order it wrote when it reported *needs_perm = 1 (16-byte aligned), else NULL:
 * the activations of such a layer are gathered through it while they are staged, inside the launch, so x is always
 * the layer's input in checkpoint order, fp16 [K]; y fp16 [N].  The group size K / G must be 32 << t, t = 0 .. 6
 * (WQ_EUNSUPPORTED otherwise); operands of wq_gptq_prepare_padded are not accepted. */
typedef struct wq_gptq_gemv_desc {
  const uint32_t* W_nk;     /* uint32 [N, K/8] */
  const uint16_t* SZ;       /* fp16 [N, G, 2] */
  const int32_t* perm;      /* int32 [K] or NULL */
  const uint16_t* x;        /* fp16 [K] */
  const uint16_t* bias;     /* fp16 [N] or NULL */
  const uint16_t* residual; /* fp16 [N] or NULL */
  uint16_t* y;              /* fp16 [N] */
  int64_t N, K, G;          /* K % 32 == 0, K <= WQ_GEMV_LIST_MAX_K */
} wq_gptq_gemv_desc;
/* Workspace for a list with row orders: wq_q4g32_gemv_list_workspace_bytes(n) plus room for the gathered activations
 * of every layer that has one.  With that much workspace a layer with a row order whose x comes from outside the list
 * has its activations gathered by a small kernel that wq_q4g32_gemv_list_run launches in front of the list kernel
 * (two launches then, still capturable); with only the plain size, and for a layer fed by another linear of the
 * list, the gather happens inside the list kernel while the activations are staged (slower by about 3 us a layer). */
size_t wq_gptq_gemv_list_workspace_bytes(const wq_gptq_gemv_desc* descs, int n);
wq_gemv_list_t* wq_gptq_gemv_list_create(const wq_gptq_gemv_desc* descs, int n, void* workspace,
                                         size_t workspace_bytes, wq_stream_t stream);

/* wq_gptq_linear for callers that cannot allocate device memory and have no workspace to
 * pass (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same arguments and results as wq_gptq_linear without the
 * workspace: with a row order the gathered activations go to a buffer built into the library
 * (WQ_GPTQ_NOALLOC_MAX_BYTES of device memory per GPU, held until the process ends), so
 * M*K*2 must not exceed that size; larger problems are refused with WQ_EINVAL.  The call
 * allocates nothing.  Every call on a GPU shares that GPU's buffer: calls that overlap in time
 * on one GPU (different streams) race; calls on one stream are ordered.
 * The first call with a row order on a device looks the buffer's address up (hipGetSymbolAddress,
 * which may load the code object): make that call outside a stream capture.  A call with M = 0
 * and a non-null perm does the look-up and nothing else. */
#define WQ_GPTQ_NOALLOC_MAX_BYTES (1u << 20)
int wq_gptq_linear_noalloc(const uint32_t* W_nk, const uint16_t* SZ, const int32_t* perm, const uint16_t* x,
                           const uint16_t* bias, const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                           int64_t K, int64_t G, wq_stream_t stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_WQ_H_ */
