/*
 * CPU oracle for Relax's weight-only quantized linear path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * arithmetic the reference defines for this path; only the tests, the smoke
 * check and the benchmark's cpu_baseline leg may load it, and only as the
 * checker.  Nothing in the shipped library links or calls it.
 *
 * Every function cites the reference text it follows (paths relative to the
 * reference tree).  What pins each function is listed beside it:
 *
 *   wqo_f16_to_f32 / wqo_f32_to_f16      exhaustive / dense comparison with
 *                                        numpy.float16 (independent library);
 *                                        semantics: round-to-nearest-even as in
 *                                        3rdparty/compiler-rt/builtin_fp16.h:65-165
 *   wqo_q4_unpack                        brute force over 16 codes x 8 slots,
 *                                        pack/unpack round trip
 *   wqo_q4g32_dequant                    exhaustive 16 codes x 65536 scale bit
 *                                        patterns against numpy.float16 arithmetic
 *   wqo_intb_dequant                     exhaustive 256 (16) codes x 65536 scales
 *   wqo_*_matmul*                        float64 matmul over the bit-exact
 *                                        dequantized weights, one-hot selection,
 *                                        zero-code and linearity invariants
 *   wqo_ft_preprocess                    golden vectors produced by an independent
 *                                        restatement of the same published layout
 *                                        that ships in the PyTorch wheel
 *                                        (torch/quantization/_quantized_conversions.py),
 *                                        bijection / +bias / inverse round trip.
 *                                        The upstream implementation itself
 *                                        (tlc-pack/cutlass_fpA_intB_gemm, an empty
 *                                        submodule, no pinned revision) is absent:
 *                                        the layout is pinned for sm in [75, 90) only.
 *   wqo_intb_encode[_grouped]            closed form (numpy restatement in float32 with
 *                                        half-away-from-zero rounding), full-scale and
 *                                        hand cases
 *   wqo_q4g32_encode                     PARITY UNPINNED: the q4f16_1 quantizer is not in
 *                                        the reference tree (only its decode side is);
 *                                        the definition used is stated at the function
 *                                        and checked through decode(encode(w)) error
 *                                        bounds, code range and a numpy restatement
 *   wqo_gptq_dequant                     a hand-computed case, exhaustive 16 codes x 16
 *                                        zero points x every scale bit pattern against
 *                                        numpy.float16 arithmetic, reduction to the pinned
 *                                        K-major q4f16_1 decode when every zero point is 6
 *                                        and g_idx[k] = k / 32, and equivariance under a
 *                                        permutation of the K rows together with g_idx
 *   wqo_kn_matmul                        float64 matmul over the dequantized weights
 *                                        (fp32 mode), a sequential numpy.float16 loop on
 *                                        small cases (fp16 mode), one-hot selection
 *
 * Build: see oracle/Makefile (gcc -O3 -mavx2 -mfma -mf16c -fopenmp).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__F16C__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------ */
/* binary16 <-> binary32, portable bit-level versions                  */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Widening is exact.  Subnormal halves are rebuilt by an integer->float
 * conversion times 2^-24, which is exact for an 10-bit integer. */
float wqo_f16_to_f32_portable(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0) {
    float v = (float)m * 5.9604644775390625e-08f; /* 2^-24 */
    return bits_f32(f32_bits(v) | sign);
  }
  if (e == 31) return bits_f32(sign | 0x7f800000u | (m << 13));
  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* Narrowing with round-to-nearest, ties-to-even; overflow goes to infinity,
 * underflow through the subnormals to signed zero, NaNs stay quiet NaNs. */
uint16_t wqo_f32_to_f16_portable(float f) {
  uint32_t u = f32_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536, incl. inf */
  if (a >= 0x38800000u) {                                  /* normal half */
    uint32_t r = a - 0x38000000u;                          /* rebias 127 -> 15 */
    uint32_t keep = r >> 13, rest = r & 0x1fffu;
    if (rest > 0x1000u || (rest == 0x1000u && (keep & 1u))) keep++;
    return (uint16_t)(sign | keep); /* a carry into the exponent is the right answer,
                                       including the step up to infinity */
  }
  if (a < 0x33000000u) return sign; /* below 2^-25: rounds to zero */
  /* subnormal half: value = sig * 2^(e-150); the half's unit is 2^-24 */
  uint32_t e = a >> 23;
  uint32_t sig = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift = 126u - e; /* 14 .. 24 */
  uint32_t keep = sig >> shift;
  uint32_t rest = sig & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1u);
  if (rest > half || (rest == half && (keep & 1u))) keep++;
  return (uint16_t)(sign | keep);
}

static inline float h2f(uint16_t h) {
#if defined(__F16C__)
  return _cvtsh_ss(h);
#else
  return wqo_f16_to_f32_portable(h);
#endif
}
static inline uint16_t f2h(float f) {
#if defined(__F16C__)
  return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
#else
  return wqo_f32_to_f16_portable(f);
#endif
}

/* The versions the rest of the oracle uses (hardware F16C when compiled in). */
float wqo_f16_to_f32(uint16_t h) { return h2f(h); }
uint16_t wqo_f32_to_f16(float f) { return f2h(f); }

void wqo_f16_to_f32_array(const uint16_t* h, float* out, int64_t n, int portable) {
  for (int64_t i = 0; i < n; ++i) out[i] = portable ? wqo_f16_to_f32_portable(h[i]) : h2f(h[i]);
}
void wqo_f32_to_f16_array(const float* f, uint16_t* out, int64_t n, int portable) {
  for (int64_t i = 0; i < n; ++i) out[i] = portable ? wqo_f32_to_f16_portable(f[i]) : f2h(f[i]);
}

/* fp16 arithmetic as the llvm CPU target performs it: widen, operate in
 * binary32, narrow (src/runtime/builtin_fp16.cc:31-41).  For + - * of two
 * halves the binary32 result rounds to the correctly rounded half. */
static inline uint16_t h_mul(uint16_t a, uint16_t b) { return f2h(h2f(a) * h2f(b)); }
static inline uint16_t h_add(uint16_t a, uint16_t b) { return f2h(h2f(a) + h2f(b)); }
static inline uint16_t h_sub(uint16_t a, uint16_t b) { return f2h(h2f(a) - h2f(b)); }

/* ------------------------------------------------------------------ */
/* Format A: q4f16_1 group quantization (uint32 [N, K/8], group 32)     */
/* ------------------------------------------------------------------ */

/* tests/python/dlight/test_gpu_gemv.py:198, test_gpu_reduction.py:42:
 *   q[n,k] = (W[n, k/8] >> ((k%8)*4)) & 15                               */
void wqo_q4_unpack(const uint32_t* W, uint8_t* q, int64_t N, int64_t K) {
  int64_t kw = K / 8;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k)
      q[n * K + k] = (uint8_t)((W[n * kw + k / 8] >> ((uint32_t)(k % 8) * 4u)) & 15u);
}

/* Inverse of the above (used by tests and input generators only). */
void wqo_q4_pack(const uint8_t* q, uint32_t* W, int64_t N, int64_t K) {
  int64_t kw = K / 8;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t j = 0; j < kw; ++j) {
      uint32_t w = 0;
      for (int i = 0; i < 8; ++i) w |= (uint32_t)(q[n * K + j * 8 + i] & 15u) << (4 * i);
      W[n * kw + j] = w;
    }
}

/* tests/python/dlight/test_gpu_reduction.py:42 (and :411):
 *   B[n,k] = (fp16(q) - fp16(7)) * S[n, k/32]           all in fp16.
 * Two-stage form, same value: test_gpu_low_batch_gemv.py:38-49.            */
void wqo_q4g32_dequant(const uint32_t* W, const uint16_t* S, uint16_t* out, int64_t N, int64_t K) {
  int64_t kw = K / 8, kg = K / 32;
  const uint16_t seven = 0x4700u; /* 7.0 */
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      uint32_t code = (W[n * kw + k / 8] >> ((uint32_t)(k % 8) * 4u)) & 15u;
      uint16_t qh = f2h((float)code);
      out[n * K + k] = h_mul(h_sub(qh, seven), S[n * kg + k / 32]);
    }
}

/* fp32-accumulate matmul over an already dequantized fp16 weight [N,K]:
 * tests/python/dlight/test_gpu_reduction.py:411-424
 *   C_fp32[n] += f32(V[k]) * f32(B[n,k]);  C[n] = fp16(C_fp32[n])
 * with the prefill epilogue of tests/python/dlight/test_gpu_matmul.py:378-401
 *   t = matmul_f32 + f32(bias[n]);  h = fp16(t);  out = h + residual  (fp16 add)
 * bias / residual may be NULL.  k runs in ascending order, single accumulator,
 * which is what the unscheduled loop nest does.  nthreads > 1 parallelises
 * over rows of the output only (no change in any sum).                      */
void wqo_nt_matmul_f32acc(const uint16_t* Bdeq, const uint16_t* X, const uint16_t* bias,
                          const uint16_t* residual, uint16_t* Y, int64_t M, int64_t N, int64_t K,
                          int nthreads) {
  float* xf = (float*)malloc(sizeof(float) * (size_t)(M * K));
  for (int64_t i = 0; i < M * K; ++i) xf[i] = h2f(X[i]);
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    const uint16_t* brow = Bdeq + n * K;
    for (int64_t m = 0; m < M; ++m) {
      const float* xr = xf + m * K;
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) acc = acc + xr[k] * h2f(brow[k]);
      if (bias) acc = acc + h2f(bias[n]);
      uint16_t h = f2h(acc);
      if (residual) h = h_add(h, residual[m * N + n]);
      Y[m * N + n] = h;
    }
  }
  free(xf);
}

/* fp16-accumulate variant: tests/python/dlight/test_gpu_reduction.py:44-51
 *   C[n] = C[n] + V[k] * B[n,k]      every product and every sum rounded to fp16 */
void wqo_nt_matmul_f16acc(const uint16_t* Bdeq, const uint16_t* X, uint16_t* Y, int64_t M,
                          int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      uint16_t acc = 0;
      for (int64_t k = 0; k < K; ++k) acc = h_add(acc, h_mul(X[m * K + k], Bdeq[n * K + k]));
      Y[m * N + n] = acc;
    }
}

/* The whole reference CPU path for one Format-A linear, as the llvm target
 * runs it (two passes: materialise the dequantized weight, then the naive
 * loop nest).  This is the function the benchmark times as the CPU baseline. */
void wqo_q4g32_linear(const uint32_t* W, const uint16_t* S, const uint16_t* X,
                      const uint16_t* bias, const uint16_t* residual, uint16_t* Y, int64_t M,
                      int64_t N, int64_t K, int nthreads) {
  uint16_t* B = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(N * K));
  /* the decode pass row by row (rows are independent: same values with any thread count) */
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t n = 0; n < N; ++n) wqo_q4g32_dequant(W + n * (K / 8), S + n * (K / 32), B + n * K, 1, K);
  wqo_nt_matmul_f32acc(B, X, bias, residual, Y, M, N, K, nthreads);
  free(B);
}

/* ------------------------------------------------------------------ */
/* Format B: fpA_intB (int8 [K,N] or int4 [K,N/2], per-channel scales)  */
/* ------------------------------------------------------------------ */

/* Signed code of element (k,n).  int4: tests/python/relax/test_codegen_cutlass.py:1371-1389
 *   ((A[k, n/2] >> (n%2)*4) & 15) << 28 >> 28    (arithmetic shifts, int32)
 * int8: :1628  A[k,n].                                                      */
static inline int intb_code(const int8_t* A, int64_t k, int64_t n, int64_t N, int nbit) {
  if (nbit == 8) return (int)A[k * N + n];
  int32_t b = (int32_t)A[k * (N / 2) + n / 2];
  int32_t nib = (b >> ((int)(n % 2) * 4)) & 15;
  return (int)((int32_t)((uint32_t)nib << 28) >> 28);
}

void wqo_intb_unpack(const int8_t* A, int8_t* q, int64_t K, int64_t N, int nbit) {
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n) q[k * N + n] = (int8_t)intb_code(A, k, n, N, nbit);
}

/* decode: w[k,n] = fp16(q) * scale   in fp16.
 * group_size <= 0: per-channel, scale = B[n]          (test_codegen_cutlass.py:1371-1389, 1628)
 * group_size  > 0: fine-grained, scale = B[k/group, n] (:2041, group 64)    */
void wqo_intb_dequant(const int8_t* A, const uint16_t* scales, uint16_t* out, int64_t K, int64_t N,
                      int nbit, int64_t group_size) {
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n) {
      uint16_t s = group_size > 0 ? scales[(k / group_size) * N + n] : scales[n];
      out[k * N + n] = h_mul(f2h((float)intb_code(A, k, n, N, nbit)), s);
    }
}

static float act_apply(float v, int activation) {
  switch (activation) {
    case 1: return v > 0.0f ? v : 0.0f;                                  /* relu */
    case 2: return v / (1.0f + expf(-v));                                /* silu */
    case 3: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f)); /* gelu (erf) */
    default: return v;
  }
}

/* What the reference asks the external kernel for
 * (python/tvm/contrib/cutlass/gemm_operation.py:441-458, build.py:701-777):
 *   C[m,n] = act( sum_k A[m,k] * w[k,n] + bias )                     fp32 accumulate, fp16 out
 *   residual form: C = unary( binary( act(...), residual[m,n] ) )
 * bias_stride == 0: bias[n] broadcast over rows; otherwise bias[m*bias_stride + n].
 * activation: 0 identity, 1 relu, 2 silu, 3 gelu.  binary_op: 0 none, 1 plus, 2 multiply.
 * unary_op: 0 identity, 1 relu.  Wdeq is the fp16 [K,N] output of wqo_intb_dequant.
 * The epilogue runs in fp32 and rounds once at the store.                   */
void wqo_nn_matmul_f32acc(const uint16_t* Xa, const uint16_t* Wdeq, const uint16_t* bias,
                          const uint16_t* residual, uint16_t* C, int64_t M, int64_t N, int64_t K,
                          int activation, int binary_op, int unary_op, int64_t bias_stride,
                          int nthreads) {
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float* acc = (float*)calloc((size_t)N, sizeof(float));
    for (int64_t k = 0; k < K; ++k) {
      float a = h2f(Xa[m * K + k]);
      const uint16_t* wr = Wdeq + k * N;
      for (int64_t n = 0; n < N; ++n) acc[n] = acc[n] + a * h2f(wr[n]);
    }
    for (int64_t n = 0; n < N; ++n) {
      float v = acc[n];
      if (bias) v = v + h2f(bias[bias_stride ? m * bias_stride + n : n]);
      v = act_apply(v, activation);
      if (residual && binary_op == 1) v = v + h2f(residual[m * N + n]);
      if (residual && binary_op == 2) v = v * h2f(residual[m * N + n]);
      if (unary_op == 1) v = v > 0.0f ? v : 0.0f;
      C[m * N + n] = f2h(v);
    }
    free(acc);
  }
}

/* Reference CPU path for one Format-B linear (decode then matmul). */
void wqo_intb_linear(const uint16_t* Xa, const int8_t* A, const uint16_t* scales,
                     const uint16_t* bias, const uint16_t* residual, uint16_t* C, int64_t M,
                     int64_t N, int64_t K, int nbit, int64_t group_size, int activation,
                     int binary_op, int unary_op, int64_t bias_stride, int nthreads) {
  uint16_t* Wd = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(N * K));
  wqo_intb_dequant(A, scales, Wd, K, N, nbit, group_size);
  wqo_nn_matmul_f32acc(Xa, Wd, bias, residual, C, M, N, K, activation, binary_op, unary_op,
                       bias_stride, nthreads);
  free(Wd);
}

/* ------------------------------------------------------------------ */
/* Weight preprocessing for the mixed-input GEMM                        */
/* ------------------------------------------------------------------ */
/*
 * cutlass.ft_preprocess_weight (src/runtime/contrib/cutlass/weight_preprocess.cc:38-59)
 * forwards to fastertransformer::preprocess_weights(out, in, num_experts, rows,
 * cols, is_int4, sm) of tlc-pack/cutlass_fpA_intB_gemm, which is not in the
 * reference tree.  Its published algorithm for sm 75..89, restated here in the
 * order the library applies it:
 *   1. permute rows inside tiles of 16 (int8) / 32 (int4) rows so that the
 *      elements one tensor-core lane consumes are adjacent;
 *   2. transpose to column-major (sub-byte aware);
 *   3. interleave 2 (int8) / 4 (int4) columns in tiles of 64 rows;
 *   4. add the bias 128 / 8 (signed -> unsigned) and reorder inside each
 *      32-bit word: bytes [0,2,1,3] / nibbles [0,2,4,6,1,3,5,7].
 * rows = K, cols = N (elements, not bytes).  Requires K % 64 == 0, N % 64 == 0.
 * Returns 0, or -1 for an unsupported sm / shape.
 */
static inline int get_elem(const uint8_t* p, int64_t idx, int nbit) {
  if (nbit == 8) return p[idx];
  return (p[idx >> 1] >> ((idx & 1) * 4)) & 15;
}
static inline void set_elem(uint8_t* p, int64_t idx, int nbit, int v) {
  if (nbit == 8) {
    p[idx] = (uint8_t)v;
  } else {
    int sh = (int)(idx & 1) * 4;
    p[idx >> 1] = (uint8_t)((p[idx >> 1] & ~(15 << sh)) | ((v & 15) << sh));
  }
}

int wqo_ft_preprocess(int8_t* out_, const int8_t* in_, int64_t num_experts, int64_t rows,
                      int64_t cols, int is_int4, int sm) {
  if (sm < 75 || sm >= 90) return -1;
  if (rows % 64 != 0 || cols % 64 != 0) return -1;
  const int nbit = is_int4 ? 4 : 8;
  const int64_t per_expert_bytes = rows * cols * nbit / 8;
  const int64_t nelem = rows * cols;
  uint8_t* t1 = (uint8_t*)malloc((size_t)per_expert_bytes);
  uint8_t* t2 = (uint8_t*)malloc((size_t)per_expert_bytes);
  uint8_t* t3 = (uint8_t*)malloc((size_t)per_expert_bytes);
  for (int64_t e = 0; e < num_experts; ++e) {
    const uint8_t* in = (const uint8_t*)in_ + e * per_expert_bytes;
    uint8_t* out = (uint8_t*)out_ + e * per_expert_bytes;
    /* step 1: row permutation, tile of R rows; E = elements per 32-bit word */
    const int E = 32 / nbit;
    const int R = 8 * (16 / nbit) ; /* 16 for int8, 32 for int4 */
    memset(t1, 0, (size_t)per_expert_bytes);
    for (int64_t r = 0; r < rows; ++r) {
      int64_t base = r - r % R, w = r % R;
      int64_t src = base + 8 * ((w % E) / 2) + (w % 2) + 2 * (w / E);
      for (int64_t c = 0; c < cols; ++c)
        set_elem(t1, r * cols + c, nbit, get_elem(in, src * cols + c, nbit));
    }
    /* step 2: transpose [rows, cols] -> [cols, rows] */
    memset(t2, 0, (size_t)per_expert_bytes);
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; ++c)
        set_elem(t2, c * rows + r, nbit, get_elem(t1, r * cols + c, nbit));
    /* step 3: column interleave, moved as 32-bit words */
    {
      const int64_t wpc = rows / E;           /* words per column */
      const int64_t T = 64 / E;               /* words per 64-row tile */
      const int64_t I = (128 * 8 / nbit) / 64; /* columns interleaved: 2 / 4 */
      const uint32_t* s = (const uint32_t*)t2;
      uint32_t* d = (uint32_t*)t3;
      for (int64_t c = 0; c < cols; ++c)
        for (int64_t v = 0; v < wpc; ++v) {
          int64_t dst = (c / I) * wpc * I + I * (v - v % T) + T * (c % I) + v % T;
          d[dst] = s[c * wpc + v];
        }
    }
    /* step 4: bias + in-word reorder */
    if (nbit == 8) {
      static const int map8[4] = {0, 2, 1, 3};
      for (int64_t w = 0; w < nelem / 4; ++w)
        for (int i = 0; i < 4; ++i)
          out[w * 4 + i] = (uint8_t)(t3[w * 4 + map8[i]] + 128);
    } else {
      static const int map4[8] = {0, 2, 4, 6, 1, 3, 5, 7};
      memset(out, 0, (size_t)per_expert_bytes);
      for (int64_t w = 0; w < nelem / 8; ++w)
        for (int i = 0; i < 8; ++i)
          set_elem(out, w * 8 + i, 4, (get_elem(t3, w * 8 + map4[i], 4) + 8) & 15);
    }
  }
  free(t1);
  free(t2);
  free(t3);
  return 0;
}

/* Inverse of wqo_ft_preprocess, found by inverting each step (tests only). */
int wqo_ft_unprocess(int8_t* out_, const int8_t* in_, int64_t num_experts, int64_t rows,
                     int64_t cols, int is_int4, int sm) {
  if (sm < 75 || sm >= 90) return -1;
  if (rows % 64 != 0 || cols % 64 != 0) return -1;
  const int nbit = is_int4 ? 4 : 8;
  const int64_t per_expert_bytes = rows * cols * nbit / 8;
  const int64_t nelem = rows * cols;
  uint8_t* t1 = (uint8_t*)malloc((size_t)per_expert_bytes);
  uint8_t* t2 = (uint8_t*)malloc((size_t)per_expert_bytes);
  uint8_t* t3 = (uint8_t*)malloc((size_t)per_expert_bytes);
  for (int64_t e = 0; e < num_experts; ++e) {
    const uint8_t* in = (const uint8_t*)in_ + e * per_expert_bytes;
    uint8_t* out = (uint8_t*)out_ + e * per_expert_bytes;
    const int E = 32 / nbit;
    const int R = 8 * (16 / nbit);
    /* undo 4 */
    memset(t3, 0, (size_t)per_expert_bytes);
    if (nbit == 8) {
      static const int map8[4] = {0, 2, 1, 3};
      for (int64_t w = 0; w < nelem / 4; ++w)
        for (int i = 0; i < 4; ++i) t3[w * 4 + map8[i]] = (uint8_t)(in[w * 4 + i] - 128);
    } else {
      static const int map4[8] = {0, 2, 4, 6, 1, 3, 5, 7};
      for (int64_t w = 0; w < nelem / 8; ++w)
        for (int i = 0; i < 8; ++i)
          set_elem(t3, w * 8 + map4[i], 4, (get_elem(in, w * 8 + i, 4) - 8) & 15);
    }
    /* undo 3 */
    {
      const int64_t wpc = rows / E, T = 64 / E, I = (128 * 8 / nbit) / 64;
      const uint32_t* s = (const uint32_t*)t3;
      uint32_t* d = (uint32_t*)t2;
      for (int64_t c = 0; c < cols; ++c)
        for (int64_t v = 0; v < wpc; ++v) {
          int64_t pos = (c / I) * wpc * I + I * (v - v % T) + T * (c % I) + v % T;
          d[c * wpc + v] = s[pos];
        }
    }
    /* undo 2 */
    memset(t1, 0, (size_t)per_expert_bytes);
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; ++c)
        set_elem(t1, r * cols + c, nbit, get_elem(t2, c * rows + r, nbit));
    /* undo 1 */
    memset(out, 0, (size_t)per_expert_bytes);
    for (int64_t r = 0; r < rows; ++r) {
      int64_t base = r - r % R, w = r % R;
      int64_t src = base + 8 * ((w % E) / 2) + (w % 2) + 2 * (w / E);
      for (int64_t c = 0; c < cols; ++c)
        set_elem(out, src * cols + c, nbit, get_elem(t1, r * cols + c, nbit));
    }
  }
  free(t1);
  free(t2);
  free(t3);
  return 0;
}

/* ------------------------------------------------------------------ */
/* Quantizers used by the reference's fixtures (Format B)               */
/* ------------------------------------------------------------------ */
/*
 * tests/python/relax/test_codegen_cutlass.py:1392-1457 (int4) and :1631-1676 (int8):
 *   max_abs[n] = max_k |A[n,k]|                       (fp16)
 *   scale[n]   = max(f32(max_abs[n]), 1e-4) * c       c = 0.125 (int4) / 0.0078125 (int8)
 *   q[k,n]     = clip(round(f32(A[n,k]) / scale[n]), lo, hi)     round = half away from zero
 *   int4: two n per byte, low nibble = even n; scales_out[n] = fp16(scale[n])
 * A is fp16 [N,K]; w_out int8 [K,N] or [K,N/2].
 */
void wqo_intb_encode(const uint16_t* A, int8_t* w_out, uint16_t* scales_out, int64_t N, int64_t K,
                     int nbit) {
  const float c = nbit == 4 ? 0.125f : 0.0078125f;
  const float lo = nbit == 4 ? -8.0f : -128.0f, hi = nbit == 4 ? 7.0f : 127.0f;
  float* scale = (float*)malloc(sizeof(float) * (size_t)N);
  for (int64_t n = 0; n < N; ++n) {
    float mx = -65504.0f;
    for (int64_t k = 0; k < K; ++k) {
      float v = fabsf(h2f(A[n * K + k]));
      if (v > mx) mx = v;
    }
    scale[n] = (mx > 0.0001f ? mx : 0.0001f) * c;
    scales_out[n] = f2h(scale[n]);
  }
  if (nbit == 4) memset(w_out, 0, (size_t)(K * N / 2));
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n) {
      float r = roundf(h2f(A[n * K + k]) / scale[n]);
      if (r < lo) r = lo;
      if (r > hi) r = hi;
      int q = (int)r;
      if (nbit == 8) {
        w_out[k * N + n] = (int8_t)q;
      } else {
        uint8_t* p = (uint8_t*)&w_out[k * (N / 2) + n / 2];
        *p = (uint8_t)(*p | ((q & 15) << ((n % 2) * 4)));
      }
    }
  free(scale);
}

/*
 * Fine-grained (group 64 along K) form of the same quantizer,
 * tests/python/relax/test_codegen_cutlass.py:2044-2109: the maximum, the scale and
 * the division are per (k / 64, n); scales_out is fp16 [K/64, N].  K % 64 == 0.
 */
void wqo_intb_encode_grouped(const uint16_t* A, int8_t* w_out, uint16_t* scales_out, int64_t N,
                             int64_t K, int nbit) {
  const float c = nbit == 4 ? 0.125f : 0.0078125f;
  const float lo = nbit == 4 ? -8.0f : -128.0f, hi = nbit == 4 ? 7.0f : 127.0f;
  if (nbit == 4) memset(w_out, 0, (size_t)(K * N / 2));
  for (int64_t g = 0; g < K / 64; ++g)
    for (int64_t n = 0; n < N; ++n) {
      float mx = -65504.0f;
      for (int64_t k = g * 64; k < g * 64 + 64; ++k) {
        float v = fabsf(h2f(A[n * K + k]));
        if (v > mx) mx = v;
      }
      const float scale = (mx > 0.0001f ? mx : 0.0001f) * c;
      scales_out[g * N + n] = f2h(scale);
      for (int64_t k = g * 64; k < g * 64 + 64; ++k) {
        float r = roundf(h2f(A[n * K + k]) / scale);
        if (r < lo) r = lo;
        if (r > hi) r = hi;
        int q = (int)r;
        if (nbit == 8) {
          w_out[k * N + n] = (int8_t)q;
        } else {
          uint8_t* p = (uint8_t*)&w_out[k * (N / 2) + n / 2];
          *p = (uint8_t)(*p | ((q & 15) << ((n % 2) * 4)));
        }
      }
    }
}

/*
 * q4f16_1 quantizer (Format A), the inverse of the decode in
 * tests/python/dlight/test_gpu_gemv.py:198.  The reference tree holds no encoder for
 * this format, so this is a definition, not a restatement (parity unpinned):
 *   per group of 32 along K:  m = max |a|  (fp16),
 *   scale = fp16( max(f32(m), 1e-4) / 7 ),
 *   code  = clip( round( f32(a) / f32(scale) ) + 7, 0, 14 )     round = half away from zero
 * so that decode gives (code - 7) * scale with |error| <= scale / 2 for every element
 * (the group maximum maps to code 0 or 14).  W uint32 [N, K/8], S fp16 [N, K/32].
 */
void wqo_q4g32_encode(const uint16_t* A, uint32_t* W, uint16_t* S, int64_t N, int64_t K) {
  for (int64_t n = 0; n < N; ++n)
    for (int64_t g = 0; g < K / 32; ++g) {
      const uint16_t* a = A + n * K + g * 32;
      float mx = 0.0f;
      for (int i = 0; i < 32; ++i) {
        float v = fabsf(h2f(a[i]));
        if (v > mx) mx = v;
      }
      const uint16_t sh = f2h((mx > 0.0001f ? mx : 0.0001f) / 7.0f);
      const float scale = h2f(sh);
      S[n * (K / 32) + g] = sh;
      for (int j = 0; j < 4; ++j) {
        uint32_t word = 0;
        for (int i = 0; i < 8; ++i) {
          float r = roundf(h2f(a[8 * j + i]) / scale) + 7.0f;
          if (r < 0.0f) r = 0.0f;
          if (r > 14.0f) r = 14.0f;
          word |= (uint32_t)(int)r << (4 * i);
        }
        W[n * (K / 8) + g * 4 + j] = word;
      }
    }
}

/* ------------------------------------------------------------------ */
/* AutoGPTQ layout: K-major int4 with packed zero points and g_idx     */
/* ------------------------------------------------------------------ */

/* tests/python/dlight/test_gpu_gemv.py:636-652 (the "decode" block):
 *   qweight uint32 [K/8, N], qzeros uint32 [G, N/8], scales fp16 [G, N], g_idx uint32 [K]
 *   g = g_idx[k]
 *   B[k,n] = (fp16((qweight[k/8,n] >> 4*(k%8)) & 15)
 *             - (fp16((qzeros[g, n/8] >> 4*(n%8)) & 15) + fp16(1))) * scales[g,n]     all in fp16
 * out fp16 [K, N].  Returns -1 if a g_idx entry is outside [0, G).             */
int wqo_gptq_dequant(const uint32_t* qweight, const uint32_t* qzeros, const uint16_t* scales,
                     const int32_t* g_idx, uint16_t* out, int64_t K, int64_t N, int64_t G) {
  const uint16_t one = 0x3c00u;
  for (int64_t k = 0; k < K; ++k) {
    const int64_t g = g_idx[k];
    if (g < 0 || g >= G) return -1;
    for (int64_t n = 0; n < N; ++n) {
      const uint32_t code = (qweight[(k / 8) * N + n] >> ((uint32_t)(k % 8) * 4u)) & 15u;
      const uint32_t zero = (qzeros[g * (N / 8) + n / 8] >> ((uint32_t)(n % 8) * 4u)) & 15u;
      const uint16_t zp = h_add(f2h((float)zero), one);
      out[k * N + n] = h_mul(h_sub(f2h((float)code), zp), scales[g * N + n]);
    }
  }
  return 0;
}

/* The matmul and the add that follow the decode, test_gpu_gemv.py:653-665:
 *   acc = fp16(0);  acc = acc + x[k] * B[k,n]   (k ascending; product and sum rounded to fp16)
 *   y = residual + acc                           (fp16 add)
 * f32acc != 0 switches to the accumulate mode the GPU build implements for every format
 * (fp32 products and sums over the same fp16 weights, one rounding to fp16, then the
 * fp16 residual add), the fp32-accumulate convention of test_gpu_reduction.py:411-424.
 * Bdeq fp16 [K, N], X fp16 [M, K], residual fp16 [M, N] or NULL, Y fp16 [M, N].  */
void wqo_kn_matmul(const uint16_t* Bdeq, const uint16_t* X, const uint16_t* residual, uint16_t* Y,
                   int64_t M, int64_t N, int64_t K, int f32acc) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      uint16_t h;
      if (f32acc) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) acc = acc + h2f(X[m * K + k]) * h2f(Bdeq[k * N + n]);
        h = f2h(acc);
      } else {
        h = 0;
        for (int64_t k = 0; k < K; ++k) h = h_add(h, h_mul(X[m * K + k], Bdeq[k * N + n]));
      }
      Y[m * N + n] = residual ? h_add(residual[m * N + n], h) : h;
    }
}
