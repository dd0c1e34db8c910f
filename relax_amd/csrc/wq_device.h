// Device-side building blocks shared by every kernel of the quantized linear path.
// gfx950 only: 64-wide wavefronts, packed fp16 VALU, v_dot2_f32_f16, MFMA.
#ifndef RELAX_AMD_CSRC_WQ_DEVICE_H_
#define RELAX_AMD_CSRC_WQ_DEVICE_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace wq {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ half_t as_half(uint16_t u) { return __builtin_bit_cast(half_t, u); }
__device__ __forceinline__ uint16_t as_u16(half_t h) { return __builtin_bit_cast(uint16_t, h); }

// (a & mask) | bits in one VALU instruction.  The compiler prefers two VOP2
// instructions with literal operands; v_and_or_b32 (VOP3, no literals on gfx9)
// needs the constants in registers: `mask` in an SGPR, `bits` in a VGPR.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(bits));
  return r;
}

// ---------------------------------------------------------------------------
// Format A: one uint32 holds 8 codes, code i in bits 4i..4i+3.
// (w >> 4i) & 0x000F000F isolates code i in the low half-word and code i+4 in the
// high half-word.  OR-ing 0x6400 into each half-word makes the fp16 number
// 1024 + code (exact), and subtracting 1031 leaves code - 7 exactly.  So
// pair i of the result is (code_i - 7, code_{i+4} - 7): the PAIRING IS (i, i+4),
// not (2i, 2i+1).  Every caller arranges its activations to match.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void q4_word_minus7(uint32_t w, half2_t out[4]) {
  const half2_t off = {(half_t)1031.0f, (half_t)1031.0f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t t = and_or(w >> (4 * i), 0x000F000Fu, 0x64006400u);
    out[i] = as_half2(t) - off;
  }
}

// The reference's dequantized weight, bit for bit: (fp16(code) - 7) * s with a single
// fp16 rounding in the multiply.  s2 holds the group's scale in both halves.
__device__ __forceinline__ void q4_word_dequant(uint32_t w, half2_t s2, half2_t out[4]) {
  half2_t d[4];
  q4_word_minus7(w, d);
#pragma unroll
  for (int i = 0; i < 4; ++i) out[i] = d[i] * s2;
}

// Same value as q4_word_dequant but in NATURAL order: out[j] = (w_{2j}, w_{2j+1}).
// One instruction more per pair (shift, shift-or to move the odd code into the high
// half-word, and-or); used where rearranging the other operand would cost more.
__device__ __forceinline__ void q4_word_dequant_natural(uint32_t w, half2_t s2, half2_t out[4]) {
  const half2_t off = {(half_t)1031.0f, (half_t)1031.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t t = (w >> (8 * j)) & 0xFFu;  // codes 2j, 2j+1 in bits 0..7 (v_bfe_u32)
    const uint32_t u = (t << 12) | t;           // code 2j+1 also in bits 16..19
    out[j] = (as_half2(and_or(u, 0x000F000Fu, 0x64006400u)) - off) * s2;
  }
}

// One pair of the above, in two steps: the fp16 bit pattern (1024 + code_{2j}, 1024 + code_{2j+1}) ...
__device__ __forceinline__ uint32_t q4_pair_bits_natural(uint32_t w, int j) {
  const uint32_t t = (w >> (8 * j)) & 0xFFu;
  const uint32_t u = (t << 12) | t;
  return and_or(u, 0x000F000Fu, 0x64006400u);
}
// ... and (w_{2j}, w_{2j+1}) from it.
__device__ __forceinline__ half2_t q4_pair_dequant_natural(uint32_t w, int j, half2_t s2) {
  const half2_t off = {(half_t)1031.0f, (half_t)1031.0f};
  return (as_half2(q4_pair_bits_natural(w, j)) - off) * s2;
}

// fp32 += a.x*b.x + a.y*b.y with exact fp16 products (v_dot2_f32_f16).
__device__ __forceinline__ float dot2(half2_t a, half2_t b, float c) {
  return __builtin_amdgcn_fdot2(a, b, c, false);
}

// Rearranges 8 consecutive halves (4 dwords, natural order) into the (i, i+4)
// pairing q4_word_minus7 produces: out[i] = (h[i], h[i+4]).
__device__ __forceinline__ void pair_i_i4(const uint32_t in[4], uint32_t out[4]) {
  // v_perm_b32(hi_src, lo_src, sel): byte k of the result = byte sel[k] of {hi_src:lo_src}
  // (bytes 0-3 from lo_src, 4-7 from hi_src).
  out[0] = __builtin_amdgcn_perm(in[2], in[0], 0x05040100u);  // (h0, h4)
  out[1] = __builtin_amdgcn_perm(in[2], in[0], 0x07060302u);  // (h1, h5)
  out[2] = __builtin_amdgcn_perm(in[3], in[1], 0x05040100u);  // (h2, h6)
  out[3] = __builtin_amdgcn_perm(in[3], in[1], 0x07060302u);  // (h3, h7)
}

// v shifted / permuted across lanes by a DPP control word; lanes without a source get 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_shift(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true));
}
// quad_perm: 0xb1 = [1,0,3,2] (xor 1), 0x4e = [2,3,0,1] (xor 2)
template <int CTRL>
__device__ __forceinline__ float dpp_quad(float v) {
  return dpp_shift<CTRL, 0xf>(v);
}

// Sum over the wavefront; the total is valid in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v += dpp_shift<0x111, 0xf>(v);  // row_shr:1
  v += dpp_shift<0x112, 0xf>(v);  // row_shr:2
  v += dpp_shift<0x114, 0xf>(v);  // row_shr:4
  v += dpp_shift<0x118, 0xf>(v);  // row_shr:8   -> lane 15 of each row holds the row sum
  v += dpp_shift<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_shift<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Sum over the 64 lanes of a wavefront; every lane receives the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---------------------------------------------------------------------------
// Format B helpers.  After preprocessing, every stored code is unsigned
// (int8: q + 128, int4: q + 8).
// ---------------------------------------------------------------------------

// Two bytes of `w` (selected by the v_perm selector `sel`, whose bytes 1 and 3
// must pick the constant 0x64) -> (q_a, q_b) as exact fp16 integers.
// sel examples: 0x04020400 -> bytes (0, 2);  0x04030401 -> bytes (1, 3).
__device__ __forceinline__ half2_t u8x2_to_half2(uint32_t w, uint32_t sel) {
  uint32_t t = __builtin_amdgcn_perm(0x64646464u, w, sel);  // (1024 + u_a, 1024 + u_b)
  const half2_t off = {(half_t)1152.0f, (half_t)1152.0f};    // 1024 + 128
  return as_half2(t) - off;
}

// Eight unsigned nibbles of `w` -> pairs (nibble i, nibble i+4) minus 8, exact.
__device__ __forceinline__ void u4_word_minus8(uint32_t w, half2_t out[4]) {
  const half2_t off = {(half_t)1032.0f, (half_t)1032.0f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t t = ((w >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
    out[i] = as_half2(t) - off;
  }
}

__device__ __forceinline__ float apply_activation(float v, int act) {
  switch (act) {
    case 1: return v > 0.0f ? v : 0.0f;
    case 2: return v / (1.0f + __expf(-v));
    case 3: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    default: return v;
  }
}

}  // namespace wq
#endif  // RELAX_AMD_CSRC_WQ_DEVICE_H_
