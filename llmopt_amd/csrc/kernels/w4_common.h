// Device helpers shared by the W4A16 kernels (gfx950, wave64).
//
// Packed format (python/llmopt_backend/quantization.py:63-121, lib/cpu.ml:131-139):
// byte b of a weight row holds K = 2b in its low nibble and K = 2b + 1 in its
// high nibble, both two's-complement int4; one fp16 scale per 64 K values.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llmopt {

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16x_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ h2_t as_h2(uint32_t bits) {
  return __builtin_bit_cast(h2_t, bits);
}

__device__ __forceinline__ uint32_t as_u32(h2_t value) {
  return __builtin_bit_cast(uint32_t, value);
}

__device__ __forceinline__ float half_bits_to_float(uint16_t bits) {
  return (float)__builtin_bit_cast(_Float16, bits);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float value) {
  return __builtin_bit_cast(uint16_t, (_Float16)value);  // round to nearest even
}

// int4 -> fp16 decode of one dword (8 nibbles = K offsets 0..7), one bit operation per pair.
//
// XOR with 8 turns a two's-complement nibble into offset binary (q + 8).  A 4-bit field in the
// mantissa of 1024.0 (0x6400, ulp 1) or of 64.0 (0x5400, ulp 1/16, field at bits 4..7) reads as
// 1024 + (q + 8) or 64 + (q + 8) exactly.  Both steps are one XOR after the mask:
// (w & mask) ^ (magic | (0x88888888 & mask)), the magic bits lying outside the mask.  The four
// results hold the pairs (k0,k4) (k1,k5) (k2,k6) (k3,k7): the activation is arranged to match.
struct W4Pairs {
  h2_t p04, p15, p26, p37;
};

// The pairs hold q + 1032 (p04, p26) and q + 72 (p15, p37).  A dot product with these is
// corrected afterwards by 1032 * sum(x at K offsets 0,4,2,6) + 72 * sum(x at K offsets 1,5,3,7),
// which does not depend on the weight row.
__device__ __forceinline__ W4Pairs w4_decode_biased(uint32_t word) {
  const uint32_t hi = word >> 8;
  W4Pairs out;
  out.p04 = as_h2((word & 0x000F000Fu) ^ 0x64086408u);
  out.p15 = as_h2((word & 0x00F000F0u) ^ 0x54805480u);
  out.p26 = as_h2((hi & 0x000F000Fu) ^ 0x64086408u);
  out.p37 = as_h2((hi & 0x00F000F0u) ^ 0x54805480u);
  return out;
}

// Exact q: the biased decode and one packed subtract per pair.
__device__ __forceinline__ W4Pairs w4_decode_pairs(uint32_t word) {
  const h2_t bias_lo = {(_Float16)1032.0f, (_Float16)1032.0f};
  const h2_t bias_hi = {(_Float16)72.0f, (_Float16)72.0f};
  W4Pairs out = w4_decode_biased(word);
  out.p04 -= bias_lo;
  out.p15 -= bias_hi;
  out.p26 -= bias_lo;
  out.p37 -= bias_hi;
  return out;
}

// The prefill GEMM's B operand of one weight dword: q * s rounded to fp16 (one rounding per
// weight, at most 2^-11 relative), the 8 values in natural K order.
__device__ __forceinline__ uint4 w4_scaled_natural(uint32_t word, _Float16 scale) {
  const h2_t scale2 = {scale, scale};
  const W4Pairs q = w4_decode_pairs(word);
  const uint32_t p04 = as_u32(q.p04 * scale2), p15 = as_u32(q.p15 * scale2);
  const uint32_t p26 = as_u32(q.p26 * scale2), p37 = as_u32(q.p37 * scale2);
  uint4 packed;
  packed.x = __builtin_amdgcn_perm(p15, p04, 0x05040100u);  // k0 k1
  packed.y = __builtin_amdgcn_perm(p37, p26, 0x05040100u);  // k2 k3
  packed.z = __builtin_amdgcn_perm(p15, p04, 0x07060302u);  // k4 k5
  packed.w = __builtin_amdgcn_perm(p37, p26, 0x07060302u);  // k6 k7
  return packed;
}

// 4 int8 (already XOR 0x80 -> q + 128) to two h2 of exact integers (b0,b1),(b2,b3).
__device__ __forceinline__ void int8x4_to_h2(uint32_t biased, h2_t &lo, h2_t &hi) {
  const h2_t offset = {(_Float16)1152.0f, (_Float16)1152.0f};  // 1024 + 128
  lo = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04010400u)) - offset;
  hi = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04030402u)) - offset;
}

// Same without the subtraction: exact integers q + 1152.  Used for K, where the
// bias becomes a per-head constant 1152 * sum_d(Q[d]) subtracted from the score.
__device__ __forceinline__ void int8x4_to_h2_biased(uint32_t biased, h2_t &lo, h2_t &hi) {
  lo = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04010400u));
  hi = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04030402u));
}

// Rearranges 8 consecutive fp16 activations (x0..x7) into the pair order of
// w4_decode_pairs: {(x0,x4), (x1,x5), (x2,x6), (x3,x7)}.
__device__ __forceinline__ uint4 pair_order(uint4 x) {
  uint4 out;
  out.x = __builtin_amdgcn_perm(x.z, x.x, 0x05040100u);
  out.y = __builtin_amdgcn_perm(x.z, x.x, 0x07060302u);
  out.z = __builtin_amdgcn_perm(x.w, x.y, 0x05040100u);
  out.w = __builtin_amdgcn_perm(x.w, x.y, 0x07060302u);
  return out;
}

// Sum over the 64 lanes of a wave with DPP row operations; every lane of each
// 16-lane row ends with the row sum, then the four row sums are combined.
__device__ __forceinline__ float wave_sum(float value) {
  value += __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), 0xB1, 0xF, 0xF, false));
  value += __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), 0x4E, 0xF, 0xF, false));
  value += __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), 0x141, 0xF, 0xF, false));
  value += __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), 0x140, 0xF, 0xF, false));
  const int bits = __builtin_bit_cast(int, value);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
  return (r0 + r1) + (r2 + r3);
}

// Rotate-half position encoding of one element (lib/metal_normalization_source.ml:765-802):
// half(half(x[col] * cos[col]) + half(+-x[col -+ half_dimension] * sin[col])), every product and
// the sum rounded to half separately.
// The same on values already in registers: `partner` is the element half_dimension away, negated
// for the columns of the first half.
__device__ __forceinline__ _Float16 rotate_half_value(_Float16 value, _Float16 partner, _Float16 cosine,
                                                      _Float16 sine, bool first_half) {
#pragma clang fp contract(off)
  const _Float16 rotated = first_half ? -partner : partner;
  const _Float16 direct = value * cosine;
  const _Float16 turned = rotated * sine;
  return direct + turned;
}

__device__ __forceinline__ _Float16 rotate_half_element(const _Float16 *input, const _Float16 *cosine,
                                                        const _Float16 *sine, uint32_t col,
                                                        uint32_t half_dimension) {
  const uint32_t rotated_col = col < half_dimension ? col + half_dimension : col - half_dimension;
  return rotate_half_value(input[col], input[rotated_col], cosine[col], sine[col], col < half_dimension);
}

__device__ __forceinline__ float wave_max(float value) {
  value = fmaxf(value, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                           0, __builtin_bit_cast(int, value), 0xB1, 0xF, 0xF, false)));
  value = fmaxf(value, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                           0, __builtin_bit_cast(int, value), 0x4E, 0xF, 0xF, false)));
  value = fmaxf(value, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                           0, __builtin_bit_cast(int, value), 0x141, 0xF, 0xF, false)));
  value = fmaxf(value, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                           0, __builtin_bit_cast(int, value), 0x140, 0xF, 0xF, false)));
  const int bits = __builtin_bit_cast(int, value);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Q8 cache quantiser of one 64-wide group, one element per lane (lib/metal_cache_source.ml:62-80):
// the stored scale half(max|x| / 127) (1.0 for an all-zero group) and this lane's int8 value
// clamp(rint(x / float(scale)), -127, 127).
__device__ __forceinline__ int8_t q8_quantize(float x, uint16_t *stored_scale) {
  const float maximum = wave_max(fabsf(x));
  const uint16_t stored = float_to_half_bits(maximum == 0.0f ? 1.0f : maximum / 127.0f);
  const float scale = half_bits_to_float(stored);
  const float rounded = rintf(x / scale);
  *stored_scale = stored;
  return (int8_t)(int)fminf(fmaxf(rounded, -127.0f), 127.0f);
}

}  // namespace llmopt
