// One 16-byte piece of a packed W4 row (32 K values of one scale group) against the matching 32
// activations of up to M sequences, the activations held in registers in the nibble decoder's pair
// order: the inner step of the fused decode launches (decode_fused.hip, the projecting attention
// merge in q8_attention.hip).
#pragma once

#include "w4_common.h"

namespace llmopt {

// 32 activations of M rows in pair order, and what the biased decode adds to a dot product with them.
template <int M>
struct Held {
  uint4 x[M][4];
  float correction[M];
};

// The lane's 32 values [32 piece, 32 piece + 32) of every row, from halves in LDS (row stride `stride` halves).
template <int M>
__device__ __forceinline__ void hold_rows(Held<M> &held, const uint16_t *rows, uint32_t stride, uint32_t piece,
                                          bool present) {
  // the correction as dot products with the constant pairs (1032, 1032) and (72, 72): exact products,
  // float32 sums, sixteen instructions instead of a conversion and an addition per value
  const h2_t bias_a = {(_Float16)1032.0f, (_Float16)1032.0f}, bias_b = {(_Float16)72.0f, (_Float16)72.0f};
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float sum_a = 0.0f, sum_b = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint4 natural = *reinterpret_cast<const uint4 *>(rows + m * stride + piece * 32 + j * 8);
      const uint4 v = present ? pair_order(natural) : make_uint4(0, 0, 0, 0);
      held.x[m][j] = v;
      sum_a = __builtin_amdgcn_fdot2(as_h2(v.x), bias_a, sum_a, false);
      sum_b = __builtin_amdgcn_fdot2(as_h2(v.y), bias_b, sum_b, false);
      sum_a = __builtin_amdgcn_fdot2(as_h2(v.z), bias_a, sum_a, false);
      sum_b = __builtin_amdgcn_fdot2(as_h2(v.w), bias_b, sum_b, false);
    }
    held.correction[m] = sum_a + sum_b;
  }
}

// One 16-byte piece of a weight row against the held activations: q . x * scale per row, this lane's share.
template <int M>
__device__ __forceinline__ void piece_dot(const u32x4_t weights, float scale, const Held<M> &held, float (&out)[M]) {
  // one accumulator per dword: four short chains instead of one of sixteen
  float part[M][4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const W4Pairs q = w4_decode_biased(weights[j]);
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float a = __builtin_amdgcn_fdot2(q.p04, as_h2(held.x[m][j].x), 0.0f, false);
      a = __builtin_amdgcn_fdot2(q.p15, as_h2(held.x[m][j].y), a, false);
      a = __builtin_amdgcn_fdot2(q.p26, as_h2(held.x[m][j].z), a, false);
      part[m][j] = __builtin_amdgcn_fdot2(q.p37, as_h2(held.x[m][j].w), a, false);
    }
  }
#pragma unroll
  for (int m = 0; m < M; ++m)
    out[m] = (((part[m][0] + part[m][1]) + (part[m][2] + part[m][3])) - held.correction[m]) * scale;
}

}  // namespace llmopt
