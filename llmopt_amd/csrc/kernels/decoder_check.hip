// Bit-exactness checks of the int4 / int8 decoders the product kernels use.
//
// Every W4A16 kernel turns nibbles into fp16 through w4_decode_pairs, w4_decode_biased or (prefill
// GEMM) w4_scaled_natural, and the Q8 attention kernels turn bytes into fp16 through
// int8x4_to_h2 / int8x4_to_h2_biased (w4_common.h).  These kernels run exactly those device
// functions over a buffer and write what they produced as float32, so a test can compare every
// byte value with the CPU restatement (python/llmopt_backend/quantization.py:91-121 for int4,
// lib/metal_cache_source.ml:382-401 for int8).  No reference kernel corresponds to them.
#include "kernels.h"
#include "w4_common.h"

namespace llmopt {
namespace {

// one thread per weight dword (8 nibbles = K offsets 0..7 of its row)
template <int DECODER>
__global__ __launch_bounds__(256) void w4_dequant_f32_kernel(const uint32_t *weight, const uint16_t *scale, float *out,
                                                             uint32_t n, uint32_t k) {
  const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t words_per_row = k >> 3;
  if (index >= (size_t)n * words_per_row) return;
  const size_t row = index / words_per_row;
  const size_t word_in_row = index - row * words_per_row;
  const uint32_t word = weight[index];
  const uint16_t scale_bits = scale[row * (k >> 6) + (word_in_row >> 3)];
  const float s = half_bits_to_float(scale_bits);
  float q[8];
  if (DECODER == 2) {
    // the GEMM's staged operand: half(q * s), already in natural order
    const uint4 staged = w4_scaled_natural(word, __builtin_bit_cast(_Float16, scale_bits));
    const uint32_t parts[4] = {staged.x, staged.y, staged.z, staged.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const h2_t pair = as_h2(parts[i]);
      out[row * k + word_in_row * 8 + 2 * i] = (float)pair[0];
      out[row * k + word_in_row * 8 + 2 * i + 1] = (float)pair[1];
    }
    return;
  }
  const W4Pairs pairs = DECODER == 0 ? w4_decode_pairs(word) : w4_decode_biased(word);
  const float bias_even = DECODER == 0 ? 0.0f : 1032.0f, bias_odd = DECODER == 0 ? 0.0f : 72.0f;
  q[0] = (float)pairs.p04[0] - bias_even;
  q[4] = (float)pairs.p04[1] - bias_even;
  q[1] = (float)pairs.p15[0] - bias_odd;
  q[5] = (float)pairs.p15[1] - bias_odd;
  q[2] = (float)pairs.p26[0] - bias_even;
  q[6] = (float)pairs.p26[1] - bias_even;
  q[3] = (float)pairs.p37[0] - bias_odd;
  q[7] = (float)pairs.p37[1] - bias_odd;
#pragma unroll
  for (int i = 0; i < 8; ++i) out[row * k + word_in_row * 8 + i] = q[i] * s;
}

// one thread per dword of int8 values
template <bool BIASED>
__global__ __launch_bounds__(256) void q8_decode_f32_kernel(const uint32_t *bytes, float *out, uint32_t words) {
  const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= words) return;
  h2_t lo, hi;
  if (BIASED)
    int8x4_to_h2_biased(bytes[index] ^ 0x80808080u, lo, hi);
  else
    int8x4_to_h2(bytes[index] ^ 0x80808080u, lo, hi);
  const float bias = BIASED ? 1152.0f : 0.0f;
  out[4 * index] = (float)lo[0] - bias;
  out[4 * index + 1] = (float)lo[1] - bias;
  out[4 * index + 2] = (float)hi[0] - bias;
  out[4 * index + 3] = (float)hi[1] - bias;
}

}  // namespace

hipError_t launch_w4_dequant_f32(const W4Matrix &w, float *out, uint32_t n, uint32_t k, uint32_t decoder,
                                 hipStream_t stream) {
  const size_t total = (size_t)n * (k >> 3);
  const dim3 grid((uint32_t)((total + 255) / 256)), block(256);
  const uint32_t *words = reinterpret_cast<const uint32_t *>(w.weight);
  if (decoder == 0)
    hipLaunchKernelGGL(w4_dequant_f32_kernel<0>, grid, block, 0, stream, words, w.scale, out, n, k);
  else if (decoder == 1)
    hipLaunchKernelGGL(w4_dequant_f32_kernel<1>, grid, block, 0, stream, words, w.scale, out, n, k);
  else if (decoder == 2)
    hipLaunchKernelGGL(w4_dequant_f32_kernel<2>, grid, block, 0, stream, words, w.scale, out, n, k);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_q8_decode_f32(const uint8_t *bytes, float *out, uint32_t count, uint32_t decoder,
                                hipStream_t stream) {
  const uint32_t words = count >> 2;
  const dim3 grid((words + 255) / 256), block(256);
  const uint32_t *source = reinterpret_cast<const uint32_t *>(bytes);
  if (decoder == 0)
    hipLaunchKernelGGL(q8_decode_f32_kernel<false>, grid, block, 0, stream, source, out, words);
  else if (decoder == 1)
    hipLaunchKernelGGL(q8_decode_f32_kernel<true>, grid, block, 0, stream, source, out, words);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace llmopt
