// Small decode-step kernels around the W4A16 linears and the Q8 attention:
// RMSNorm, rotate-half RoPE for Q and K, fp16 embedding gather, broadcasting
// fp16 add, byte copy and the two-step argmax of the LM head.  All of them move
// a few kilobytes per launch at decode sizes and are launch-latency bound; they
// are written for clarity, one wave per row where a row reduction is needed.
#include <algorithm>

#include "kernels.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int kRowWaves = 4;  // rows (waves) per workgroup of the row kernels

template <typename In>
__device__ __forceinline__ float load_as_float(const In *p, size_t i);
template <>
__device__ __forceinline__ float load_as_float<uint16_t>(const uint16_t *p, size_t i) {
  return half_bits_to_float(p[i]);
}
template <>
__device__ __forceinline__ float load_as_float<float>(const float *p, size_t i) {
  return p[i];
}

// lib/metal_normalization_source.ml:70-91 and lib/metal_w4a16_source.ml:496-526
template <typename In, bool WEIGHT_FIRST>
__global__ __launch_bounds__(kRowWaves * 64) void rms_norm_kernel(const In *input, const uint16_t *weight,
                                                                  uint16_t *output, uint32_t rows,
                                                                  uint32_t width, float epsilon) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * kRowWaves + (threadIdx.x >> 6);
  if (row >= rows) return;  // whole wave
  const size_t base = (size_t)row * width;
  float square_sum = 0.0f;
  for (uint32_t col = lane; col < width; col += 64) {
    const float value = load_as_float(input, base + col);
    square_sum += value * value;
  }
  square_sum = wave_sum(square_sum);
  const float inverse = rsqrtf(square_sum / (float)width + epsilon);
  for (uint32_t col = lane; col < width; col += 64) {
    const float value = load_as_float(input, base + col);
    const float w = half_bits_to_float(weight[col]);
    output[base + col] = float_to_half_bits(WEIGHT_FIRST ? value * w * inverse : value * inverse * w);
  }
}

// The LM head's normalisation (lib/metal_w4a16_source.ml:1038-1046 keeps
// x * w * inverse in float32 and multiplies it with the dequantised weights).
// The GEMV kernels take fp16 activations, so the float32 value v goes out as
// two fp16 rows, hi = half(v) and lo = half(v - hi): W.hi + W.lo, accumulated
// in float32, differs from W.v by 2^-22 relative instead of the 2^-11 of a
// single fp16 row.  Output rows 2r (hi) and 2r + 1 (lo).
template <typename In>
__global__ __launch_bounds__(kRowWaves * 64) void rms_norm_split_kernel(const In *input, const uint16_t *weight,
                                                                        uint16_t *output, uint32_t rows,
                                                                        uint32_t width, float epsilon) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * kRowWaves + (threadIdx.x >> 6);
  if (row >= rows) return;  // whole wave
  const size_t base = (size_t)row * width;
  float square_sum = 0.0f;
  for (uint32_t col = lane; col < width; col += 64) {
    const float value = load_as_float(input, base + col);
    square_sum += value * value;
  }
  square_sum = wave_sum(square_sum);
  const float inverse = rsqrtf(square_sum / (float)width + epsilon);
  uint16_t *high = output + (size_t)(2 * row) * width;
  uint16_t *low = high + width;
  for (uint32_t col = lane; col < width; col += 64) {
    const float value = load_as_float(input, base + col) * half_bits_to_float(weight[col]) * inverse;
    const uint16_t high_bits = float_to_half_bits(value);
    high[col] = high_bits;
    low[col] = float_to_half_bits(value - half_bits_to_float(high_bits));
  }
}

// The same for f16 rows of up to 64 * 8 * kRmsVectors values, width a multiple
// of 8: the row and the weights are requested once, 16 bytes per lane, all
// loads in flight together, and stay in registers between the two passes (the
// loop above walks the row one 2-byte load latency at a time, twice).
constexpr int kRmsVectors = 4;

template <bool WEIGHT_FIRST>
__global__ __launch_bounds__(kRowWaves * 64) void rms_norm_f16_rows_kernel(const uint16_t *input,
                                                                           const uint16_t *weight,
                                                                           uint16_t *output, uint32_t rows,
                                                                           uint32_t width, float epsilon) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * kRowWaves + (threadIdx.x >> 6);
  if (row >= rows) return;  // whole wave
  const uint32_t vectors = width / 8;
  const uint4 *in = reinterpret_cast<const uint4 *>(input + (size_t)row * width);
  const uint4 *w = reinterpret_cast<const uint4 *>(weight);
  uint4 x_raw[kRmsVectors], w_raw[kRmsVectors];
#pragma unroll
  for (int v = 0; v < kRmsVectors; ++v) {
    const uint32_t index = lane + 64 * v;
    x_raw[v] = index < vectors ? in[index] : make_uint4(0, 0, 0, 0);
    w_raw[v] = index < vectors ? w[index] : make_uint4(0, 0, 0, 0);
  }
  float square_sum = 0.0f;
#pragma unroll
  for (int v = 0; v < kRmsVectors; ++v) {
    const h8_t x = __builtin_bit_cast(h8_t, x_raw[v]);
#pragma unroll
    for (int e = 0; e < 8; ++e) square_sum += (float)x[e] * (float)x[e];
  }
  square_sum = wave_sum(square_sum);
  const float inverse = rsqrtf(square_sum / (float)width + epsilon);
  uint4 *out = reinterpret_cast<uint4 *>(output + (size_t)row * width);
#pragma unroll
  for (int v = 0; v < kRmsVectors; ++v) {
    const uint32_t index = lane + 64 * v;
    if (index >= vectors) continue;
    const h8_t x = __builtin_bit_cast(h8_t, x_raw[v]);
    const h8_t g = __builtin_bit_cast(h8_t, w_raw[v]);
    h8_t y;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float value = (float)x[e], gain = (float)g[e];
      y[e] = (_Float16)(WEIGHT_FIRST ? value * gain * inverse : value * inverse * gain);
    }
    out[index] = __builtin_bit_cast(uint4, y);
  }
}

// lib/metal_normalization_source.ml:765-802
__global__ __launch_bounds__(kRowWaves * 64) void rotary_qk_kernel(RotaryQkArgs a) {
#pragma clang fp contract(off)  // every product and the sum round to half separately
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * kRowWaves + (threadIdx.x >> 6);
  const uint32_t total_rows = a.batches * (a.q_heads + a.k_heads) * a.tokens;
  if (row >= total_rows) return;
  const uint32_t q_rows = a.batches * a.q_heads * a.tokens;
  const bool is_q = row < q_rows;
  const uint32_t local_row = is_q ? row : row - q_rows;
  const uint32_t heads = is_q ? a.q_heads : a.k_heads;
  const uint32_t batch = local_row / (heads * a.tokens);
  const uint32_t head_token = local_row % (heads * a.tokens);
  const uint32_t head = head_token / a.tokens;
  const uint32_t token = head_token % a.tokens;
  const size_t input_base = ((size_t)(batch * a.tokens + token) * heads + head) * a.width;
  const _Float16 *input = reinterpret_cast<const _Float16 *>(is_q ? a.q_input : a.k_input);
  _Float16 *output = reinterpret_cast<_Float16 *>(is_q ? a.q_output : a.k_output);
  const _Float16 *cosine = reinterpret_cast<const _Float16 *>(a.cosine);
  const _Float16 *sine = reinterpret_cast<const _Float16 *>(a.sine);
  const uint32_t trig_batch = a.trig_batches == 1 ? 0 : batch;
  const size_t trig_base = (size_t)(trig_batch * a.tokens + token) * a.width;
  const size_t output_base = (size_t)local_row * a.width;
  for (uint32_t col = lane; col < a.width; col += 64)
    output[output_base + col] =
        rotate_half_element(input + input_base, cosine + trig_base, sine + trig_base, col, a.half_dimension);
}

// lib/metal_tensor_source.ml:306-320
__global__ void embedding_kernel(EmbeddingArgs a) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t count = (size_t)a.tokens * a.width;
  if (gid >= count) return;
  const uint32_t token = (uint32_t)(gid / a.width);
  const uint32_t dimension = (uint32_t)(gid % a.width);
  const int64_t index = a.indices[token];
  a.output[gid] =
      (index >= 0 && index < (int64_t)a.vocabulary) ? a.weight[(size_t)index * a.width + dimension] : (uint16_t)0;
}

// llmopt_pointwise_offset, lib/metal_tensor_source.ml:1014-1028
__device__ __forceinline__ uint32_t pointwise_offset(uint32_t gid, const PointwiseArgs &a, bool is_left) {
  uint32_t remaining = gid, offset = 0, stride = 1;
  for (int axis = (int)a.rank - 1; axis >= 0; --axis) {
    const uint32_t output_dimension = a.output_shape[axis];
    const uint32_t coordinate = remaining % output_dimension;
    remaining /= output_dimension;
    const uint32_t input_dimension = is_left ? a.left_shape[axis] : a.right_shape[axis];
    offset += (input_dimension == 1 ? 0 : coordinate) * stride;
    stride *= input_dimension;
  }
  return offset;
}

__global__ void add_f16_kernel(PointwiseArgs a) {
  const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= a.count) return;
  const _Float16 left = a.left_scalar
                            ? (_Float16)a.left_f32
                            : reinterpret_cast<const _Float16 *>(a.left)[pointwise_offset(gid, a, true)];
  const _Float16 right = a.right_scalar
                             ? (_Float16)a.right_f32
                             : reinterpret_cast<const _Float16 *>(a.right)[pointwise_offset(gid, a, false)];
  reinterpret_cast<_Float16 *>(a.output)[gid] = left + right;
}

// both operands have the output's shape: 8 halves per thread
__global__ void add_f16_same_shape_kernel(const uint4 *left, const uint4 *right, uint4 *output,
                                          uint32_t vectors) {
  const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= vectors) return;
  const uint4 l = left[gid], r = right[gid];
  uint4 out;
  out.x = as_u32(as_h2(l.x) + as_h2(r.x));
  out.y = as_u32(as_h2(l.y) + as_h2(r.y));
  out.z = as_u32(as_h2(l.z) + as_h2(r.z));
  out.w = as_u32(as_h2(l.w) + as_h2(r.w));
  output[gid] = out;
}

__global__ void copy_vectors_kernel(const u32x4_t *source, u32x4_t *destination, size_t vectors) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vectors; i += stride)
    destination[i] = __builtin_nontemporal_load(source + i);
}

__global__ void copy_bytes_kernel(const uint8_t *source, uint8_t *destination, size_t bytes) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < bytes; i += stride)
    destination[i] = source[i];
}

struct Candidate {
  float value;
  uint32_t index;
};

__device__ __forceinline__ bool better(float value, uint32_t index, float best_value, uint32_t best_index) {
  return value > best_value || (value == best_value && index < best_index);
}

// 256 (value, index) candidates per row, the record the reference's stage 1
// hands to its reduce kernel (lib/metal_w4a16_source.ml:1256-1283; there one
// candidate per threadgroup of columns, here candidate t is the best of columns
// t, t + 256, ... - the reduce step only needs every column covered once and
// ties resolved to the lowest index).  Four slices of 256 threads scan a quarter
// of those columns each with several independent loads in flight, then meet in
// LDS: a single thread per candidate would walk its 192 columns of a 49152-wide
// vocabulary one load latency at a time.
constexpr int kArgmaxSlices = 4;
constexpr int kArgmaxUnroll = 4;

// `pairs`: logits holds two rows per output row (the products with the hi and
// the lo half of the activation, see rms_norm_split_kernel) whose sum is the
// logit; `half_logits`, when not null, receives half(logit) [rows, n].
__global__ __launch_bounds__(256 * kArgmaxSlices) void argmax_candidates_kernel(const float *logits,
                                                                                Candidate *candidates,
                                                                                uint32_t n, bool pairs,
                                                                                uint16_t *half_logits) {
  __shared__ float slice_values[kArgmaxSlices][256];
  __shared__ uint32_t slice_indices[kArgmaxSlices][256];
  const uint32_t row = blockIdx.x;
  const uint32_t t = threadIdx.x & 255;
  const uint32_t slice = threadIdx.x >> 8;
  const float *row_logits = logits + (size_t)row * n * (pairs ? 2 : 1);
  const float *row_low = row_logits + n;  // read only with `pairs`
  uint16_t *row_half = half_logits != nullptr ? half_logits + (size_t)row * n : nullptr;
  float best_value = -3.402823466e+38f;
  uint32_t best_index = 0;
  bool found = false;
  const uint32_t step = 256 * kArgmaxSlices;
  uint32_t col = t + 256 * slice;
  // columns are visited in increasing order, so `>` alone keeps the lowest index among equals
  for (; col + (kArgmaxUnroll - 1) * step < n; col += kArgmaxUnroll * step) {
    float value[kArgmaxUnroll], low[kArgmaxUnroll];
#pragma unroll
    for (int u = 0; u < kArgmaxUnroll; ++u) {
      value[u] = row_logits[col + u * step];
      low[u] = pairs ? row_low[col + u * step] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < kArgmaxUnroll; ++u) {
      value[u] += low[u];
      if (row_half != nullptr) row_half[col + u * step] = float_to_half_bits(value[u]);
    }
#pragma unroll
    for (int u = 0; u < kArgmaxUnroll; ++u)
      if (!found || value[u] > best_value) {
        best_value = value[u];
        best_index = col + u * step;
        found = true;
      }
  }
  for (; col < n; col += step) {
    const float value = row_logits[col] + (pairs ? row_low[col] : 0.0f);
    if (row_half != nullptr) row_half[col] = float_to_half_bits(value);
    if (!found || value > best_value) {
      best_value = value;
      best_index = col;
      found = true;
    }
  }
  // a slice that saw no column keeps (lowest float, index 0), which never beats a real column
  // except against equal values at a higher index - impossible for index 0
  slice_values[slice][t] = found ? best_value : -3.402823466e+38f;
  slice_indices[slice][t] = found ? best_index : 0xffffffffu;
  __syncthreads();
  if (slice == 0) {
    float value = slice_values[0][t];
    uint32_t index = slice_indices[0][t];
#pragma unroll
    for (int other = 1; other < kArgmaxSlices; ++other)
      if (slice_indices[other][t] != 0xffffffffu &&
          (index == 0xffffffffu || better(slice_values[other][t], slice_indices[other][t], value, index))) {
        value = slice_values[other][t];
        index = slice_indices[other][t];
      }
    // a candidate with no column at all (n <= t): the reference's initial (lowest float, 0)
    if (index == 0xffffffffu) {
      value = -3.402823466e+38f;
      index = 0;
    }
    candidates[row * 256 + t] = {value, index};
  }
}

// lib/metal_w4a16_source.ml:1287-1315
__global__ __launch_bounds__(256) void argmax_reduce_kernel(const Candidate *candidates, uint32_t *token_ids) {
  __shared__ float best_values[256];
  __shared__ uint32_t best_indices[256];
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  best_values[tid] = candidates[row * 256 + tid].value;
  best_indices[tid] = candidates[row * 256 + tid].index;
  __syncthreads();
  for (uint32_t width = 128; width > 0; width >>= 1) {
    if (tid < width && better(best_values[tid + width], best_indices[tid + width], best_values[tid],
                              best_indices[tid])) {
      best_values[tid] = best_values[tid + width];
      best_indices[tid] = best_indices[tid + width];
    }
    __syncthreads();
  }
  if (tid == 0) token_ids[row] = best_indices[0];
}

}  // namespace

hipError_t launch_rms_norm(const RmsNormArgs &a, hipStream_t stream) {
  const dim3 grid((a.rows + kRowWaves - 1) / kRowWaves), block(kRowWaves * 64);
  if (a.input_f32) {
    const float *in = static_cast<const float *>(a.input);
    if (a.weight_first)
      hipLaunchKernelGGL((rms_norm_kernel<float, true>), grid, block, 0, stream, in, a.weight, a.output, a.rows,
                         a.width, a.epsilon);
    else
      hipLaunchKernelGGL((rms_norm_kernel<float, false>), grid, block, 0, stream, in, a.weight, a.output,
                         a.rows, a.width, a.epsilon);
  } else {
    const uint16_t *in = static_cast<const uint16_t *>(a.input);
    const bool vector_rows = a.width % 8 == 0 && a.width <= 64 * 8 * kRmsVectors &&
                             reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                             reinterpret_cast<uintptr_t>(a.weight) % 16 == 0 &&
                             reinterpret_cast<uintptr_t>(a.output) % 16 == 0;
    if (vector_rows) {
      if (a.weight_first)
        hipLaunchKernelGGL((rms_norm_f16_rows_kernel<true>), grid, block, 0, stream, in, a.weight, a.output, a.rows,
                           a.width, a.epsilon);
      else
        hipLaunchKernelGGL((rms_norm_f16_rows_kernel<false>), grid, block, 0, stream, in, a.weight, a.output, a.rows,
                           a.width, a.epsilon);
      return hipGetLastError();
    }
    if (a.weight_first)
      hipLaunchKernelGGL((rms_norm_kernel<uint16_t, true>), grid, block, 0, stream, in, a.weight, a.output,
                         a.rows, a.width, a.epsilon);
    else
      hipLaunchKernelGGL((rms_norm_kernel<uint16_t, false>), grid, block, 0, stream, in, a.weight, a.output,
                         a.rows, a.width, a.epsilon);
  }
  return hipGetLastError();
}

hipError_t launch_rotary_qk(const RotaryQkArgs &a, hipStream_t stream) {
  const uint32_t rows = a.batches * (a.q_heads + a.k_heads) * a.tokens;
  hipLaunchKernelGGL(rotary_qk_kernel, dim3((rows + kRowWaves - 1) / kRowWaves), dim3(kRowWaves * 64), 0,
                     stream, a);
  return hipGetLastError();
}

hipError_t launch_embedding(const EmbeddingArgs &a, hipStream_t stream) {
  const size_t count = (size_t)a.tokens * a.width;
  hipLaunchKernelGGL(embedding_kernel, dim3((uint32_t)((count + 255) / 256)), dim3(256), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_add_f16(const PointwiseArgs &a, hipStream_t stream) {
  bool same_shape = !a.left_scalar && !a.right_scalar && a.count % 8 == 0;
  for (uint32_t axis = 0; axis < a.rank && same_shape; ++axis)
    same_shape = a.left_shape[axis] == a.output_shape[axis] && a.right_shape[axis] == a.output_shape[axis];
  const auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (same_shape && aligned(a.left) && aligned(a.right) && aligned(a.output)) {
    const uint32_t vectors = a.count / 8;
    hipLaunchKernelGGL(add_f16_same_shape_kernel, dim3((vectors + 255) / 256), dim3(256), 0, stream,
                       reinterpret_cast<const uint4 *>(a.left), reinterpret_cast<const uint4 *>(a.right),
                       reinterpret_cast<uint4 *>(a.output), vectors);
  } else {
    hipLaunchKernelGGL(add_f16_kernel, dim3((a.count + 255) / 256), dim3(256), 0, stream, a);
  }
  return hipGetLastError();
}

namespace {
// The per-step state of a retained decode plan, written in stream order ahead of its graph:
// the input token (given, or the previous step's output token: llmopt_chain_token_id,
// native/ocaml_metal_stubs.m:1570-1577) and the context length every sequence attends to.
__global__ void plan_state_kernel(int64_t *token, int64_t value, const int32_t *chain_from, uint32_t *past,
                                  uint32_t past_value, uint32_t past_count, uint32_t *checkpoint,
                                  uint32_t checkpoint_value) {
  if (threadIdx.x == 0 && token != nullptr) *token = chain_from != nullptr ? (int64_t)*chain_from : value;
  if (threadIdx.x == 0 && checkpoint != nullptr) *checkpoint = checkpoint_value;
  for (uint32_t i = threadIdx.x; i < past_count; i += blockDim.x) past[i] = past_value;
}

// *found = 1 when the range holds a NaN (not an infinity): fp16 words, or float32 words.
__global__ void nan_scan_kernel(const uint8_t *data, size_t words, bool f32, uint32_t *found) {
  bool seen = false;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (size_t)gridDim.x * blockDim.x) {
    if (f32) {
      const uint32_t v = reinterpret_cast<const uint32_t *>(data)[i];
      seen |= (v & 0x7F800000u) == 0x7F800000u && (v & 0x007FFFFFu) != 0;
    } else {
      const uint16_t v = reinterpret_cast<const uint16_t *>(data)[i];
      seen |= (v & 0x7C00u) == 0x7C00u && (v & 0x03FFu) != 0;
    }
  }
  if (seen) *found = 1u;  // every writer stores the same value
}
}  // namespace

hipError_t launch_nan_scan(const void *data, size_t bytes, bool f32, uint32_t *found, hipStream_t stream) {
  const size_t words = bytes / (f32 ? 4 : 2);
  if (words == 0) return hipSuccess;
  const uint32_t blocks = (uint32_t)std::min<size_t>((words + 255) / 256, 2048);
  hipLaunchKernelGGL(nan_scan_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const uint8_t *>(data), words, f32,
                     found);
  return hipGetLastError();
}

hipError_t launch_plan_state(int64_t *token, int64_t value, const int32_t *chain_from, uint32_t *past,
                             uint32_t past_value, uint32_t past_count, uint32_t *checkpoint, uint32_t checkpoint_value,
                             hipStream_t stream) {
  hipLaunchKernelGGL(plan_state_kernel, dim3(1), dim3(256), 0, stream, token, value, chain_from, past, past_value,
                     past_count, checkpoint, checkpoint_value);
  return hipGetLastError();
}

hipError_t launch_copy_bytes(void *destination, const void *source, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const bool vector_ok = ((reinterpret_cast<uintptr_t>(destination) | reinterpret_cast<uintptr_t>(source)) & 15) == 0;
  const size_t vectors = vector_ok ? bytes / 16 : 0;
  if (vectors > 0) {
    const size_t wanted = (vectors + 255) / 256;
    const uint32_t blocks = (uint32_t)std::min<size_t>(wanted, 8192);
    hipLaunchKernelGGL(copy_vectors_kernel, dim3(blocks), dim3(256), 0, stream,
                       static_cast<const u32x4_t *>(source), static_cast<u32x4_t *>(destination), vectors);
  }
  const size_t done = vectors * 16;
  if (done < bytes) {
    const size_t rest = bytes - done;
    const uint32_t blocks = (uint32_t)std::min<size_t>((rest + 255) / 256, 8192);
    hipLaunchKernelGGL(copy_bytes_kernel, dim3(blocks), dim3(256), 0, stream,
                       static_cast<const uint8_t *>(source) + done, static_cast<uint8_t *>(destination) + done, rest);
  }
  return hipGetLastError();
}

hipError_t launch_argmax_candidates(const float *logits, void *candidates, uint32_t rows, uint32_t n, bool pairs,
                                    uint16_t *half_logits, hipStream_t stream) {
  hipLaunchKernelGGL(argmax_candidates_kernel, dim3(rows), dim3(256 * kArgmaxSlices), 0, stream, logits,
                     static_cast<Candidate *>(candidates), n, pairs, half_logits);
  return hipGetLastError();
}

hipError_t launch_rms_norm_split(const RmsNormArgs &a, hipStream_t stream) {
  const dim3 grid((a.rows + kRowWaves - 1) / kRowWaves), block(kRowWaves * 64);
  if (a.input_f32)
    hipLaunchKernelGGL(rms_norm_split_kernel<float>, grid, block, 0, stream, static_cast<const float *>(a.input),
                       a.weight, a.output, a.rows, a.width, a.epsilon);
  else
    hipLaunchKernelGGL(rms_norm_split_kernel<uint16_t>, grid, block, 0, stream,
                       static_cast<const uint16_t *>(a.input), a.weight, a.output, a.rows, a.width, a.epsilon);
  return hipGetLastError();
}

hipError_t launch_argmax_reduce(const void *candidates, uint32_t *token_ids, uint32_t rows, hipStream_t stream) {
  hipLaunchKernelGGL(argmax_reduce_kernel, dim3(rows), dim3(256), 0, stream,
                     static_cast<const Candidate *>(candidates), token_ids);
  return hipGetLastError();
}

}  // namespace llmopt
