// Grouped-Q8 KV cache quantiser and dequantiser for gfx950.
//
// Arithmetic of llmopt_cache_pack_attention_q8{,_simd,_pair_simd} and
// llmopt_cache_unpack_attention_q8{,_vec4} (lib/metal_cache_source.ml:46-243):
// per (token, kv head, 64-wide group) the stored scale is
// half(max|x| / 127) (1.0 for an all-zero group) and
// q = clamp(rint(x / float(scale)), -127, 127), all in float32 with
// round-half-even.  Pool slot layout (lib/kv_cache.ml:126-166): token_elements
// int8 values followed by token_elements/64 fp16 scales.
//
// One wave handles one 64-wide group: lane i owns element i, the maximum is a
// DPP wave reduction, the int8 store is a fully coalesced 64-byte row.
#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

template <bool PAIR>
__global__ __launch_bounds__(256) void q8_pack_kernel(Q8PackArgs a) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t groups_per_head = a.head_dim >> 6;
  const uint32_t segment_groups = a.heads * groups_per_head;
  const uint32_t total = a.items * segment_groups;
  const uint32_t logical_group = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (logical_group >= total) return;
  const uint32_t item = logical_group / segment_groups;
  const uint32_t local_group = logical_group - item * segment_groups;
  const uint32_t head = local_group / groups_per_head;
  const uint32_t group_in_head = local_group - head * groups_per_head;
  const size_t source_row =
      a.item_major ? (size_t)item * a.heads + head : (size_t)head * a.source_items + a.source_offset + item;
  const size_t source_index = source_row * a.head_dim + (size_t)group_in_head * 64 + lane;
  const size_t slot_base = (size_t)a.slots[item] * a.token_stride;
  int8_t *values = reinterpret_cast<int8_t *>(a.pool + slot_base);
  uint16_t *scales = reinterpret_cast<uint16_t *>(a.pool + slot_base + a.token_elements);
  const uint32_t local_offset = head * a.head_dim + group_in_head * 64;
#pragma unroll
  for (int which = 0; which < (PAIR ? 2 : 1); ++which) {
    const uint16_t *source = which == 0 ? a.source[0] : a.source[1];
    const uint32_t segment_offset = a.segment_offset[which];
    uint16_t stored;
    values[segment_offset + local_offset + lane] = q8_quantize(half_bits_to_float(source[source_index]), &stored);
    if (lane == 0) scales[(segment_offset >> 6) + local_group] = stored;
  }
}

// One wave per row of head_dim values, four rows per workgroup: the query rows of every
// (sequence, token) (rotated), then the key rows (rotated, stored as fp16 for this step's attention
// and as Q8 in the token's pool slot), then the value rows (Q8 only).  A row is walked in 64-wide
// pieces, which are the Q8 groups.  Inputs are token-major [sequence, token, head, width], the
// rotated outputs head-major [sequence, head, token, width] as llmopt_rotary_qk_f16_simd_h64
// leaves them (lib/metal_normalization_source.ml:765-802); with one token per sequence - a decode
// step - the two are the same.  Slot and, when the table is not shared, cosine / sine row of item
// sequence * tokens + token.
__global__ __launch_bounds__(256) void rotary_qk_pack_kernel(RotaryPackArgs a) {
  const RotaryQkArgs &r = a.rotary;
  const Q8PackArgs &p = a.pack;
  const uint32_t lane = threadIdx.x & 63;
  // the row is the same for the whole wave, and said to be: which input, which output and which
  // segment the wave takes are then scalar selects among the arguments, and its pool slot a scalar
  // load - left to per-lane values they were vector loads from the argument block and the slot
  // table, each a trip to memory the row's own loads had to wait for
  const uint32_t row = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t items = r.batches * r.tokens;
  const uint32_t q_rows = items * r.q_heads, kv_rows = items * r.k_heads;
  if (row >= q_rows + 2 * kv_rows) return;
  const bool is_q = row < q_rows;
  const bool is_v = row >= q_rows + kv_rows;
  const uint32_t local_row = is_q ? row : is_v ? row - q_rows - kv_rows : row - q_rows;  // [sequence, token, head]
  const uint32_t heads = is_q ? r.q_heads : r.k_heads;
  const uint32_t item = local_row / heads;
  const uint32_t head = local_row - item * heads;
  const uint32_t batch = item / r.tokens, token = item - batch * r.tokens;
  const size_t base = (size_t)local_row * r.width;
  const _Float16 *input = reinterpret_cast<const _Float16 *>(is_q ? r.q_input : is_v ? p.source[1] : r.k_input) + base;
  _Float16 *output = reinterpret_cast<_Float16 *>(is_q ? r.q_output : r.k_output) +
                     (((size_t)batch * heads + head) * r.tokens + token) * r.width;
  const size_t trig_base = ((size_t)(r.trig_batches == 1 ? 0 : batch) * r.tokens + token) * r.width;
  const _Float16 *cosine = reinterpret_cast<const _Float16 *>(r.cosine) + trig_base;
  const _Float16 *sine = reinterpret_cast<const _Float16 *>(r.sine) + trig_base;
  size_t slot_base = 0;
  if (!is_q) slot_base = (size_t)p.slots[item] * p.token_stride;
  int8_t *values = reinterpret_cast<int8_t *>(p.pool + slot_base);
  uint16_t *scales = reinterpret_cast<uint16_t *>(p.pool + slot_base + p.token_elements);
  const uint32_t segment_offset = p.segment_offset[is_v ? 1 : 0];
  for (uint32_t col = lane; col < r.width; col += 64) {
    _Float16 value;
    if (is_v) {
      value = input[col];
    } else {
      value = rotate_half_element(input, cosine, sine, col, r.half_dimension);
      output[col] = value;
    }
    if (is_q) continue;
    uint16_t stored;
    values[segment_offset + head * r.width + col] = q8_quantize((float)value, &stored);
    if (lane == 0) scales[(segment_offset >> 6) + head * (r.width >> 6) + (col >> 6)] = stored;
  }
}

// One wave per 64-wide group of the layer's state.
__global__ __launch_bounds__(256) void q8_checkpoint_pack_kernel(Q8CheckpointArgs a) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t layer_groups = a.layer_elements >> 6;
  const uint32_t group = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (group >= layer_groups) return;
  const uint32_t checkpoint = min(a.device_checkpoint ? *a.device_checkpoint : a.checkpoint, a.max_checkpoint);
  uint8_t *slot = a.pool + (size_t)checkpoint * a.checkpoint_stride;
  int8_t *values = reinterpret_cast<int8_t *>(slot);
  uint16_t *scales = reinterpret_cast<uint16_t *>(slot + a.checkpoint_elements);
  uint16_t stored;
  values[(size_t)a.layer * a.layer_elements + group * 64 + lane] =
      q8_quantize(half_bits_to_float(a.source[(size_t)group * 64 + lane]), &stored);
  if (lane == 0) scales[(size_t)a.layer * layer_groups + group] = stored;
}

// One thread per four consecutive values.
__global__ __launch_bounds__(256) void q8_checkpoint_unpack_kernel(Q8CheckpointArgs a) {
  const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= a.layer_elements / 4) return;
  const uint32_t local = (uint32_t)index * 4;
  const uint32_t checkpoint = min(a.device_checkpoint ? *a.device_checkpoint : a.checkpoint, a.max_checkpoint);
  const uint8_t *slot = a.pool + (size_t)checkpoint * a.checkpoint_stride;
  // (a checkpoint slot is only 2-byte aligned: its stride is elements + 2 * groups)
  typedef uint32_t unaligned_u32_t __attribute__((aligned(1)));
  const uint32_t packed = *reinterpret_cast<const unaligned_u32_t *>(slot + (size_t)a.layer * a.layer_elements + local);
  const uint16_t *scales = reinterpret_cast<const uint16_t *>(slot + a.checkpoint_elements);
  const float scale = half_bits_to_float(scales[(size_t)a.layer * (a.layer_elements >> 6) + (local >> 6)]);
  uint16_t out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) out[i] = float_to_half_bits((float)(int8_t)((packed >> (8 * i)) & 0xffu) * scale);
  *reinterpret_cast<uint2 *>(a.destination + local) =
      make_uint2((uint32_t)out[0] | ((uint32_t)out[1] << 16), (uint32_t)out[2] | ((uint32_t)out[3] << 16));
}

__global__ __launch_bounds__(256) void q8_unpack_kernel(Q8UnpackArgs a) {
  // one thread per 4 consecutive elements of one (item, head)
  const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t segment_elements = a.heads * a.head_dim;
  const size_t vectors = (size_t)a.items * segment_elements / 4;
  if (index >= vectors) return;
  const size_t linear = index * 4;
  const uint32_t item = (uint32_t)(linear / segment_elements);
  const uint32_t local = (uint32_t)(linear - (size_t)item * segment_elements);
  const uint32_t head = local / a.head_dim;
  const uint32_t within_head = local - head * a.head_dim;
  const uint32_t local_group = head * (a.head_dim >> 6) + (within_head >> 6);
  const size_t slot_base = (size_t)a.slots[item] * a.token_stride;
  const uint32_t packed =
      *reinterpret_cast<const uint32_t *>(a.pool + slot_base + a.segment_offset + local);
  const uint16_t *scales = reinterpret_cast<const uint16_t *>(a.pool + slot_base + a.token_elements);
  const float scale = half_bits_to_float(scales[(a.segment_offset >> 6) + local_group]);
  uint16_t out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    out[i] = float_to_half_bits((float)(int8_t)((packed >> (8 * i)) & 0xffu) * scale);
  uint16_t *destination = a.destination + ((size_t)head * a.items + item) * a.head_dim + within_head;
  *reinterpret_cast<uint2 *>(destination) =
      make_uint2((uint32_t)out[0] | ((uint32_t)out[1] << 16), (uint32_t)out[2] | ((uint32_t)out[3] << 16));
}

}  // namespace

hipError_t launch_q8_pack(const Q8PackArgs &args, bool pair, hipStream_t stream) {
  const uint32_t groups = args.items * args.heads * (args.head_dim >> 6);
  if (groups == 0) return hipSuccess;
  const uint32_t blocks = (groups + 3) / 4;
  if (pair)
    hipLaunchKernelGGL(q8_pack_kernel<true>, dim3(blocks), dim3(256), 0, stream, args);
  else
    hipLaunchKernelGGL(q8_pack_kernel<false>, dim3(blocks), dim3(256), 0, stream, args);
  return hipGetLastError();
}

hipError_t launch_rotary_qk_pack(const RotaryPackArgs &args, hipStream_t stream) {
  const RotaryQkArgs &r = args.rotary;
  if (r.tokens == 0 || r.width % 64 != 0 || args.pack.items != r.batches * r.tokens || args.pack.heads != r.k_heads ||
      args.pack.head_dim != r.width || !args.pack.item_major)
    return hipErrorInvalidValue;
  const uint32_t rows = r.batches * r.tokens * (r.q_heads + 2 * r.k_heads);
  if (rows == 0) return hipSuccess;
  hipLaunchKernelGGL(rotary_qk_pack_kernel, dim3((rows + 3) / 4), dim3(256), 0, stream, args);
  return hipGetLastError();
}

hipError_t launch_q8_checkpoint_pack(const Q8CheckpointArgs &args, hipStream_t stream) {
  const uint32_t groups = args.layer_elements >> 6;
  if (groups == 0) return hipSuccess;
  hipLaunchKernelGGL(q8_checkpoint_pack_kernel, dim3((groups + 3) / 4), dim3(256), 0, stream, args);
  return hipGetLastError();
}

hipError_t launch_q8_checkpoint_unpack(const Q8CheckpointArgs &args, hipStream_t stream) {
  const uint32_t vectors = args.layer_elements / 4;
  if (vectors == 0) return hipSuccess;
  hipLaunchKernelGGL(q8_checkpoint_unpack_kernel, dim3((vectors + 255) / 256), dim3(256), 0, stream, args);
  return hipGetLastError();
}

hipError_t launch_q8_unpack(const Q8UnpackArgs &args, hipStream_t stream) {
  const size_t vectors = (size_t)args.items * args.heads * args.head_dim / 4;
  if (vectors == 0) return hipSuccess;
  const uint32_t blocks = (uint32_t)((vectors + 255) / 256);
  hipLaunchKernelGGL(q8_unpack_kernel, dim3(blocks), dim3(256), 0, stream, args);
  return hipGetLastError();
}

}  // namespace llmopt
