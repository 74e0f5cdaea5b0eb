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
    const float x = half_bits_to_float(source[source_index]);
    const float maximum = wave_max(fabsf(x));
    const uint16_t stored = float_to_half_bits(maximum == 0.0f ? 1.0f : maximum / 127.0f);
    const float scale = half_bits_to_float(stored);
    const float rounded = rintf(x / scale);
    const int quantized = (int)fminf(fmaxf(rounded, -127.0f), 127.0f);
    values[segment_offset + local_offset + lane] = (int8_t)quantized;
    if (lane == 0) scales[(segment_offset >> 6) + local_group] = stored;
  }
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

hipError_t launch_q8_unpack(const Q8UnpackArgs &args, hipStream_t stream) {
  const size_t vectors = (size_t)args.items * args.heads * args.head_dim / 4;
  if (vectors == 0) return hipSuccess;
  const uint32_t blocks = (uint32_t)((vectors + 255) / 256);
  hipLaunchKernelGGL(q8_unpack_kernel, dim3(blocks), dim3(256), 0, stream, args);
  return hipGetLastError();
}

}  // namespace llmopt
