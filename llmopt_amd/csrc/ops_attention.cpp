// Entry points of the grouped-Q8 KV cache and paged decode attention family:
// buffer order and parameter-block layout of lib/metal_cache_source.ml:9-34,
// 46-243,352-583 (host side lib/metal_cache.ml:230-511,
// lib/metal_dispatch_attention.ml:104-217, lib/metal_parameters.ml:119-140).
#include <algorithm>

#include "kernels/kernels.h"
#include "runtime.h"

namespace llmopt {
namespace {

int launched(hipError_t status, const char *name) {
  if (status != hipSuccess)
    return fail(LLMOPT_ERR_FAILURE, "%s launch failed: %s", name, hipGetErrorString(status));
  return LLMOPT_OK;
}

int check_cache_geometry(const char *name, uint32_t heads, uint32_t head_dim, uint32_t group_size,
                         uint32_t token_elements, uint32_t token_stride) {
  if (group_size != 64)
    return fail(LLMOPT_ERR_INVALID, "%s supports the Q8 group size 64 only, got %u", name, group_size);
  if (heads == 0 || head_dim == 0 || head_dim % 64 != 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires head_dim to be a positive multiple of 64", name);
  if (token_elements % 64 != 0 || token_stride < token_elements + 2 * (token_elements / 64))
    return fail(LLMOPT_ERR_INVALID, "%s received an inconsistent Q8 token layout", name);
  return LLMOPT_OK;
}

// AttentionCacheParams, 10 x u32 (lib/metal_cache_source.ml:9-20).
// buffers: source, slots, pool.
int cache_pack(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (int status = require_parameter_bytes(record, 40)) return status;
  Q8PackArgs args = {};
  args.items = param_u32(record, 0);
  args.segment_offset[0] = param_u32(record, 4);
  args.heads = param_u32(record, 8);
  args.head_dim = param_u32(record, 12);
  const uint32_t group_size = param_u32(record, 16);
  args.token_elements = param_u32(record, 20);
  args.token_stride = param_u32(record, 28);
  args.source_items = param_u32(record, 32);
  args.source_offset = param_u32(record, 36);
  if (int status = check_cache_geometry(record.name.c_str(), args.heads, args.head_dim, group_size,
                                        args.token_elements, args.token_stride))
    return status;
  if (args.segment_offset[0] % 64 != 0 ||
      (uint64_t)args.segment_offset[0] + (uint64_t)args.heads * args.head_dim > args.token_elements)
    return fail(LLMOPT_ERR_INVALID, "%s segment lies outside the token", record.name.c_str());
  if ((uint64_t)args.source_offset + args.items > args.source_items)
    return fail(LLMOPT_ERR_INVALID, "%s source window lies outside the source", record.name.c_str());
  if (int status = require_buffer_size(
          record.buffers[0], (uint64_t)args.heads * args.source_items * args.head_dim * 2, "cache source"))
    return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)args.items * 4, "slots")) return status;
  if (int status = require_buffer_size(record.buffers[2], args.token_stride, "pool")) return status;
  args.source[0] = reinterpret_cast<const uint16_t *>(record.buffers[0].device);
  args.slots = reinterpret_cast<const uint32_t *>(record.buffers[1].device);
  args.pool = record.buffers[2].device;
  return launched(launch_q8_pack(args, false, context->stream), record.name.c_str());
}

// AttentionCachePairParams, 11 x u32 (lib/metal_cache_source.ml:22-34).
// buffers: key_source, value_source, slots, pool.
// `at`: byte offset of the 11 words in the record's parameters; the buffers are
// record.buffers[key], [value], [slots], [pool].
int parse_pack_pair(const DispatchRecord &record, size_t at, size_t key, size_t value, size_t slots, size_t pool,
                    bool item_major, Q8PackArgs *out) {
  Q8PackArgs args = {};
  args.items = param_u32(record, at + 0);
  args.segment_offset[0] = param_u32(record, at + 4);
  args.segment_offset[1] = param_u32(record, at + 8);
  args.heads = param_u32(record, at + 12);
  args.head_dim = param_u32(record, at + 16);
  const uint32_t group_size = param_u32(record, at + 20);
  args.token_elements = param_u32(record, at + 24);
  args.token_stride = param_u32(record, at + 32);
  args.source_items = param_u32(record, at + 36);
  args.source_offset = param_u32(record, at + 40);
  args.item_major = item_major ? 1 : 0;
  if (item_major) {
    args.source_items = args.items;
    args.source_offset = 0;
  }
  if (int status = check_cache_geometry(record.name.c_str(), args.heads, args.head_dim, group_size,
                                        args.token_elements, args.token_stride))
    return status;
  for (int which = 0; which < 2; ++which)
    if (args.segment_offset[which] % 64 != 0 ||
        (uint64_t)args.segment_offset[which] + (uint64_t)args.heads * args.head_dim > args.token_elements)
      return fail(LLMOPT_ERR_INVALID, "%s segment lies outside the token", record.name.c_str());
  if ((uint64_t)args.source_offset + args.items > args.source_items)
    return fail(LLMOPT_ERR_INVALID, "%s source window lies outside the source", record.name.c_str());
  const uint64_t source_bytes = (uint64_t)args.heads * args.source_items * args.head_dim * 2;
  if (int status = require_buffer_size(record.buffers[key], source_bytes, "key source")) return status;
  if (int status = require_buffer_size(record.buffers[value], source_bytes, "value source")) return status;
  if (int status = require_buffer_size(record.buffers[slots], (uint64_t)args.items * 4, "slots")) return status;
  if (int status = require_buffer_size(record.buffers[pool], args.token_stride, "pool")) return status;
  args.source[0] = reinterpret_cast<const uint16_t *>(record.buffers[key].device);
  args.source[1] = reinterpret_cast<const uint16_t *>(record.buffers[value].device);
  args.slots = reinterpret_cast<const uint32_t *>(record.buffers[slots].device);
  args.pool = record.buffers[pool].device;
  *out = args;
  return LLMOPT_OK;
}

int cache_pack_pair_layout(llmopt_hip_context *context, const DispatchRecord &record, bool item_major) {
  if (int status = require_buffer_count(record, 4)) return status;
  if (int status = require_parameter_bytes(record, 44)) return status;
  Q8PackArgs args = {};
  if (int status = parse_pack_pair(record, 0, 0, 1, 2, 3, item_major, &args)) return status;
  return launched(launch_q8_pack(args, true, context->stream), record.name.c_str());
}

int cache_pack_pair(llmopt_hip_context *context, const DispatchRecord &record) {
  return cache_pack_pair_layout(context, record, false);
}

// Extension (no reference kernel): the same pair quantiser for one new token of
// each of `items` sequences, sources laid out [items, heads, head_dim].
int cache_pack_pair_batched(llmopt_hip_context *context, const DispatchRecord &record) {
  return cache_pack_pair_layout(context, record, true);
}

// Extension (no reference kernel): llmopt_rotary_qk_f16_simd_h64 followed by
// llmopt_cache_pack_attention_q8_pair_batched on the rotated keys, as one launch - a decode
// step is bound by its number of launches.  Parameters: RotaryQKParams (7 words, tokens = 1)
// then AttentionCachePairParams (11 words); buffers: q_input, k_input, cosine, sine, q_output,
// k_output (also the quantiser's key source), value source, slots, pool.
int rotary_qk_pack_batched(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 9)) return status;
  if (int status = require_parameter_bytes(record, 28 + 44)) return status;
  RotaryPackArgs args = {};
  if (int status = parse_rotary_qk(record, &args.rotary)) return status;
  if (int status = parse_pack_pair(record, 28, 5, 6, 7, 8, true, &args.pack)) return status;
  if ((uint64_t)args.pack.items != (uint64_t)args.rotary.batches * args.rotary.tokens ||
      args.pack.heads != args.rotary.k_heads || args.pack.head_dim != args.rotary.width)
    return fail(LLMOPT_ERR_INVALID, "%s requires the same tokens (sequences x tokens items), KV heads and width "
                "in both parameter blocks", record.name.c_str());
  return launched(launch_rotary_qk_pack(args, context->stream), record.name.c_str());
}

// buffers: pool, slots, destination; AttentionCacheParams.
int cache_unpack(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (int status = require_parameter_bytes(record, 40)) return status;
  Q8UnpackArgs args = {};
  args.items = param_u32(record, 0);
  args.segment_offset = param_u32(record, 4);
  args.heads = param_u32(record, 8);
  args.head_dim = param_u32(record, 12);
  const uint32_t group_size = param_u32(record, 16);
  args.token_elements = param_u32(record, 20);
  args.token_stride = param_u32(record, 28);
  if (int status = check_cache_geometry(record.name.c_str(), args.heads, args.head_dim, group_size,
                                        args.token_elements, args.token_stride))
    return status;
  if (args.segment_offset % 64 != 0 ||
      (uint64_t)args.segment_offset + (uint64_t)args.heads * args.head_dim > args.token_elements)
    return fail(LLMOPT_ERR_INVALID, "%s segment lies outside the token", record.name.c_str());
  if (int status = require_buffer_size(record.buffers[0], args.token_stride, "pool")) return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)args.items * 4, "slots")) return status;
  if (int status = require_buffer_size(
          record.buffers[2], (uint64_t)args.heads * args.items * args.head_dim * 2, "cache destination"))
    return status;
  args.pool = record.buffers[0].device;
  args.slots = reinterpret_cast<const uint32_t *>(record.buffers[1].device);
  args.destination = reinterpret_cast<uint16_t *>(record.buffers[2].device);
  return launched(launch_q8_unpack(args, context->stream), record.name.c_str());
}

// CheckpointCacheParams, 28 bytes (lib/metal_cache_source.ml:36-44): checkpoint 0, layer 4,
// layer_elements 8, group_size 12, checkpoint_elements 16, checkpoint_groups 20, checkpoint_stride 24.
// pack buffers: source, pool; unpack buffers: pool, destination.
int cache_checkpoint(llmopt_hip_context *context, const DispatchRecord &record, bool pack) {
  if (int status = require_buffer_count(record, 2)) return status;
  if (int status = require_parameter_bytes(record, 28)) return status;
  const char *name = record.name.c_str();
  Q8CheckpointArgs args = {};
  args.checkpoint = param_u32(record, 0);
  args.layer = param_u32(record, 4);
  args.layer_elements = param_u32(record, 8);
  const uint32_t group_size = param_u32(record, 12);
  args.checkpoint_elements = param_u32(record, 16);
  const uint32_t checkpoint_groups = param_u32(record, 20);
  args.checkpoint_stride = param_u32(record, 24);
  if (group_size != 64) return fail(LLMOPT_ERR_INVALID, "%s supports the Q8 group size 64 only, got %u", name, group_size);
  if (args.layer_elements % 64 != 0 || args.checkpoint_elements % 64 != 0 ||
      checkpoint_groups != args.checkpoint_elements / 64 ||
      (uint64_t)args.checkpoint_stride < (uint64_t)args.checkpoint_elements + 2ull * checkpoint_groups ||
      args.checkpoint_stride % 2 != 0)
    return fail(LLMOPT_ERR_INVALID, "%s received an inconsistent Q8 checkpoint layout", name);
  if (((uint64_t)args.layer + 1) * args.layer_elements > args.checkpoint_elements)
    return fail(LLMOPT_ERR_INVALID, "%s layer lies outside the checkpoint", name);
  const BoundBuffer &pool = record.buffers[pack ? 1 : 0];
  const BoundBuffer &state = record.buffers[pack ? 0 : 1];
  if (int status = require_buffer_size(pool, args.checkpoint_stride, "checkpoint pool")) return status;
  args.max_checkpoint = (uint32_t)std::min<uint64_t>(pool.length / args.checkpoint_stride - 1, 0xffffffffull);
  if (record.device_checkpoint == nullptr && args.checkpoint > args.max_checkpoint)
    return fail(LLMOPT_ERR_INVALID, "HIP checkpoint pool buffer is too small: required=%llu actual=%llu",
                (unsigned long long)(args.checkpoint + 1ull) * args.checkpoint_stride, (unsigned long long)pool.length);
  if (int status = require_buffer_size(state, (uint64_t)args.layer_elements * 2, pack ? "checkpoint source" : "checkpoint destination"))
    return status;
  if ((reinterpret_cast<uintptr_t>(pool.device) & 1) != 0 || (reinterpret_cast<uintptr_t>(state.device) & 7) != 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires 2-byte aligned pools and 8-byte aligned states", name);
  args.pool = pool.device;
  args.device_checkpoint = record.device_checkpoint;
  if (pack) {
    args.source = reinterpret_cast<const uint16_t *>(state.device);
    return launched(launch_q8_checkpoint_pack(args, context->stream), name);
  }
  args.destination = reinterpret_cast<uint16_t *>(state.device);
  return launched(launch_q8_checkpoint_unpack(args, context->stream), name);
}

int cache_pack_checkpoint(llmopt_hip_context *context, const DispatchRecord &record) {
  return cache_checkpoint(context, record, true);
}

int cache_unpack_checkpoint(llmopt_hip_context *context, const DispatchRecord &record) {
  return cache_checkpoint(context, record, false);
}

// Q8PagedAttentionParams, 64 bytes (lib/metal_cache_source.ml:352-369):
// batches 0, query_heads 4, kv_heads 8, past_length 12, head_dim 16,
// mask_batches 20, mask_heads 24, token_elements 28, key_offset 32,
// value_offset 36, group_size 40, token_stride 44, scale(f32) 48,
// query_length 52, mask_dtype 56, window 60.
// buffers: query, current_key, current_value, pool, slots, mask (the slots
// buffer again when there is no mask), output.
//
// The batched extension appends u32 max_past_length at byte 64 and two
// buffers: past_lengths u32[batches], slot_offsets u32[batches].
// projecting (extension llmopt_attention_q8_paged_batched_w4a16_partial_g64, batched only): the output rows
// are not stored but multiplied, head by head, into an output projection; buffer 6 receives the float32
// partial sums [query_heads, batches, hidden] instead, two more buffers hold the projection's packed
// weights [hidden, query_heads * 64 / 2] and scales, and u32 hidden follows the batched parameter words.
int paged_attention(llmopt_hip_context *context, const DispatchRecord &record, bool batched, bool projecting = false) {
  if (int status = require_buffer_count(record, projecting ? 11 : batched ? 9 : 7)) return status;
  if (int status = require_parameter_bytes(record, projecting ? 72 : batched ? 68 : 64)) return status;
  Q8AttentionArgs args = {};
  args.batches = param_u32(record, 0);
  args.query_heads = param_u32(record, 4);
  args.kv_heads = param_u32(record, 8);
  args.past_length = param_u32(record, 12);
  args.head_dim = param_u32(record, 16);
  args.mask_batches = param_u32(record, 20);
  args.mask_heads = param_u32(record, 24);
  args.token_elements = param_u32(record, 28);
  args.key_offset = param_u32(record, 32);
  args.value_offset = param_u32(record, 36);
  const uint32_t group_size = param_u32(record, 40);
  args.token_stride = param_u32(record, 44);
  args.scale = param_f32(record, 48);
  args.query_length = param_u32(record, 52);
  args.mask_dtype = param_u32(record, 56);
  args.window = param_u32(record, 60);
  args.max_past_length = batched ? param_u32(record, 64) : args.past_length;
  const char *name = record.name.c_str();
  const bool retained = !batched && record.device_past_lengths != nullptr;
  if (retained) args.max_past_length = record.device_past_capacity;  // see DispatchRecord
  if (int status = check_cache_geometry(name, args.kv_heads, args.head_dim, group_size,
                                        args.token_elements, args.token_stride))
    return status;
  if (args.batches == 0 || args.query_heads == 0 || args.query_heads % args.kv_heads != 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires query heads to be a multiple of kv heads", name);
  if (args.head_dim > 512)
    return fail(LLMOPT_ERR_INVALID, "%s supports head_dim up to 512, got %u", name, args.head_dim);
  const uint64_t segment = (uint64_t)args.kv_heads * args.head_dim;
  if (args.key_offset % 64 != 0 || args.value_offset % 64 != 0 ||
      args.key_offset + segment > args.token_elements || args.value_offset + segment > args.token_elements)
    return fail(LLMOPT_ERR_INVALID, "%s K/V segments lie outside the token", name);
  if (args.mask_dtype > 2) return fail(LLMOPT_ERR_INVALID, "%s mask dtype %u is unsupported", name, args.mask_dtype);
  const uint32_t q_len = args.query_length == 0 ? 1 : args.query_length;
  const uint64_t q_bytes = (uint64_t)args.batches * args.query_heads * q_len * args.head_dim * 2;
  const uint64_t kv_bytes = (uint64_t)args.batches * args.kv_heads * q_len * args.head_dim * 2;
  if (int status = require_buffer_size(record.buffers[0], q_bytes, "query")) return status;
  if (int status = require_buffer_size(record.buffers[1], kv_bytes, "current key")) return status;
  if (int status = require_buffer_size(record.buffers[2], kv_bytes, "current value")) return status;
  if (args.max_past_length > 0) {
    if (int status = require_buffer_size(record.buffers[3], args.token_stride, "pool")) return status;
    if (int status = require_buffer_size(record.buffers[4], (uint64_t)args.max_past_length * 4, "slots"))
      return status;
  }
  const bool masked = args.mask_batches > 0 && args.mask_dtype != 0;
  if (masked) {
    const uint64_t mask_elements = (uint64_t)args.mask_batches * args.mask_heads * q_len *
                                   ((uint64_t)args.max_past_length + q_len);
    if (int status = require_buffer_size(record.buffers[5], mask_elements * (args.mask_dtype == 2 ? 2 : 1), "mask"))
      return status;
    if (batched && args.mask_batches != 0)
      return fail(LLMOPT_ERR_INVALID, "%s does not take a mask", name);
  }
  if (projecting) {
    args.projected_width = param_u32(record, 68);
    const uint64_t hidden = args.projected_width, width = (uint64_t)args.query_heads * args.head_dim;
    if (hidden == 0 || args.head_dim != 64)
      return fail(LLMOPT_ERR_INVALID, "%s takes heads of 64 and a positive projection width", name);
    if (int status = require_buffer_size(record.buffers[6], (uint64_t)args.query_heads * args.batches * hidden * 4, "partial sums"))
      return status;
    if (int status = require_buffer_size(record.buffers[9], hidden * (width / 2), "projection packed weight")) return status;
    if (int status = require_buffer_size(record.buffers[10], hidden * (width / 64) * 2, "projection scale")) return status;
    args.projection = {record.buffers[9].device, reinterpret_cast<const uint16_t *>(record.buffers[10].device)};
    args.projected = reinterpret_cast<float *>(record.buffers[6].device);
  } else if (int status = require_buffer_size(record.buffers[6], q_bytes, "output")) {
    return status;
  }
  args.query = reinterpret_cast<const uint16_t *>(record.buffers[0].device);
  args.current_key = reinterpret_cast<const uint16_t *>(record.buffers[1].device);
  args.current_value = reinterpret_cast<const uint16_t *>(record.buffers[2].device);
  args.pool = record.buffers[3].device;
  args.pool_bytes = record.buffers[3].length;
  args.slots = reinterpret_cast<const uint32_t *>(record.buffers[4].device);
  args.mask = masked ? record.buffers[5].device : nullptr;
  args.output = projecting ? nullptr : reinterpret_cast<uint16_t *>(record.buffers[6].device);
  if (retained) {
    if (masked) return fail(LLMOPT_ERR_INVALID, "%s with a mask cannot read its context length from device memory", name);
    args.past_lengths = record.device_past_lengths;
  }
  if (batched) {
    if (int status = require_buffer_size(record.buffers[7], (uint64_t)args.batches * 4, "past lengths")) return status;
    if (int status = require_buffer_size(record.buffers[8], (uint64_t)args.batches * 4, "slot offsets")) return status;
    args.past_lengths = reinterpret_cast<const uint32_t *>(record.buffers[7].device);
    args.slot_offsets = reinterpret_cast<const uint32_t *>(record.buffers[8].device);
  }
  if (projecting && !q8_attention_can_project(args))
    return fail(LLMOPT_ERR_INVALID, "%s takes what the split-context kernels take (one query token, no mask, contexts of "
                "64 tokens and more in the launch) and a projection of at most 1024 rows", name);
  const size_t workspace_bytes = q8_attention_workspace_bytes(args);
  if (workspace_bytes > 0) {
    args.workspace = context_workspace(context, workspace_bytes);
    if (args.workspace == nullptr) return LLMOPT_ERR_FAILURE;
    args.workspace_bytes = workspace_bytes;
  }
  return launched(launch_q8_attention(args, context->stream), name);
}

int paged_attention_reference(llmopt_hip_context *context, const DispatchRecord &record) {
  return paged_attention(context, record, false);
}

int paged_attention_batched(llmopt_hip_context *context, const DispatchRecord &record) {
  return paged_attention(context, record, true);
}

int paged_attention_batched_projecting(llmopt_hip_context *context, const DispatchRecord &record) {
  return paged_attention(context, record, true, true);
}

// AttentionParams, 14 x 4 bytes (lib/metal_attention_source.ml:251-256,
// lib/metal_parameters.ml:95-117).  buffers: query, key, value, mask (the query
// buffer again when there is no mask, lib/metal_dispatch_attention.ml:52-54),
// output.
int dense_attention(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 5)) return status;
  if (int status = require_parameter_bytes(record, 56)) return status;
  DenseAttentionArgs args = {};
  args.batches = param_u32(record, 0);
  args.heads = param_u32(record, 4);
  args.query_length = param_u32(record, 8);
  args.key_length = param_u32(record, 12);
  args.head_dim = param_u32(record, 16);
  args.mask_batches = param_u32(record, 20);
  args.mask_heads = param_u32(record, 24);
  args.causal = param_u32(record, 28);
  args.scale = param_f32(record, 32);
  args.kv_heads = param_u32(record, 36);
  args.token_first_output = param_u32(record, 40);
  args.past_length = param_u32(record, 44);
  args.token_first_value = param_u32(record, 48);
  args.mask_dtype = param_u32(record, 52);
  const char *name = record.name.c_str();
  if (args.head_dim == 0 || args.head_dim > 512)
    return fail(LLMOPT_ERR_INVALID, "%s supports head dimensions 1..512, got %u", name, args.head_dim);
  const uint32_t kv_heads = args.kv_heads > 0 ? args.kv_heads : args.heads;
  if (kv_heads == 0 || (kv_heads < args.heads && args.heads % kv_heads != 0) || kv_heads > args.heads)
    return fail(LLMOPT_ERR_INVALID, "%s requires heads to be a multiple of kv_heads", name);
  if (args.mask_batches > 0 && (args.mask_heads == 0 || (args.mask_dtype != 1 && args.mask_dtype != 2)))
    return fail(LLMOPT_ERR_INVALID, "%s received an inconsistent mask description", name);
  if (args.mask_batches > 1 && args.mask_batches != args.batches)
    return fail(LLMOPT_ERR_INVALID, "%s mask batches must be 1 or the batch count", name);
  if (args.mask_batches > 0 && args.mask_heads > 1 && args.mask_heads != args.heads)
    return fail(LLMOPT_ERR_INVALID, "%s mask heads must be 1 or the head count", name);
  const uint64_t rows = (uint64_t)args.batches * args.heads * args.query_length;
  const uint64_t kv_elements = (uint64_t)args.batches * kv_heads * args.key_length * args.head_dim;
  if (rows != 0 && args.key_length == 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires at least one key", name);
  if (int status = require_buffer_size(record.buffers[0], rows * args.head_dim * 2, "attention query")) return status;
  if (int status = require_buffer_size(record.buffers[1], kv_elements * 2, "attention key")) return status;
  if (int status = require_buffer_size(record.buffers[2], kv_elements * 2, "attention value")) return status;
  if (args.mask_batches > 0) {
    const uint64_t mask_elements =
        (uint64_t)args.mask_batches * args.mask_heads * args.query_length * args.key_length;
    if (int status = require_buffer_size(record.buffers[3], mask_elements * (args.mask_dtype == 2 ? 2 : 1),
                                         "attention mask"))
      return status;
    args.mask = record.buffers[3].device;
  }
  if (int status = require_buffer_size(record.buffers[4], rows * args.head_dim * 2, "attention output")) return status;
  args.query = reinterpret_cast<const uint16_t *>(record.buffers[0].device);
  args.key = reinterpret_cast<const uint16_t *>(record.buffers[1].device);
  args.value = reinterpret_cast<const uint16_t *>(record.buffers[2].device);
  args.output = reinterpret_cast<uint16_t *>(record.buffers[4].device);
  const size_t map_bytes = dense_attention_workspace_bytes(args);
  if (map_bytes > 0) {
    args.stage_map = static_cast<uint8_t *>(context_workspace(context, map_bytes));
    if (args.stage_map == nullptr) return LLMOPT_ERR_FAILURE;
    args.stage_map_bytes = map_bytes;
  }
  return launched(launch_dense_attention(args, context->stream), name);
}

// llmopt_attention_tree_speculative_f16{,_simd_h64} (lib/metal_attention_source.ml:351-512, dispatch
// lib/metal_dispatch_attention.ml:219-245): dense attention of a few draft tokens over past_length
// cached keys and each other, who sees whom among the drafts given by eight bit masks.
// SpeculativeAttentionParams, 64 bytes: batches 0, heads 4, query_length 8, key_length 12,
// head_dimension 16, kv_heads 20, past_length 24, scale(f32) 28, tree_mask_0..7 at 32..60.
// buffers: query [b, h, q, D], key [b, kvh, L, D], value [b, L, kvh, D] (token-major), output
// [b, q, h, D] (token-major).  The masks are written out as a byte mask [q, L] in the context's
// scratch memory and the dense attention kernels run with it.
int speculative_attention(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 4)) return status;
  if (int status = require_parameter_bytes(record, 64)) return status;
  const char *name = record.name.c_str();
  DenseAttentionArgs args = {};
  args.batches = param_u32(record, 0);
  args.heads = param_u32(record, 4);
  args.query_length = param_u32(record, 8);
  args.key_length = param_u32(record, 12);
  args.head_dim = param_u32(record, 16);
  args.kv_heads = param_u32(record, 20);
  const uint32_t past_length = param_u32(record, 24);
  args.scale = param_f32(record, 28);
  uint32_t tree_masks[8];
  for (int i = 0; i < 8; ++i) tree_masks[i] = param_u32(record, 32 + 4 * i);
  if (args.head_dim == 0 || args.head_dim > 512)
    return fail(LLMOPT_ERR_INVALID, "%s supports head dimensions 1..512, got %u", name, args.head_dim);
  const uint32_t kv_heads = args.kv_heads > 0 ? args.kv_heads : args.heads;
  if (kv_heads == 0 || (kv_heads < args.heads && args.heads % kv_heads != 0) || kv_heads > args.heads)
    return fail(LLMOPT_ERR_INVALID, "%s requires heads to be a multiple of kv_heads", name);
  const uint64_t rows = (uint64_t)args.batches * args.heads * args.query_length;
  if (rows != 0 && args.key_length == 0) return fail(LLMOPT_ERR_INVALID, "%s requires at least one key", name);
  const uint64_t kv_elements = (uint64_t)args.batches * kv_heads * args.key_length * args.head_dim;
  if (int status = require_buffer_size(record.buffers[0], rows * args.head_dim * 2, "attention query")) return status;
  if (int status = require_buffer_size(record.buffers[1], kv_elements * 2, "attention key")) return status;
  if (int status = require_buffer_size(record.buffers[2], kv_elements * 2, "attention value")) return status;
  if (int status = require_buffer_size(record.buffers[3], rows * args.head_dim * 2, "attention output")) return status;
  if (rows == 0) return LLMOPT_OK;
  args.query = reinterpret_cast<const uint16_t *>(record.buffers[0].device);
  args.key = reinterpret_cast<const uint16_t *>(record.buffers[1].device);
  args.value = reinterpret_cast<const uint16_t *>(record.buffers[2].device);
  args.output = reinterpret_cast<uint16_t *>(record.buffers[3].device);
  args.mask_batches = 1, args.mask_heads = 1, args.mask_dtype = 1, args.causal = 0;
  args.token_first_output = 1, args.token_first_value = 1;
  const size_t mask_bytes = ((size_t)args.query_length * args.key_length + 255) & ~(size_t)255;
  // the dense kernels' own scratch is sized for any 16-byte aligned mask address
  args.mask = reinterpret_cast<const uint8_t *>((uintptr_t)4096);
  const size_t map_bytes = dense_attention_workspace_bytes(args);
  uint8_t *scratch = static_cast<uint8_t *>(context_workspace(context, mask_bytes + map_bytes));
  if (scratch == nullptr) return LLMOPT_ERR_FAILURE;
  args.mask = scratch;
  if (map_bytes > 0) {
    args.stage_map = scratch + mask_bytes;
    args.stage_map_bytes = map_bytes;
  }
  if (int status = launched(launch_tree_mask(scratch, args.query_length, args.key_length, past_length, tree_masks,
                                             context->stream), name))
    return status;
  return launched(launch_dense_attention(args, context->stream), name);
}

}  // namespace

void register_cache_kernels(std::vector<KernelEntryPoint> &table) {
  static const char *const cache = "cache";
  table.push_back({"llmopt_cache_pack_attention_q8", cache, cache_pack});
  table.push_back({"llmopt_cache_pack_attention_q8_simd", cache, cache_pack});
  table.push_back({"llmopt_cache_pack_attention_q8_pair_simd", cache, cache_pack_pair});
  table.push_back({"llmopt_cache_pack_attention_q8_pair_batched", cache, cache_pack_pair_batched});
  table.push_back({"llmopt_rotary_qk_pack_q8_batched", cache, rotary_qk_pack_batched});
  table.push_back({"llmopt_cache_unpack_attention_q8", cache, cache_unpack});
  table.push_back({"llmopt_cache_unpack_attention_q8_vec4", cache, cache_unpack});
  table.push_back({"llmopt_cache_pack_checkpoint_q8", cache, cache_pack_checkpoint});
  table.push_back({"llmopt_cache_pack_checkpoint_q8_simd", cache, cache_pack_checkpoint});
  table.push_back({"llmopt_cache_unpack_checkpoint_q8", cache, cache_unpack_checkpoint});
  table.push_back({"llmopt_cache_unpack_checkpoint_q8_vec4", cache, cache_unpack_checkpoint});
}

void register_attention_kernels(std::vector<KernelEntryPoint> &table) {
  static const char *const attention = "attention";
  static const char *const names[] = {
      "llmopt_attention_q8_paged_simd_generic",   "llmopt_attention_q8_paged_simd_h64",
      "llmopt_attention_q8_paged_simd_h64_gqa3",  "llmopt_attention_q8_paged_simd_h256",
      "llmopt_attention_q8_paged_simd_h512",      "llmopt_attention_q8_paged_simd_h64_split8",
      "llmopt_attention_q8_paged_simd_h64_gqa3_split8"};
  for (const char *name : names) table.push_back({name, attention, paged_attention_reference});
  // dense fp16 attention: the portable entry and the per-head-dimension ones
  // the reference generates on demand (lib/metal_dispatch_common.ml:166-189)
  static const char *const dense[] = {"llmopt_attention_f16",           "llmopt_attention_f16_simd_h64",
                                      "llmopt_attention_f16_simd_h128", "llmopt_attention_f16_simd_h256",
                                      "llmopt_attention_f16_simd_h512"};
  for (const char *name : dense) table.push_back({name, attention, dense_attention});
  table.push_back({"llmopt_attention_tree_speculative_f16", attention, speculative_attention});
  table.push_back({"llmopt_attention_tree_speculative_f16_simd_h64", attention, speculative_attention});
  // Extension: per-sequence context lengths and slot tables in one launch.
  table.push_back({"llmopt_attention_q8_paged_batched", attention, paged_attention_batched});
  // Extension: the same with every head's output row multiplied into its columns of a W4 output projection.
  table.push_back({"llmopt_attention_q8_paged_batched_w4a16_partial_g64", attention, paged_attention_batched_projecting});
}

}  // namespace llmopt
