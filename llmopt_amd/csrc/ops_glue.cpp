// Entry points of the decode-step glue kernels: RMSNorm, rotate-half RoPE,
// fp16 embedding, fp16 add, the RMSNorm stage of the SwiGLU FFN macro-op and
// the LM-head argmax family.  Buffer order and parameter blocks follow the
// reference kernels (lib/metal_normalization_source.ml:70-91,765-802,
// lib/metal_tensor_source.ml:306-320,1007-1032, lib/metal_w4a16_source.ml:496-526,
// 1006-1378; host side lib/metal_dispatch_linear.ml:570-721).
#include <cmath>
#include <cstring>

#include "kernels/kernels.h"
#include "kernels/kernels_internal.h"
#include "runtime.h"

namespace llmopt {

// The first 28 parameter bytes and the first 6 buffers of a rotary record, checked.
int parse_rotary_qk(const DispatchRecord &record, RotaryQkArgs *out) {
  RotaryQkArgs args = {};
  args.batches = param_u32(record, 0);
  args.tokens = param_u32(record, 4);
  args.q_heads = param_u32(record, 8);
  args.k_heads = param_u32(record, 12);
  args.width = param_u32(record, 16);
  args.half_dimension = param_u32(record, 20);
  args.trig_batches = param_u32(record, 24);
  if (args.batches == 0 || args.tokens == 0 || args.width == 0 || args.q_heads + args.k_heads == 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires positive batches, tokens, heads and width", record.name.c_str());
  if (args.half_dimension * 2 != args.width)
    return fail(LLMOPT_ERR_INVALID, "%s requires half_dimension = width / 2", record.name.c_str());
  if (args.trig_batches != 1 && args.trig_batches != args.batches)
    return fail(LLMOPT_ERR_INVALID, "%s requires trig_batches to be 1 or batches", record.name.c_str());
  const uint64_t token_rows = (uint64_t)args.batches * args.tokens;
  const uint64_t q_bytes = token_rows * args.q_heads * args.width * 2;
  const uint64_t k_bytes = token_rows * args.k_heads * args.width * 2;
  const uint64_t trig_bytes = (uint64_t)args.trig_batches * args.tokens * args.width * 2;
  if (int status = require_buffer_size(record.buffers[0], q_bytes, "q input")) return status;
  if (int status = require_buffer_size(record.buffers[1], k_bytes, "k input")) return status;
  if (int status = require_buffer_size(record.buffers[2], trig_bytes, "cosine")) return status;
  if (int status = require_buffer_size(record.buffers[3], trig_bytes, "sine")) return status;
  if (int status = require_buffer_size(record.buffers[4], q_bytes, "q output")) return status;
  if (int status = require_buffer_size(record.buffers[5], k_bytes, "k output")) return status;
  args.q_input = reinterpret_cast<const uint16_t *>(record.buffers[0].device);
  args.k_input = reinterpret_cast<const uint16_t *>(record.buffers[1].device);
  args.cosine = reinterpret_cast<const uint16_t *>(record.buffers[2].device);
  args.sine = reinterpret_cast<const uint16_t *>(record.buffers[3].device);
  args.q_output = reinterpret_cast<uint16_t *>(record.buffers[4].device);
  args.k_output = reinterpret_cast<uint16_t *>(record.buffers[5].device);
  *out = args;
  return LLMOPT_OK;
}

namespace {

const uint16_t *as_f16(const BoundBuffer &buffer) {
  return reinterpret_cast<const uint16_t *>(buffer.device);
}
uint16_t *as_f16_out(const BoundBuffer &buffer) { return reinterpret_cast<uint16_t *>(buffer.device); }

int launched(hipError_t status, const char *name) {
  if (status != hipSuccess) return fail(LLMOPT_ERR_FAILURE, "%s launch failed: %s", name, hipGetErrorString(status));
  return LLMOPT_OK;
}

bool valid_epsilon(float epsilon) { return std::isfinite(epsilon) && epsilon > 0.0f; }

// RmsNormParams {u32 rows, width; f32 epsilon}; buffers: input, weight, output.
int rms_norm_f16(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (int status = require_parameter_bytes(record, 12)) return status;
  const uint32_t rows = param_u32(record, 0), width = param_u32(record, 4);
  const float epsilon = param_f32(record, 8);
  if (rows == 0 || width == 0) return fail(LLMOPT_ERR_INVALID, "%s requires positive rows and width", record.name.c_str());
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)rows * width * 2, "input")) return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)width * 2, "weight")) return status;
  if (int status = require_buffer_size(record.buffers[2], (uint64_t)rows * width * 2, "output")) return status;
  RmsNormArgs args = {};
  args.input = record.buffers[0].device;
  args.input_f32 = false;
  args.weight = as_f16(record.buffers[1]);
  args.output = as_f16_out(record.buffers[2]);
  args.rows = rows;
  args.width = width;
  args.epsilon = epsilon;
  args.weight_first = false;
  return launched(launch_rms_norm(args, context->stream), record.name.c_str());
}

// W4A16SwiGLUFFNParams {u32 m, n, k; f32 epsilon}; buffers: input (f16 or f32), norm_weight, normalized.
template <bool F32>
int swiglu_rms(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (int status = require_parameter_bytes(record, 16)) return status;
  const uint32_t m = param_u32(record, 0), k = param_u32(record, 8);
  const float epsilon = param_f32(record, 12);
  if (m == 0 || k == 0) return fail(LLMOPT_ERR_INVALID, "%s requires positive m and k", record.name.c_str());
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * k * (F32 ? 4 : 2), "input")) return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)k * 2, "norm weight")) return status;
  if (int status = require_buffer_size(record.buffers[2], (uint64_t)m * k * 2, "normalized")) return status;
  RmsNormArgs args = {};
  args.input = record.buffers[0].device;
  args.input_f32 = F32;
  args.weight = as_f16(record.buffers[1]);
  args.output = as_f16_out(record.buffers[2]);
  args.rows = m;
  args.width = k;
  args.epsilon = epsilon;
  args.weight_first = true;
  return launched(launch_rms_norm(args, context->stream), record.name.c_str());
}

// RotaryQKParams {u32 batches, tokens, q_heads, k_heads, width, half_dimension, trig_batches};
// buffers: q_input, k_input, cosine, sine, q_output, k_output.
int rotary_qk(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 6)) return status;
  if (int status = require_parameter_bytes(record, 28)) return status;
  RotaryQkArgs args = {};
  if (int status = parse_rotary_qk(record, &args)) return status;
  return launched(launch_rotary_qk(args, context->stream), record.name.c_str());
}

// EmbeddingParams {u32 tokens, vocabulary, width}; buffers: indices (i64), weight, output.
int embedding_f16(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (int status = require_parameter_bytes(record, 12)) return status;
  EmbeddingArgs args = {};
  args.tokens = param_u32(record, 0);
  args.vocabulary = param_u32(record, 4);
  args.width = param_u32(record, 8);
  if (args.tokens == 0 || args.width == 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires positive tokens and width", record.name.c_str());
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)args.tokens * 8, "indices")) return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)args.vocabulary * args.width * 2, "weight"))
    return status;
  if (int status = require_buffer_size(record.buffers[2], (uint64_t)args.tokens * args.width * 2, "output"))
    return status;
  args.indices = reinterpret_cast<const int64_t *>(record.buffers[0].device);
  args.weight = as_f16(record.buffers[1]);
  args.output = as_f16_out(record.buffers[2]);
  return launched(launch_embedding(args, context->stream), record.name.c_str());
}

// PointwiseParams (136 bytes, lib/metal_parameters.ml:350-380); buffers: left, right, output.
int add_f16(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (int status = require_parameter_bytes(record, 136)) return status;
  PointwiseArgs args = {};
  args.count = param_u32(record, 0);
  args.rank = param_u32(record, 4);
  args.left_scalar = param_u32(record, 8);
  args.right_scalar = param_u32(record, 12);
  if (args.rank > 8) return fail(LLMOPT_ERR_INVALID, "%s supports rank at most eight", record.name.c_str());
  uint64_t out_count = 1, left_count = 1, right_count = 1;
  for (uint32_t axis = 0; axis < 8; ++axis) {
    args.output_shape[axis] = param_u32(record, 16 + 4 * axis);
    args.left_shape[axis] = param_u32(record, 48 + 4 * axis);
    args.right_shape[axis] = param_u32(record, 80 + 4 * axis);
    if (axis < args.rank) {
      const uint32_t o = args.output_shape[axis], l = args.left_shape[axis], r = args.right_shape[axis];
      if (o == 0 || (l != 1 && l != o) || (r != 1 && r != o))
        return fail(LLMOPT_ERR_INVALID, "%s input shape is not broadcastable to output", record.name.c_str());
      out_count *= o;
      left_count *= l;
      right_count *= r;
    }
  }
  if (out_count != args.count)
    return fail(LLMOPT_ERR_INVALID, "%s count does not match the output shape", record.name.c_str());
  args.left_f32 = param_f32(record, 128);
  args.right_f32 = param_f32(record, 132);
  if (args.count == 0) return LLMOPT_OK;
  if (!args.left_scalar)
    if (int status = require_buffer_size(record.buffers[0], left_count * 2, "left")) return status;
  if (!args.right_scalar)
    if (int status = require_buffer_size(record.buffers[1], right_count * 2, "right")) return status;
  if (int status = require_buffer_size(record.buffers[2], out_count * 2, "output")) return status;
  args.left = as_f16(record.buffers[0]);
  args.right = as_f16(record.buffers[1]);
  args.output = as_f16_out(record.buffers[2]);
  return launched(launch_add_f16(args, context->stream), record.name.c_str());
}

// ---- LM head ------------------------------------------------------------------
//
// RMSNorm, vocabulary GEMV with float32 logits, argmax with ties to the lowest
// index.  The reference keeps the normalised activation in float32
// (lib/metal_w4a16_source.ml:1038-1046); the GEMV kernels take fp16 rows, so the
// float32 value travels as a hi and a lo fp16 row (2^-22 relative together) and
// the two float32 products are added in the argmax kernel.
//
// W4A16LmHeadParams {u32 m, n, k; f32 epsilon}.
// Buffers: input, norm_weight, weight, scale, result [, logits f16 [m, n]]
// where result is token_ids (u32 [m]) or, for the stage1 entries, the
// candidate array (256 x {f32, u32} per row).
struct LmHeadVariant {
  bool input_f32, extra, stage1;
};

size_t round_up_256(size_t bytes) { return (bytes + 255) & ~(size_t)255; }

int lm_head(llmopt_hip_context *context, const DispatchRecord &record, LmHeadVariant variant) {
  const char *name = record.name.c_str();
  if (int status = require_buffer_count(record, variant.extra ? 6 : 5)) return status;
  if (int status = require_parameter_bytes(record, 16)) return status;
  const uint32_t m = param_u32(record, 0), n = param_u32(record, 4), k = param_u32(record, 8);
  const float epsilon = param_f32(record, 12);
  if (m == 0 || n == 0 || k == 0 || k % 64 != 0 || !valid_epsilon(epsilon))
    return fail(LLMOPT_ERR_INVALID, "%s input metadata is inconsistent", name);
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * k * (variant.input_f32 ? 4 : 2), "input"))
    return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)k * 2, "norm weight")) return status;
  if (int status = require_buffer_size(record.buffers[2], (uint64_t)n * (k / 2), "packed weight")) return status;
  if (int status = require_buffer_size(record.buffers[3], (uint64_t)n * (k / 64) * 2, "scale")) return status;
  const uint64_t result_bytes = variant.stage1 ? (uint64_t)m * 256 * 8 : (uint64_t)m * 4;
  if (int status = require_buffer_size(record.buffers[4], result_bytes, variant.stage1 ? "candidates" : "token ids"))
    return status;
  if (variant.extra)
    if (int status = require_buffer_size(record.buffers[5], (uint64_t)m * n * 2, "logits")) return status;

  // workspace: normalised activation (hi and lo row per input row) | float32 partial logits
  // [2m, n] | candidates | GEMV scratch
  const uint32_t gemv_rows = 2 * m;
  const size_t normalized_bytes = round_up_256((size_t)gemv_rows * k * 2);
  const size_t logits_bytes = round_up_256((size_t)gemv_rows * n * 4);
  const size_t candidate_bytes = round_up_256((size_t)m * 256 * 8);
  const size_t gemv_bytes = w4a16_gemv_workspace_bytes(std::min(gemv_rows, kGemvMaxRows), n, k);
  uint8_t *workspace = static_cast<uint8_t *>(
      context_workspace(context, normalized_bytes + logits_bytes + candidate_bytes + gemv_bytes));
  if (workspace == nullptr) return LLMOPT_ERR_FAILURE;
  uint16_t *normalized = reinterpret_cast<uint16_t *>(workspace);
  float *logits = reinterpret_cast<float *>(workspace + normalized_bytes);
  void *candidates = variant.stage1 ? static_cast<void *>(record.buffers[4].device)
                                    : static_cast<void *>(workspace + normalized_bytes + logits_bytes);

  // input * weight * inverse (lib/metal_w4a16_source.ml:1043-1044) stays float32 there; here it
  // goes through the fp16 GEMV as a hi and a lo row, whose float32 products are added again
  RmsNormArgs norm = {};
  norm.input = record.buffers[0].device;
  norm.input_f32 = variant.input_f32;
  norm.weight = as_f16(record.buffers[1]);
  norm.output = normalized;
  norm.rows = m;
  norm.width = k;
  norm.epsilon = epsilon;
  if (int status = launched(launch_rms_norm_split(norm, context->stream), name)) return status;

  // the decode GEMV keeps float32 results; more rows go through it in groups: of eight a launch, or - when one
  // workgroup covers K, so that nothing is handed over between workgroups - up to 128 rows a launch as row groups
  // of one grid (the 64 rows of 32 sequences at 49152 x 576: one launch instead of eight)
  const uint32_t rows_per_launch = w4a16_gemv_mfma_needs_split(k) ? kGemvMaxRows : 128;
  for (uint32_t first = 0; first < gemv_rows; first += rows_per_launch) {
    const uint32_t rows = std::min(rows_per_launch, gemv_rows - first);
    W4LinearArgs linear = {};
    linear.x = normalized + (size_t)first * k;
    linear.w = {record.buffers[2].device, as_f16(record.buffers[3])};
    linear.y = nullptr;
    linear.y_f32 = logits + (size_t)first * n;
    linear.m = rows;
    linear.n = n;
    linear.k = k;
    if (gemv_bytes > 0) {
      linear.workspace = workspace + normalized_bytes + logits_bytes + candidate_bytes;
      linear.workspace_bytes = gemv_bytes;
      linear.counters = context_counters(context, &linear.counter_count);
      if (linear.counters == nullptr) return LLMOPT_ERR_FAILURE;
    }
    if (int status = launched(rows > kGemvMaxRows ? launch_w4a16_gemv_mfma_linear(linear, context->stream)
                                                  : launch_w4a16_linear(linear, context->stream),
                              name))
      return status;
  }
  uint16_t *half_logits = variant.extra ? as_f16_out(record.buffers[5]) : nullptr;
  if (int status = launched(launch_argmax_candidates(logits, candidates, m, n, true, half_logits, context->stream),
                            name))
    return status;
  if (variant.stage1) return LLMOPT_OK;
  return launched(launch_argmax_reduce(candidates, reinterpret_cast<uint32_t *>(record.buffers[4].device), m,
                                       context->stream),
                  name);
}

template <bool F32, bool EXTRA, bool STAGE1>
int lm_head_entry(llmopt_hip_context *context, const DispatchRecord &record) {
  return lm_head(context, record, {F32, EXTRA, STAGE1});
}

// buffers: candidates, token_ids; parameters {u32 m}.
int lm_head_reduce(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 2)) return status;
  if (int status = require_parameter_bytes(record, 4)) return status;
  const uint32_t m = param_u32(record, 0);
  if (m == 0) return fail(LLMOPT_ERR_INVALID, "%s requires positive m", record.name.c_str());
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * 256 * 8, "candidates")) return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)m * 4, "token ids")) return status;
  return launched(launch_argmax_reduce(record.buffers[0].device,
                                       reinterpret_cast<uint32_t *>(record.buffers[1].device), m, context->stream),
                  record.name.c_str());
}

}  // namespace

void register_glue_kernels(std::vector<KernelEntryPoint> &table) {
  static const char *const ffn = "w4a16-swiglu-ffn-g64";
  static const char *const head = "w4a16-lm-head-argmax";
  table.push_back({"llmopt_rms_norm_f16_simd", "rms-norm", rms_norm_f16});
  table.push_back({"llmopt_rotary_qk_f16_simd_h64", "rotary-qk", rotary_qk});
  table.push_back({"llmopt_embedding_f16", "embedding", embedding_f16});
  table.push_back({"llmopt_add_f16", "pointwise", add_f16});
  table.push_back({"llmopt_w4a16_swiglu_rms_f16_g64", ffn, swiglu_rms<false>});
  table.push_back({"llmopt_w4a16_swiglu_rms_f32_g64", ffn, swiglu_rms<true>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_f16", head, lm_head_entry<false, false, false>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_f32", head, lm_head_entry<true, false, false>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_extra_f16", head, lm_head_entry<false, true, false>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_extra_f32", head, lm_head_entry<true, true, false>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_stage1_f16", head, lm_head_entry<false, false, true>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_stage1_f32", head, lm_head_entry<true, false, true>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_stage1_extra_f16", head, lm_head_entry<false, true, true>});
  table.push_back({"llmopt_w4a16_lm_head_argmax_stage1_extra_f32", head, lm_head_entry<true, true, true>});
  table.push_back({"llmopt_w4a16_lm_head_reduce", head, lm_head_reduce});
}

}  // namespace llmopt
