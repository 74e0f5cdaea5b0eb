// Entry points of the W4A16 linear family: buffer order, parameter-block
// layout and size checks of the reference's kernels
// (lib/metal_w4a16_source.ml; host side lib/metal_dispatch_linear.ml:252-455,
// 938-982), bound to the gfx950 launchers.
#include <cmath>

#include "kernels/kernels.h"
#include "runtime.h"

namespace llmopt {
namespace {

const uint16_t *as_f16(const BoundBuffer &buffer) {
  return reinterpret_cast<const uint16_t *>(buffer.device);
}

int check_w4_shape(const char *name, uint32_t m, uint32_t n, uint32_t k) {
  if (m == 0 || n == 0 || k == 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires positive m, n and k", name);
  if (k % 64 != 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires k to be a multiple of the group size 64, got %u",
                name, k);
  return LLMOPT_OK;
}

int check_w4_matrix(const BoundBuffer &weight, const BoundBuffer &scale, uint64_t n, uint64_t k,
                    const char *label) {
  std::string weight_name = std::string(label) + " packed weight";
  std::string scale_name = std::string(label) + " scale";
  if (int status = require_buffer_size(weight, n * (k / 2), weight_name.c_str())) return status;
  return require_buffer_size(scale, n * (k / 64) * 2, scale_name.c_str());
}

int launched(hipError_t status, const char *name) {
  if (status != hipSuccess) return fail(LLMOPT_ERR_FAILURE, "%s launch failed: %s", name, hipGetErrorString(status));
  return LLMOPT_OK;
}

// Scratch for the decode path when it splits K over workgroups (m x k beyond
// the LDS budget); none is needed for most shapes.
int attach_linear_scratch(llmopt_hip_context *context, W4LinearArgs *args) {
  const size_t bytes = args->m > kGemvMaxRows ? w4a16_gemm_workspace_bytes(args->m, args->n, args->k)
                                              : w4a16_gemv_workspace_bytes(args->m, args->n, args->k);
  if (bytes == 0) return LLMOPT_OK;
  args->workspace = context_workspace(context, bytes);
  if (args->workspace == nullptr) return LLMOPT_ERR_FAILURE;
  args->workspace_bytes = bytes;
  args->counters = context_counters(context, &args->counter_count);
  if (args->counters == nullptr) return LLMOPT_ERR_FAILURE;
  return LLMOPT_OK;
}

// W4A16Params {u32 m, n, k, has_bias, bias_row_stride}  (lib/metal_w4a16_source.ml:7)
// buffers: input, packed_weight, scale, bias_or_scale, output.
int w4a16_linear(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 5)) return status;
  if (int status = require_parameter_bytes(record, 20)) return status;
  const uint32_t m = param_u32(record, 0), n = param_u32(record, 4), k = param_u32(record, 8);
  const uint32_t has_bias = param_u32(record, 12), stride = param_u32(record, 16);
  if (int status = check_w4_shape(record.name.c_str(), m, n, k)) return status;
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * k * 2, "input")) return status;
  if (int status = check_w4_matrix(record.buffers[1], record.buffers[2], n, k, "W4A16")) return status;
  if (has_bias) {
    const uint64_t last = (uint64_t)(m - 1) * stride + n;
    if (int status = require_buffer_size(record.buffers[3], last * 2, "bias")) return status;
  }
  if (int status = require_buffer_size(record.buffers[4], (uint64_t)m * n * 2, "output")) return status;
  W4LinearArgs args = {};
  args.x = as_f16(record.buffers[0]);
  args.w = {record.buffers[1].device, as_f16(record.buffers[2])};
  args.addend = as_f16(record.buffers[3]);
  args.has_addend = has_bias;
  args.addend_row_stride = stride;
  args.y = reinterpret_cast<uint16_t *>(record.buffers[4].device);
  args.m = m;
  args.n = n;
  args.k = k;
  if (int status = attach_linear_scratch(context, &args)) return status;
  return launched(launch_w4a16_linear(args, context->stream), record.name.c_str());
}

// The activation of a normalising entry: either the kernel normalises (*norm is set and *x stays
// the raw input) or the rows are normalised into the context's scratch here (*x moves there).
int normalise_input(llmopt_hip_context *context, const DispatchRecord &record, const W4Norm &wanted, uint32_t m,
                    uint32_t k, uint64_t columns, const uint16_t **x, W4Norm *norm) {
  if (!std::isfinite(wanted.epsilon) || wanted.epsilon <= 0.0f)
    return fail(LLMOPT_ERR_INVALID, "%s requires a positive finite epsilon", record.name.c_str());
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)k * 2, "norm weight")) return status;
  const bool aligned = ((reinterpret_cast<uintptr_t>(*x) | reinterpret_cast<uintptr_t>(wanted.weight)) & 15) == 0;
  if (aligned && w4a16_norm_in_kernel(m, columns, k)) {
    *norm = wanted;
    return LLMOPT_OK;
  }
  uint16_t *scratch = static_cast<uint16_t *>(context_workspace(context, (size_t)m * k * 2));
  if (scratch == nullptr) return LLMOPT_ERR_FAILURE;
  RmsNormArgs args = {};
  args.input = *x;
  args.weight = wanted.weight;
  args.output = scratch;
  args.rows = m;
  args.width = k;
  args.epsilon = wanted.epsilon;
  args.weight_first = wanted.weight_first != 0;
  if (int status = launched(launch_rms_norm(args, context->stream), record.name.c_str())) return status;
  *x = scratch;
  return LLMOPT_OK;
}

// W4A16QKVParams {u32 m, k, n_q, n_k, n_v}  (lib/metal_w4a16_source.ml:211-217)
// buffers: input, qW, qS, kW, kS, vW, vS, qOut, kOut, vOut.
// With `normalised` the record is the extension llmopt_rms_w4a16_qkv_linear_f16_g64: the norm
// weight follows the input in the buffer list and f32 epsilon the five words.
int qkv_linear(llmopt_hip_context *context, const DispatchRecord &record, bool normalised) {
  const size_t b = normalised ? 1 : 0;  // buffers after the input move up by one
  if (int status = require_buffer_count(record, 10 + b)) return status;
  if (int status = require_parameter_bytes(record, normalised ? 24 : 20)) return status;
  const uint32_t m = param_u32(record, 0), k = param_u32(record, 4);
  const uint32_t n[3] = {param_u32(record, 8), param_u32(record, 12), param_u32(record, 16)};
  W4QkvArgs args = {};
  static const char *const labels[3] = {"query", "key", "value"};
  for (int i = 0; i < 3; ++i) {
    if (int status = check_w4_shape(record.name.c_str(), m, n[i], k)) return status;
    if (int status =
            check_w4_matrix(record.buffers[b + 1 + 2 * i], record.buffers[b + 2 + 2 * i], n[i], k, labels[i]))
      return status;
    if (int status = require_buffer_size(record.buffers[b + 7 + i], (uint64_t)m * n[i] * 2, "output")) return status;
    args.w[i] = {record.buffers[b + 1 + 2 * i].device, as_f16(record.buffers[b + 2 + 2 * i])};
    args.y[i] = reinterpret_cast<uint16_t *>(record.buffers[b + 7 + i].device);
    args.n[i] = n[i];
  }
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * k * 2, "input")) return status;
  args.x = as_f16(record.buffers[0]);
  args.m = m;
  args.k = k;
  if (normalised) {
    const W4Norm norm = {as_f16(record.buffers[1]), param_f32(record, 20), 0};  // llmopt_rms_norm_f16_simd's order
    if (int status = normalise_input(context, record, norm, m, k, (uint64_t)n[0] + n[1] + n[2], &args.x, &args.norm))
      return status;
  }
  return launched(launch_w4a16_qkv(args, context->stream), record.name.c_str());
}

int w4a16_qkv_linear(llmopt_hip_context *context, const DispatchRecord &record) {
  return qkv_linear(context, record, false);
}

// Extension (no reference kernel): llmopt_rms_norm_f16_simd followed by llmopt_w4a16_qkv_linear_f16_g64
// without the normalised rows passing through memory where the projection kernel can normalise
// them itself, else as those two launches.  buffers: input, norm weight, qW, qS, kW, kS, vW, vS,
// qOut, kOut, vOut; parameters W4A16QKVParams + f32 epsilon.
int rms_w4a16_qkv_linear(llmopt_hip_context *context, const DispatchRecord &record) {
  return qkv_linear(context, record, true);
}

// W4A16SwiGLUFFNParams {u32 m, n, k; f32 eps}: n = intermediate width, k = hidden width
// (lib/metal_parameters.ml:45-50).  buffers: normalized, gateW, gateS, upW, upS, product.
int dual_swiglu(llmopt_hip_context *context, const DispatchRecord &record, bool normalised) {
  const size_t b = normalised ? 1 : 0;
  if (int status = require_buffer_count(record, 6 + b)) return status;
  if (int status = require_parameter_bytes(record, 16)) return status;
  const uint32_t m = param_u32(record, 0), n = param_u32(record, 4), k = param_u32(record, 8);
  if (int status = check_w4_shape(record.name.c_str(), m, n, k)) return status;
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * k * 2, normalised ? "input" : "normalized"))
    return status;
  if (int status = check_w4_matrix(record.buffers[b + 1], record.buffers[b + 2], n, k, "gate")) return status;
  if (int status = check_w4_matrix(record.buffers[b + 3], record.buffers[b + 4], n, k, "up")) return status;
  if (int status = require_buffer_size(record.buffers[b + 5], (uint64_t)m * n * 2, "product")) return status;
  W4DualSwigluArgs args = {};
  args.x = as_f16(record.buffers[0]);
  args.gate = {record.buffers[b + 1].device, as_f16(record.buffers[b + 2])};
  args.up = {record.buffers[b + 3].device, as_f16(record.buffers[b + 4])};
  args.product = reinterpret_cast<uint16_t *>(record.buffers[b + 5].device);
  args.m = m;
  args.n = n;
  args.k = k;
  if (normalised) {
    const W4Norm norm = {as_f16(record.buffers[1]), param_f32(record, 12), 1};  // llmopt_w4a16_swiglu_rms_f16_g64's order
    if (int status = normalise_input(context, record, norm, m, k, 2ull * n, &args.x, &args.norm)) return status;
  }
  return launched(launch_w4a16_dual_swiglu(args, context->stream), record.name.c_str());
}

int w4a16_dual_swiglu(llmopt_hip_context *context, const DispatchRecord &record) {
  return dual_swiglu(context, record, false);
}

// Extension (no reference kernel): llmopt_w4a16_swiglu_rms_f16_g64 followed by
// llmopt_w4a16_dual_swiglu_f16_g64, as above.  buffers: input, norm weight, gateW, gateS, upW, upS,
// product; parameters W4A16SwiGLUFFNParams.
int rms_w4a16_dual_swiglu(llmopt_hip_context *context, const DispatchRecord &record) {
  return dual_swiglu(context, record, true);
}

// Same parameter block; the contraction runs over n and the output has k
// columns: output[m,k] = half(product[m,n] . downW[k,n/2]^T + residual[m,k]).
// buffers: product, downW, downS, residual, output.
int w4a16_down_add(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 5)) return status;
  if (int status = require_parameter_bytes(record, 16)) return status;
  const uint32_t m = param_u32(record, 0), n = param_u32(record, 4), k = param_u32(record, 8);
  if (int status = check_w4_shape(record.name.c_str(), m, k, n)) return status;
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * n * 2, "product")) return status;
  if (int status = check_w4_matrix(record.buffers[1], record.buffers[2], k, n, "down")) return status;
  if (int status = require_buffer_size(record.buffers[3], (uint64_t)m * k * 2, "residual")) return status;
  if (int status = require_buffer_size(record.buffers[4], (uint64_t)m * k * 2, "output")) return status;
  W4LinearArgs args = {};
  args.x = as_f16(record.buffers[0]);
  args.w = {record.buffers[1].device, as_f16(record.buffers[2])};
  args.addend = as_f16(record.buffers[3]);
  args.has_addend = 1;
  args.addend_row_stride = k;
  args.y = reinterpret_cast<uint16_t *>(record.buffers[4].device);
  args.m = m;
  args.n = k;
  args.k = n;
  if (int status = attach_linear_scratch(context, &args)) return status;
  return launched(launch_w4a16_linear(args, context->stream), record.name.c_str());
}

// Extension (no reference kernel): one new token per sequence through llmopt_rms_norm_f16_simd,
// llmopt_w4a16_qkv_linear_f16_g64, llmopt_rotary_qk_f16_simd_h64 and
// llmopt_cache_pack_attention_q8_pair_simd as ONE launch, heads of 64.  The residual stream comes in as
// `input` plus `partial_count` pending partial sums of the previous layer's down projection
// (llmopt_rms_w4a16_swiglu_down_partial_f16_g64), and is written out whole to `stream`.
// buffers: input f16 [m,k], partials f32 [partial_count,m,k] (any buffer when partial_count = 0),
// stream f16 [m,k], norm weight, qW, qS, kW, kS, vW, vS, trig f16 [2,m,64] (cosine rows, then sine rows),
// qOut f16 [m,n_q] (rotated), kOut f16 [m,n_k] (rotated), vOut f16 [m,n_v], slots u32 [m], pool.
// parameters: u32 m, k, n_q, n_k, n_v; f32 epsilon; u32 partial_count, key_offset, value_offset,
// token_elements, token_stride.
int rms_w4a16_qkv_rotary_pack(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 16)) return status;
  if (int status = require_parameter_bytes(record, 44)) return status;
  const char *name = record.name.c_str();
  FusedQkvArgs args = {};
  args.m = param_u32(record, 0);
  args.k = param_u32(record, 4);
  args.norm = {as_f16(record.buffers[3]), param_f32(record, 20), 0};
  args.in.partial_count = param_u32(record, 24);
  args.key_offset = param_u32(record, 28);
  args.value_offset = param_u32(record, 32);
  args.token_elements = param_u32(record, 36);
  args.token_stride = param_u32(record, 40);
  static const char *const labels[3] = {"query", "key", "value"};
  for (int i = 0; i < 3; ++i) {
    args.n[i] = param_u32(record, 8 + 4 * i);
    if (int status = check_w4_shape(name, args.m, args.n[i], args.k)) return status;
    if (args.n[i] % 64 != 0) return fail(LLMOPT_ERR_INVALID, "%s requires whole heads of 64 columns, got %u", name, args.n[i]);
    if (int status = check_w4_matrix(record.buffers[4 + 2 * i], record.buffers[5 + 2 * i], args.n[i], args.k, labels[i]))
      return status;
    if (int status = require_buffer_size(record.buffers[11 + i], (uint64_t)args.m * args.n[i] * 2, "output")) return status;
    args.w[i] = {record.buffers[4 + 2 * i].device, as_f16(record.buffers[5 + 2 * i])};
  }
  if (args.k > kFusedMaxWidth) return fail(LLMOPT_ERR_INVALID, "%s takes activations of at most %u values, got %u", name, kFusedMaxWidth, args.k);
  if (args.in.partial_count > kFusedMaxPartials)
    return fail(LLMOPT_ERR_INVALID, "%s takes at most %u partial sums, got %u", name, kFusedMaxPartials, args.in.partial_count);
  if (!std::isfinite(args.norm.epsilon) || args.norm.epsilon <= 0.0f)
    return fail(LLMOPT_ERR_INVALID, "%s requires a positive finite epsilon", name);
  if (args.token_elements % 64 != 0 || args.token_stride % 2 != 0 ||
      (uint64_t)args.token_stride < (uint64_t)args.token_elements + 2ull * (args.token_elements / 64) ||
      args.key_offset % 64 != 0 || args.value_offset % 64 != 0 ||
      (uint64_t)args.key_offset + args.n[1] > args.token_elements ||
      (uint64_t)args.value_offset + args.n[2] > args.token_elements)
    return fail(LLMOPT_ERR_INVALID, "%s received an inconsistent Q8 token layout", name);
  const uint64_t stream_bytes = (uint64_t)args.m * args.k * 2;
  if (int status = require_buffer_size(record.buffers[0], stream_bytes, "input")) return status;
  if (args.in.partial_count != 0)
    if (int status = require_buffer_size(record.buffers[1], (uint64_t)args.in.partial_count * args.m * args.k * 4, "partial sums"))
      return status;
  if (int status = require_buffer_size(record.buffers[2], stream_bytes, "stream")) return status;
  if (int status = require_buffer_size(record.buffers[3], (uint64_t)args.k * 2, "norm weight")) return status;
  if (int status = require_buffer_size(record.buffers[10], (uint64_t)args.m * 64 * 2 * 2, "cosine and sine rows")) return status;
  if (int status = require_buffer_size(record.buffers[14], (uint64_t)args.m * 4, "slots")) return status;
  if (int status = require_buffer_size(record.buffers[15], args.token_stride, "pool")) return status;
  args.in.x = as_f16(record.buffers[0]);
  args.in.partials = reinterpret_cast<const float *>(record.buffers[1].device);
  args.in.x_out = reinterpret_cast<uint16_t *>(record.buffers[2].device);
  args.cosine = as_f16(record.buffers[10]);
  args.sine = args.cosine + (size_t)args.m * 64;
  args.q_out = reinterpret_cast<uint16_t *>(record.buffers[11].device);
  args.k_out = reinterpret_cast<uint16_t *>(record.buffers[12].device);
  args.v_out = reinterpret_cast<uint16_t *>(record.buffers[13].device);
  args.slots = reinterpret_cast<const uint32_t *>(record.buffers[14].device);
  args.pool = record.buffers[15].device;
  if (args.in.x == args.in.x_out)
    return fail(LLMOPT_ERR_INVALID, "%s writes the stream while other workgroups still read the input: two buffers", name);
  if (!fused_qkv_ok(args))
    return fail(LLMOPT_ERR_INVALID, "%s requires 16-byte aligned buffers, and rows of more than 1024 values take at most 32 "
                "partial sums", name);
  return launched(launch_fused_qkv(args, context->stream), name);
}

// Extension (no reference kernel): llmopt_w4a16_swiglu_rms_f16_g64, llmopt_w4a16_dual_swiglu_f16_g64 and
// the contraction of llmopt_w4a16_down_add_f16_g64 as ONE launch that leaves, per `slice` columns of the
// intermediate, a float32 partial sum of every output; the launch that reads the stream next adds them
// and the residual (llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64).  W4A16SwiGLUFFNParams {u32 m, n, k; f32 eps},
// then u32 slice: 64 or 32 (32: twice the workgroups with half the weights each, and twice the partial sums).
// buffers: input f16 [m,k], norm weight, gateW, gateS, upW, upS, downW, downS, partials f32 [n/slice,m,k].
// `summing` (llmopt_sum_rms_w4a16_swiglu_down_partial_f16_g64): the input itself arrives as rows plus
// pending partial sums (of the projecting attention entry) and is written out whole: buffers input,
// pending f32 [pending_count,m,k], stream f16 [m,k], then as above; u32 pending_count follows epsilon, slice follows it.
int swiglu_down_partial(llmopt_hip_context *context, const DispatchRecord &record, bool summing) {
  const size_t b = summing ? 2 : 0;
  if (int status = require_buffer_count(record, 9 + b)) return status;
  if (int status = require_parameter_bytes(record, summing ? 24 : 20)) return status;
  const char *name = record.name.c_str();
  const uint32_t m = param_u32(record, 0), n = param_u32(record, 4), k = param_u32(record, 8);
  const float epsilon = param_f32(record, 12);
  if (int status = check_w4_shape(name, m, n, k)) return status;
  const uint32_t slice = param_u32(record, summing ? 20 : 16);
  if (slice != 32 && slice != 64) return fail(LLMOPT_ERR_INVALID, "%s takes slices of 32 or 64 columns, got %u", name, slice);
  if (!fused_ffn_ok(m, n, k, summing && param_u32(record, 16) != 0, slice))
    return fail(LLMOPT_ERR_INVALID, "%s takes a hidden width k whose slice of the three matrices fits a workgroup's "
                "memory (slices of 64: k <= 1472, with pending sums k <= 1344) and n a multiple of the slice up to %u "
                "slices, got k = %u, n = %u, slice = %u", name, kFusedMaxPartials, k, n, slice);
  if (!std::isfinite(epsilon) || epsilon <= 0.0f) return fail(LLMOPT_ERR_INVALID, "%s requires a positive finite epsilon", name);
  if (int status = require_buffer_size(record.buffers[0], (uint64_t)m * k * 2, "input")) return status;
  if (int status = require_buffer_size(record.buffers[b + 1], (uint64_t)k * 2, "norm weight")) return status;
  if (int status = check_w4_matrix(record.buffers[b + 2], record.buffers[b + 3], n, k, "gate")) return status;
  if (int status = check_w4_matrix(record.buffers[b + 4], record.buffers[b + 5], n, k, "up")) return status;
  if (int status = check_w4_matrix(record.buffers[b + 6], record.buffers[b + 7], k, n, "down")) return status;
  if (int status = require_buffer_size(record.buffers[b + 8], (uint64_t)(n / slice) * m * k * 4, "partial sums")) return status;
  FusedFfnArgs args = {};
  args.in.x = as_f16(record.buffers[0]);
  if (summing) {
    args.in.partial_count = param_u32(record, 16);
    if (args.in.partial_count > kFusedMaxPartials)
      return fail(LLMOPT_ERR_INVALID, "%s takes at most %u pending partial sums, got %u", name, kFusedMaxPartials, args.in.partial_count);
    if (args.in.partial_count != 0)
      if (int status = require_buffer_size(record.buffers[1], (uint64_t)args.in.partial_count * m * k * 4, "pending partial sums"))
        return status;
    if (int status = require_buffer_size(record.buffers[2], (uint64_t)m * k * 2, "stream")) return status;
    args.in.partials = reinterpret_cast<const float *>(record.buffers[1].device);
    args.in.x_out = reinterpret_cast<uint16_t *>(record.buffers[2].device);
    if (args.in.x_out == args.in.x)
      return fail(LLMOPT_ERR_INVALID, "%s writes the stream while other workgroups still read the input: two buffers", name);
  }
  args.norm = {as_f16(record.buffers[b + 1]), epsilon, 1};
  args.gate = {record.buffers[b + 2].device, as_f16(record.buffers[b + 3])};
  args.up = {record.buffers[b + 4].device, as_f16(record.buffers[b + 5])};
  args.down = {record.buffers[b + 6].device, as_f16(record.buffers[b + 7])};
  args.partials = reinterpret_cast<float *>(record.buffers[b + 8].device);
  args.m = m;
  args.n = n;
  args.k = k;
  args.slice = slice;
  return launched(launch_fused_ffn(args, context->stream), name);
}

int rms_w4a16_swiglu_down_partial(llmopt_hip_context *context, const DispatchRecord &record) {
  return swiglu_down_partial(context, record, false);
}

int sum_rms_w4a16_swiglu_down_partial(llmopt_hip_context *context, const DispatchRecord &record) {
  return swiglu_down_partial(context, record, true);
}

// Extension (no reference kernel): float32 [n,k] from the product kernels' own nibble decoders,
// for checking the unpack arithmetic bit for bit.  Parameters {u32 n, k} or {u32 n, k, decoder}:
// decoder 0 (default) = w4_decode_pairs x scale, 1 = w4_decode_biased minus its bias x scale, 2 = the
// prefill GEMM's staged half(q * scale).  buffers: packed, scale, output.
int w4_dequant_f32(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 3)) return status;
  if (record.parameters.size() != 8 && record.parameters.size() != 12)
    return fail(LLMOPT_ERR_INVALID, "%s expects an 8- or 12-byte parameter block, got %zu", record.name.c_str(),
                record.parameters.size());
  const uint32_t n = param_u32(record, 0), k = param_u32(record, 4);
  const uint32_t decoder = record.parameters.size() == 12 ? param_u32(record, 8) : 0;
  if (decoder > 2) return fail(LLMOPT_ERR_INVALID, "%s knows decoders 0, 1 and 2, got %u", record.name.c_str(), decoder);
  if (int status = check_w4_shape(record.name.c_str(), 1, n, k)) return status;
  if (int status = check_w4_matrix(record.buffers[0], record.buffers[1], n, k, "W4A16")) return status;
  if (int status = require_buffer_size(record.buffers[2], (uint64_t)n * k * 4, "output")) return status;
  W4Matrix w = {record.buffers[0].device, as_f16(record.buffers[1])};
  return launched(launch_w4_dequant_f32(w, reinterpret_cast<float *>(record.buffers[2].device), n, k, decoder,
                                        context->stream),
                  record.name.c_str());
}

// Extension (no reference kernel): float32 [count] from the attention kernels' own int8
// decoders.  Parameters {u32 count, decoder}: count a multiple of 4; decoder 0 = int8x4_to_h2,
// 1 = int8x4_to_h2_biased minus its bias.  buffers: int8 bytes, output.
int q8_decode_f32(llmopt_hip_context *context, const DispatchRecord &record) {
  if (int status = require_buffer_count(record, 2)) return status;
  if (int status = require_parameter_bytes(record, 8)) return status;
  const uint32_t count = param_u32(record, 0), decoder = param_u32(record, 4);
  if (count == 0 || count % 4 != 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires a positive multiple of 4 bytes, got %u", record.name.c_str(), count);
  if (decoder > 1) return fail(LLMOPT_ERR_INVALID, "%s knows decoders 0 and 1, got %u", record.name.c_str(), decoder);
  if (int status = require_buffer_size(record.buffers[0], count, "int8")) return status;
  if (int status = require_buffer_size(record.buffers[1], (uint64_t)count * 4, "output")) return status;
  return launched(launch_q8_decode_f32(record.buffers[0].device, reinterpret_cast<float *>(record.buffers[1].device),
                                       count, decoder, context->stream),
                  record.name.c_str());
}

}  // namespace

void register_linear_kernels(std::vector<KernelEntryPoint> &table) {
  static const char *const linear = "w4a16-linear-g64";
  static const char *const qkv = "w4a16-qkv-linear-g64";
  static const char *const ffn = "w4a16-swiglu-ffn-g64";
  table.push_back({"llmopt_w4a16_linear_f16_g64", linear, w4a16_linear});
  table.push_back({"llmopt_w4a16_linear_f16_g64_m4", linear, w4a16_linear});
  table.push_back({"llmopt_w4a16_linear_f16_g64_m8", linear, w4a16_linear});
  table.push_back({"llmopt_w4a16_qkv_linear_f16_g64", qkv, w4a16_qkv_linear});
  table.push_back({"llmopt_w4a16_qkv_linear_f16_g64_m4", qkv, w4a16_qkv_linear});
  table.push_back({"llmopt_w4a16_qkv_linear_f16_g64_m8", qkv, w4a16_qkv_linear});
  table.push_back({"llmopt_rms_w4a16_qkv_linear_f16_g64", qkv, rms_w4a16_qkv_linear});
  table.push_back({"llmopt_rms_w4a16_dual_swiglu_f16_g64", ffn, rms_w4a16_dual_swiglu});
  table.push_back({"llmopt_w4a16_dual_swiglu_f16_g64", ffn, w4a16_dual_swiglu});
  table.push_back({"llmopt_w4a16_dual_swiglu_f16_g64_m4", ffn, w4a16_dual_swiglu});
  table.push_back({"llmopt_w4a16_dual_swiglu_f16_g64_m8", ffn, w4a16_dual_swiglu});
  table.push_back({"llmopt_w4a16_down_add_f16_g64", ffn, w4a16_down_add});
  table.push_back({"llmopt_w4a16_down_add_f16_g64_m4", ffn, w4a16_down_add});
  table.push_back({"llmopt_w4a16_down_add_f16_g64_m8", ffn, w4a16_down_add});
  table.push_back({"llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64", qkv, rms_w4a16_qkv_rotary_pack});
  table.push_back({"llmopt_rms_w4a16_swiglu_down_partial_f16_g64", ffn, rms_w4a16_swiglu_down_partial});
  table.push_back({"llmopt_sum_rms_w4a16_swiglu_down_partial_f16_g64", ffn, sum_rms_w4a16_swiglu_down_partial});
  table.push_back({"llmopt_w4_dequant_f32", linear, w4_dequant_f32});
  table.push_back({"llmopt_q8_decode_f32", "cache", q8_decode_f32});
}

}  // namespace llmopt
