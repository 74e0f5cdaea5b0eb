// Operator layer above the flat kernel ABI: the reference's dispatch_* operators
// (lib/metal_dispatch_linear.ml, lib/metal_dispatch_attention.ml), the helpers
// they use (lib/metal_dispatch_common.ml, lib/metal_parameters.ml) and the
// kernel-entry lookup (lib/metal_native.ml:461-512) with plain C types.
//
// Buffers, batches and dispatches go through the public functions of
// llmopt_hip.h only (plus the library's error slot and kernel registry): this
// file is the host-language side of the boundary, written in C++ because the
// reference's host language (OCaml) is compiled code and has no toolchain here.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <limits>
#include <string>
#include <vector>

#include "../../../include/llmopt_hip_ops.h"
#include "../runtime.h"

struct llmopt_op_context {
  llmopt_hip_context *device = nullptr;
  llmopt_hip_library *library = nullptr;
  llmopt_hip_batch *batch = nullptr;  // not owned
  // Execution_batch scratch (lib/metal_execution_state.ml:80-101), grown on demand
  llmopt_hip_buffer *swiglu_normalized = nullptr;
  llmopt_hip_buffer *swiglu_product = nullptr;
  llmopt_hip_buffer *candidates = nullptr;
  std::string kernels;
};

namespace {

using llmopt::fail;

constexpr int64_t kMaxInt = std::numeric_limits<int64_t>::max() >> 1;  // OCaml's max_int (63-bit)

// ---- Metal_parameters ---------------------------------------------------------

struct Parameters {
  std::vector<uint8_t> bytes;
  int status = LLMOPT_OK;

  void u32(int64_t value) {  // set_u32, lib/metal_parameters.ml:6-12
    if (value < 0 || value > 0xffffffffll) {
      if (status == LLMOPT_OK)
        status = fail(LLMOPT_ERR_FAILURE, "Metal parameter does not fit uint32: %lld", (long long)value);
      value = 0;
    }
    const uint32_t encoded = (uint32_t)value;
    const uint8_t *raw = reinterpret_cast<const uint8_t *>(&encoded);
    bytes.insert(bytes.end(), raw, raw + 4);
  }
  void f32(double value) {  // Int32.bits_of_float: OCaml rounds the double to single
    const float encoded = (float)value;
    const uint8_t *raw = reinterpret_cast<const uint8_t *>(&encoded);
    bytes.insert(bytes.end(), raw, raw + 4);
  }
};

// ---- lib/metal_dispatch_common.ml ----------------------------------------------

int64_t round_up(int64_t value, int64_t multiple) {
  if (value > kMaxInt - (multiple - 1)) return -1;
  return ((value + multiple - 1) / multiple) * multiple;
}

int64_t linear_f16_grid(int64_t columns) {
  const int64_t rounded = round_up(columns, 8);
  if (rounded < 0) return -1;
  if (rounded > kMaxInt / 32) return -1;
  return rounded * 32;
}

const char *paged_kernel_name(bool experimental_gqa3_split8, bool split8, int64_t query_heads,
                              int64_t kv_heads, int64_t head_dimension) {
  const bool gqa3_shape = query_heads == 3 * kv_heads;
  if (head_dimension == 256) return "llmopt_attention_q8_paged_simd_h256";
  if (head_dimension == 512) return "llmopt_attention_q8_paged_simd_h512";
  if (head_dimension != 64) return "llmopt_attention_q8_paged_simd_generic";
  if (split8 && gqa3_shape && experimental_gqa3_split8) return "llmopt_attention_q8_paged_simd_h64_gqa3_split8";
  if (split8) return "llmopt_attention_q8_paged_simd_h64_split8";
  if (gqa3_shape) return "llmopt_attention_q8_paged_simd_h64_gqa3";
  return "llmopt_attention_q8_paged_simd_h64";
}

bool groups_by_kv_head(const char *name) {
  return strcmp(name, "llmopt_attention_q8_paged_simd_h64_gqa3") == 0 ||
         strcmp(name, "llmopt_attention_q8_paged_simd_h64_gqa3_split8") == 0;
}

// ---- values ----------------------------------------------------------------------

int64_t numel(const llmopt_op_value &value) {
  int64_t count = 1;
  for (uint32_t axis = 0; axis < value.rank && axis < 8; ++axis) count *= value.dims[axis];
  return count;
}

bool has_dims(const llmopt_op_value &value, std::initializer_list<int64_t> dims) {
  if (value.rank != dims.size()) return false;
  uint32_t axis = 0;
  for (int64_t d : dims)
    if (value.dims[axis++] != d) return false;
  return true;
}

bool same_shape(const llmopt_op_value &a, const llmopt_op_value &b) {
  if (a.rank != b.rank) return false;
  for (uint32_t axis = 0; axis < a.rank && axis < 8; ++axis)
    if (a.dims[axis] != b.dims[axis]) return false;
  return true;
}

// Metal_execution_state.find_value: a value without a buffer is not bound.
int find_value(const llmopt_op_value *value, llmopt_hip_buffer **out) {
  if (value == nullptr || value->buffer == nullptr)
    return fail(LLMOPT_ERR_FAILURE, "schedule value is not bound to a Metal buffer");
  *out = value->buffer;
  return LLMOPT_OK;
}

// ---- Metal_native.kernel_entry + dispatch -------------------------------------------

// "exactly one entry with this name, operation and dtypes" (lib/metal_native.ml:473-487):
// here a name is registered once, so the check is name + operation.
int kernel_entry(llmopt_op_context *context, const char *name, const char *operation) {
  const int present = llmopt_hip_has_function(context->library, name);
  if (present < 0) return present;
  const llmopt::KernelEntryPoint *entry = llmopt::find_kernel(name);
  if (present == 0 || entry == nullptr || strcmp(entry->operation, operation) != 0)
    return fail(LLMOPT_ERR_FAILURE, "model package does not contain the selected kernel %s for %s", name,
                operation);
  return LLMOPT_OK;
}

int dispatch(llmopt_op_context *context, const char *name, const char *operation,
             const std::vector<llmopt_hip_buffer *> &buffers, const Parameters &parameters, int64_t grid_x,
             int64_t grid_y = 1) {
  if (parameters.status != LLMOPT_OK) return parameters.status;
  if (int status = kernel_entry(context, name, operation)) return status;
  llmopt_hip_dispatch_item item = {};
  item.name = name;
  item.buffers = buffers.data();
  item.buffer_count = (uint32_t)buffers.size();
  item.parameters = parameters.bytes.data();
  item.parameter_bytes = (uint32_t)parameters.bytes.size();
  item.grid[0] = grid_x;
  item.grid[1] = grid_y;
  item.grid[2] = 1;
  item.group[0] = 256;  // every entry of this path declares a (256,1,1) threadgroup
  item.group[1] = item.group[2] = 1;
  const int status = context->batch != nullptr ? llmopt_hip_batch_dispatch(context->batch, context->library, &item)
                                               : llmopt_hip_dispatch(context->library, &item);
  if (status == LLMOPT_OK) {
    if (!context->kernels.empty()) context->kernels += "\n";
    context->kernels += name;
  }
  return status;
}

// Execution_batch scratch: reuse when large enough, else allocate and keep
// (lib/metal_dispatch_linear.ml:321-345).  A replaced buffer may still be used
// by dispatches recorded in an open batch: it is retained by those records.
int scratch(llmopt_op_context *context, llmopt_hip_buffer **slot, int64_t bytes) {
  if (*slot != nullptr) {
    const int64_t length = llmopt_hip_buffer_length(*slot);
    if (length < 0) return (int)length;
    if (length >= bytes) return LLMOPT_OK;
    llmopt_hip_release_buffer(*slot);
    *slot = nullptr;
  }
  return llmopt_hip_create_buffer(context->device, bytes, slot);
}

bool valid_epsilon(double epsilon) { return isfinite(epsilon) && epsilon > 0.0; }

}  // namespace

extern "C" {

int llmopt_op_context_create(llmopt_hip_context *device, llmopt_hip_library *library, llmopt_op_context **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "operator context output pointer is null");
  *out = nullptr;
  if (device == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  llmopt_op_context *context = new llmopt_op_context();
  context->device = device;
  context->library = library;
  *out = context;
  return LLMOPT_OK;
}

void llmopt_op_context_release(llmopt_op_context *context) {
  if (context == nullptr) return;
  if (context->swiglu_normalized) llmopt_hip_release_buffer(context->swiglu_normalized);
  if (context->swiglu_product) llmopt_hip_release_buffer(context->swiglu_product);
  if (context->candidates) llmopt_hip_release_buffer(context->candidates);
  delete context;
}

int llmopt_op_context_set_batch(llmopt_op_context *context, llmopt_hip_batch *batch) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->batch = batch;
  return LLMOPT_OK;
}

const char *llmopt_op_last_kernels(llmopt_op_context *context) {
  return context == nullptr ? "" : context->kernels.c_str();
}

int llmopt_op_w4a16_linear(llmopt_op_context *context, int64_t m, int64_t n, int64_t k, int has_bias,
                           const llmopt_op_value *values, size_t value_count, const llmopt_op_value *output) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->kernels.clear();
  if (values == nullptr || !((value_count == 3 && !has_bias) || (value_count == 4 && has_bias)))
    return fail(LLMOPT_ERR_FAILURE, "W4A16 schedule command has inconsistent bias inputs");
  llmopt_hip_buffer *input, *weight, *scale, *bias, *out;
  if (int status = find_value(&values[0], &input)) return status;
  if (int status = find_value(&values[1], &weight)) return status;
  if (int status = find_value(&values[2], &scale)) return status;
  bias = scale;
  if (has_bias)
    if (int status = find_value(&values[3], &bias)) return status;
  if (int status = find_value(output, &out)) return status;
  const int64_t bias_row_stride = (has_bias && numel(values[3]) == m * n) ? n : 0;
  Parameters parameters;
  for (int64_t value : {m, n, k, (int64_t)(has_bias ? 1 : 0), bias_row_stride}) parameters.u32(value);
  const bool single = m == 1;
  const int64_t grid = linear_f16_grid(single ? m * n : ((m + 3) / 4) * n);
  if (grid < 0) return fail(LLMOPT_ERR_FAILURE, "Metal float16 linear grid dimension overflows");
  return dispatch(context, single ? "llmopt_w4a16_linear_f16_g64" : "llmopt_w4a16_linear_f16_g64_m4",
                  "w4a16-linear-g64", {input, weight, scale, bias, out}, parameters, grid);
}

int llmopt_op_w4a16_qkv_linear(llmopt_op_context *context, int64_t m, int64_t k, int64_t n_q, int64_t n_k,
                               int64_t n_v, const llmopt_op_value *values, size_t value_count,
                               const llmopt_op_value *output, const llmopt_op_value *extra_outputs,
                               size_t extra_count) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->kernels.clear();
  if (values == nullptr || value_count != 7)
    return fail(LLMOPT_ERR_FAILURE, "W4A16 QKV linear command has inconsistent inputs");
  std::vector<llmopt_hip_buffer *> buffers(10);
  for (size_t i = 0; i < 7; ++i)
    if (int status = find_value(&values[i], &buffers[i])) return status;
  if (int status = find_value(output, &buffers[7])) return status;
  if (extra_outputs == nullptr || extra_count != 2)
    return fail(LLMOPT_ERR_FAILURE, "W4A16 QKV linear command requires 2 extra outputs (K and V)");
  if (int status = find_value(&extra_outputs[0], &buffers[8])) return status;
  if (int status = find_value(&extra_outputs[1], &buffers[9])) return status;
  Parameters parameters;
  for (int64_t value : {m, k, n_q, n_k, n_v}) parameters.u32(value);
  const int64_t total = n_q + n_k + n_v;
  const bool single = m == 1;
  const int64_t grid = linear_f16_grid(single ? m * total : ((m + 3) / 4) * total);
  if (grid < 0) return fail(LLMOPT_ERR_FAILURE, "Metal float16 linear grid dimension overflows");
  return dispatch(context, single ? "llmopt_w4a16_qkv_linear_f16_g64" : "llmopt_w4a16_qkv_linear_f16_g64_m4",
                  "w4a16-qkv-linear-g64", buffers, parameters, grid);
}

int llmopt_op_w4a16_swiglu_ffn(llmopt_op_context *context, int64_t m, int64_t n, int64_t k, double epsilon,
                               const llmopt_op_value *values, size_t value_count,
                               const llmopt_op_value *output) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->kernels.clear();
  if (values == nullptr || value_count != 9)
    return fail(LLMOPT_ERR_FAILURE, "W4A16 SwiGLU command has inconsistent inputs");
  const llmopt_op_value &activation = values[0], &residual = values[1], &gate_w = values[2],
                        &gate_s = values[3], &up_w = values[4], &up_s = values[5], &down_w = values[6],
                        &down_s = values[7], &norm_w = values[8];
  std::vector<llmopt_hip_buffer *> bound(9);
  for (size_t i = 0; i < 9; ++i)
    if (int status = find_value(&values[i], &bound[i])) return status;
  llmopt_hip_buffer *out;
  if (int status = find_value(output, &out)) return status;
  const bool consistent =
      valid_epsilon(epsilon) && m > 0 && n > 0 && k > 0 && n % 64 == 0 && k % 64 == 0 && k <= 2048 &&
      n <= 8192 && (activation.dtype == LLMOPT_F16 || activation.dtype == LLMOPT_F32) &&
      residual.dtype == LLMOPT_F16 && gate_w.dtype == LLMOPT_U8 && gate_s.dtype == LLMOPT_F16 &&
      up_w.dtype == LLMOPT_U8 && up_s.dtype == LLMOPT_F16 && down_w.dtype == LLMOPT_U8 &&
      down_s.dtype == LLMOPT_F16 && norm_w.dtype == LLMOPT_F16 && output->dtype == LLMOPT_F16 &&
      numel(activation) == m * k && same_shape(residual, *output) && numel(*output) == m * k &&
      has_dims(gate_w, {n, k / 2}) && has_dims(gate_s, {n, k / 64}) && has_dims(up_w, {n, k / 2}) &&
      has_dims(up_s, {n, k / 64}) && has_dims(down_w, {k, n / 2}) && has_dims(down_s, {k, n / 64}) &&
      has_dims(norm_w, {k});
  if (!consistent) return fail(LLMOPT_ERR_FAILURE, "W4A16 SwiGLU input metadata is inconsistent");
  if (int status = scratch(context, &context->swiglu_normalized, m * k * 2)) return status;
  if (int status = scratch(context, &context->swiglu_product, m * n * 2)) return status;
  Parameters parameters;  // Parameters.w4a16_swiglu_ffn, lib/metal_parameters.ml:45-51
  for (int64_t value : {m, n, k}) parameters.u32(value);
  parameters.f32(epsilon);
  static const char *const operation = "w4a16-swiglu-ffn-g64";
  const char *rms = activation.dtype == LLMOPT_F16 ? "llmopt_w4a16_swiglu_rms_f16_g64"
                                                   : "llmopt_w4a16_swiglu_rms_f32_g64";
  if (int status = dispatch(context, rms, operation, {bound[0], bound[8], context->swiglu_normalized},
                            parameters, m * 256))
    return status;
  const bool single = m == 1;
  const int64_t blocks = single ? m : (m + 3) / 4;
  const int64_t dual_grid = linear_f16_grid(blocks * n), down_grid = linear_f16_grid(blocks * k);
  if (dual_grid < 0 || down_grid < 0)
    return fail(LLMOPT_ERR_FAILURE, "Metal float16 linear grid dimension overflows");
  if (int status = dispatch(context,
                            single ? "llmopt_w4a16_dual_swiglu_f16_g64" : "llmopt_w4a16_dual_swiglu_f16_g64_m4",
                            operation,
                            {context->swiglu_normalized, bound[2], bound[3], bound[4], bound[5],
                             context->swiglu_product},
                            parameters, dual_grid))
    return status;
  return dispatch(context, single ? "llmopt_w4a16_down_add_f16_g64" : "llmopt_w4a16_down_add_f16_g64_m4",
                  operation, {context->swiglu_product, bound[6], bound[7], bound[1], out}, parameters, down_grid);
}

int llmopt_op_w4a16_lm_head_argmax(llmopt_op_context *context, int64_t m, int64_t n, int64_t k, double epsilon,
                                   const llmopt_op_value *values, size_t value_count,
                                   const llmopt_op_value *output, const llmopt_op_value *extra_outputs,
                                   size_t extra_count) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->kernels.clear();
  if (values == nullptr || value_count != 4)
    return fail(LLMOPT_ERR_FAILURE, "W4A16 LM-head argmax command has inconsistent inputs");
  const llmopt_op_value &input = values[0], &norm_w = values[1], &weight = values[2], &scale = values[3];
  std::vector<llmopt_hip_buffer *> bound(4);
  for (size_t i = 0; i < 4; ++i)
    if (int status = find_value(&values[i], &bound[i])) return status;
  llmopt_hip_buffer *out;
  if (int status = find_value(output, &out)) return status;
  if (extra_count > 1)
    return fail(LLMOPT_ERR_FAILURE, "W4A16 LM-head argmax command receives at most one extra output (logits)");
  const llmopt_op_value *extra = extra_count == 1 ? &extra_outputs[0] : nullptr;
  llmopt_hip_buffer *extra_buffer = nullptr;
  if (extra != nullptr)
    if (int status = find_value(extra, &extra_buffer)) return status;
  const bool consistent = valid_epsilon(epsilon) && m > 0 && n > 0 && k > 0 && k % 64 == 0 && k <= 2048 &&
                          (input.dtype == LLMOPT_F16 || input.dtype == LLMOPT_F32) && numel(input) == m * k &&
                          has_dims(norm_w, {k}) && has_dims(weight, {n, k / 2}) &&
                          has_dims(scale, {n, k / 64}) && numel(*output) == m &&
                          (extra == nullptr || (extra->dtype == LLMOPT_F16 && has_dims(*extra, {m, n})));
  if (!consistent) return fail(LLMOPT_ERR_FAILURE, "W4A16 LM-head argmax input metadata is inconsistent");
  // two-stage form: stage 1 leaves 256 candidates per row, the reduce picks the winner
  if (int status = scratch(context, &context->candidates, m * 256 * 8)) return status;
  Parameters parameters;  // Parameters.w4a16_lm_head_argmax, lib/metal_parameters.ml:38-43
  for (int64_t value : {m, n, k}) parameters.u32(value);
  parameters.f32(epsilon);
  std::string stage1 = std::string("llmopt_w4a16_lm_head_argmax_stage1") + (extra ? "_extra" : "") +
                       (input.dtype == LLMOPT_F16 ? "_f16" : "_f32");
  std::vector<llmopt_hip_buffer *> buffers = {bound[0], bound[1], bound[2], bound[3], context->candidates};
  if (extra_buffer) buffers.push_back(extra_buffer);
  static const char *const operation = "w4a16-lm-head-argmax";
  // stage-1 grid: the reference takes threadgroups x threads from its cost model
  // (lib/metal_dispatch_linear.ml:662-670); one 256-thread group per 256 columns here
  const int64_t stage1_threads = ((n + 255) / 256) * 256;
  if (int status = dispatch(context, stage1.c_str(), operation, buffers, parameters, stage1_threads, m))
    return status;
  Parameters reduce_parameters;
  reduce_parameters.u32(m);
  return dispatch(context, "llmopt_w4a16_lm_head_reduce", operation, {context->candidates, out},
                  reduce_parameters, m * 256);
}

int llmopt_op_paged_attention_q8(llmopt_op_context *context, const llmopt_op_paged_attention_config *config,
                                 const llmopt_op_value *query, const llmopt_op_value *current_key,
                                 const llmopt_op_value *current_value, const llmopt_op_value *pool,
                                 const llmopt_op_value *slots, const llmopt_op_value *mask_values,
                                 size_t mask_count, const llmopt_op_value *output) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->kernels.clear();
  if (config == nullptr || query == nullptr || current_key == nullptr || current_value == nullptr ||
      pool == nullptr || slots == nullptr || output == nullptr)
    return fail(LLMOPT_ERR_INVALID, "paged Q8 attention argument is null");
  if (mask_count > 1) return fail(LLMOPT_ERR_FAILURE, "paged Q8 attention receives at most one mask value");
  if (query->rank != 4) return fail(LLMOPT_ERR_FAILURE, "paged Q8 attention query must have shape [b,h,q,d]");
  const int64_t batches = query->dims[0], query_heads = query->dims[1], query_length = query->dims[2],
                head_dimension = query->dims[3];
  if (current_key->rank != 4 || current_key->dims[2] != query_length)
    return fail(LLMOPT_ERR_FAILURE, "paged Q8 attention current key must match query tokens");
  const int64_t kv_heads = current_key->dims[1];
  if (slots->rank != 1) return fail(LLMOPT_ERR_FAILURE, "paged Q8 attention slots must have rank one");
  const int64_t past_length = slots->dims[0];
  int64_t mask_batches = 0, mask_heads = 0, mask_dtype = 0;
  const llmopt_op_value *mask_buffer = slots;
  if (mask_count == 0) {
    if (query_length != 1) return fail(LLMOPT_ERR_FAILURE, "maskless paged Q8 attention requires one query token");
  } else {
    const llmopt_op_value &mask = mask_values[0];
    if (mask.rank != 4 || !(mask.dims[2] == query_length || mask.dims[2] == 1))
      return fail(LLMOPT_ERR_FAILURE, "paged Q8 attention mask must have rank four");
    if (mask.dtype == LLMOPT_BOOL)
      mask_dtype = 1;
    else if (mask.dtype == LLMOPT_F16)
      mask_dtype = 2;
    else
      return fail(LLMOPT_ERR_FAILURE, "paged Q8 attention mask dtype %d is unsupported", mask.dtype);
    mask_batches = mask.dims[0];
    mask_heads = mask.dims[1];
    mask_buffer = &mask;
  }
  std::vector<llmopt_hip_buffer *> buffers(7);
  const llmopt_op_value *ordered[6] = {query, current_key, current_value, pool, slots, mask_buffer};
  for (size_t i = 0; i < 6; ++i)
    if (int status = find_value(ordered[i], &buffers[i])) return status;
  if (int status = find_value(output, &buffers[6])) return status;
  uint8_t raw[64];
  if (int status = llmopt_op_parameters_paged_attention_q8(
          raw, batches, query_heads, kv_heads, past_length, head_dimension, mask_batches, mask_heads,
          config->token_elements, config->key_offset, config->value_offset, config->group_size,
          config->token_stride, config->scale, mask_dtype, query_length, config->window))
    return status;
  Parameters parameters;
  parameters.bytes.assign(raw, raw + 64);
  const char *split8_env = getenv("LLMOPT_EXPERIMENTAL_SPLIT8");
  const char *gqa3_env = getenv("LLMOPT_EXPERIMENTAL_GQA3_SPLIT8");
  const bool split8 = split8_env != nullptr && strcmp(split8_env, "1") == 0 && head_dimension == 64 &&
                      query_length == 1 && past_length >= 64;
  const char *name = paged_kernel_name(gqa3_env != nullptr && strcmp(gqa3_env, "1") == 0, split8, query_heads,
                                       kv_heads, head_dimension);
  const int64_t rows = batches * (groups_by_kv_head(name) ? kv_heads : query_heads) * query_length;
  int64_t grid;
  if (split8) {
    if (rows > kMaxInt / 256) return fail(LLMOPT_ERR_FAILURE, "paged Q8 split attention grid dimension overflows");
    grid = rows * 256;
  } else {
    grid = linear_f16_grid(rows);
    if (grid < 0) return fail(LLMOPT_ERR_FAILURE, "Metal float16 linear grid dimension overflows");
  }
  return dispatch(context, name, "attention", buffers, parameters, grid);
}

// dispatch_attention (lib/metal_dispatch_attention.ml:6-102): dense fp16
// attention, the prefill side of the KV cache.
int llmopt_op_attention(llmopt_op_context *context, double scale, int causal, const llmopt_op_value *query,
                        const llmopt_op_value *key, const llmopt_op_value *value, const llmopt_op_value *mask,
                        const llmopt_op_value *output) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "operator context has been finalized");
  context->kernels.clear();
  if (query == nullptr || key == nullptr || value == nullptr || output == nullptr)
    return fail(LLMOPT_ERR_INVALID, "attention argument is null");
  if (query->rank != 4) return fail(LLMOPT_ERR_FAILURE, "attention query must have rank four");
  const int64_t batches = query->dims[0], heads = query->dims[1], query_length = query->dims[2],
                head_dimension = query->dims[3];
  if (key->rank != 4) return fail(LLMOPT_ERR_FAILURE, "attention key must have rank four");
  const int64_t kv_heads = key->dims[1], key_length = key->dims[2];
  int64_t token_first_value;
  if (has_dims(*value, {batches, kv_heads, key_length, head_dimension}))
    token_first_value = 0;  // also when kv_heads == key_length: head-major is tried first
  else if (has_dims(*value, {batches, key_length, kv_heads, head_dimension}))
    token_first_value = 1;
  else
    return fail(LLMOPT_ERR_FAILURE, "attention value must match key in head-major or token-major layout");
  int64_t mask_batches = 0, mask_heads = 0, mask_dtype = 0;
  const llmopt_op_value *mask_buffer = query;  // the query buffer fills the slot when there is no mask
  if (mask != nullptr) {
    if (mask->rank != 4) return fail(LLMOPT_ERR_FAILURE, "attention mask must have rank four");
    if (mask->dtype == LLMOPT_BOOL)
      mask_dtype = 1;
    else if (mask->dtype == LLMOPT_F16)
      mask_dtype = 2;
    else
      return fail(LLMOPT_ERR_FAILURE, "attention mask dtype %d is unsupported", mask->dtype);
    mask_batches = mask->dims[0];
    mask_heads = mask->dims[1];
    mask_buffer = mask;
  }
  const int64_t token_first_output =
      (has_dims(*output, {batches, query_length, heads * head_dimension}) ||
       has_dims(*output, {batches, query_length, heads, head_dimension}))
          ? 1
          : 0;
  std::vector<llmopt_hip_buffer *> buffers(5);
  const llmopt_op_value *ordered[5] = {query, key, value, mask_buffer, output};
  for (size_t i = 0; i < 5; ++i)
    if (int status = find_value(ordered[i], &buffers[i])) return status;
  const int64_t past_length = key_length > query_length ? key_length - query_length : 0;
  Parameters parameters;  // Parameters.attention, lib/metal_parameters.ml:95-117
  for (int64_t field : {batches, heads, query_length, key_length, head_dimension, mask_batches, mask_heads,
                        (int64_t)(causal != 0 ? 1 : 0)})
    parameters.u32(field);
  parameters.f32(scale);
  for (int64_t field : {kv_heads, token_first_output, past_length, token_first_value, mask_dtype})
    parameters.u32(field);
  // select_attention_kernel (lib/metal_dispatch_common.ml:166-189): the head-dimension entry
  // when the package has it, else the portable one
  char specialized[64];
  snprintf(specialized, sizeof specialized, "llmopt_attention_f16_simd_h%lld", (long long)head_dimension);
  const bool simd = head_dimension % 8 == 0 && llmopt_hip_has_function(context->library, specialized) == 1;
  const char *name = simd ? specialized : "llmopt_attention_f16";
  int64_t grid;
  if (simd) {
    const int64_t q_tiles = (query_length + 31) / 32;
    const int64_t groups = batches * heads * q_tiles;
    if (groups > kMaxInt / 128) return fail(LLMOPT_ERR_FAILURE, "Metal attention grid dimension overflows");
    grid = groups * 128;
  } else {
    grid = batches * heads * query_length;
  }
  return dispatch(context, name, "attention", buffers, parameters, grid);
}

const char *llmopt_op_paged_attention_kernel_name(int experimental_gqa3_split8, int split8, int64_t query_heads,
                                                  int64_t kv_heads, int64_t head_dimension) {
  return paged_kernel_name(experimental_gqa3_split8 != 0, split8 != 0, query_heads, kv_heads, head_dimension);
}

int64_t llmopt_op_linear_f16_grid(int64_t columns) { return linear_f16_grid(columns); }
int64_t llmopt_op_simd_rows_grid(int64_t rows) { return linear_f16_grid(rows); }

int llmopt_op_parameters_paged_attention_q8(uint8_t out[64], int64_t batches, int64_t query_heads,
                                            int64_t kv_heads, int64_t past_length, int64_t head_dimension,
                                            int64_t mask_batches, int64_t mask_heads, int64_t token_elements,
                                            int64_t key_offset, int64_t value_offset, int64_t group_size,
                                            int64_t token_stride, double scale, int64_t mask_dtype,
                                            int64_t query_length, int64_t window) {
  Parameters parameters;
  for (int64_t value : {batches, query_heads, kv_heads, past_length, head_dimension, mask_batches, mask_heads,
                        token_elements, key_offset, value_offset, group_size, token_stride})
    parameters.u32(value);
  parameters.f32(scale);
  parameters.u32(query_length);
  parameters.u32(mask_dtype);
  parameters.u32(window);
  if (parameters.status != LLMOPT_OK) return parameters.status;
  memcpy(out, parameters.bytes.data(), 64);
  return LLMOPT_OK;
}

// Kv_cache.Format.bytes_for_elements (lib/kv_cache.ml:10-21).
int64_t llmopt_op_kv_bytes_for_elements(int64_t elements) {
  if (elements < 0) return -1;
  const int64_t groups = elements / 64 + (elements % 64 == 0 ? 0 : 1);
  if (groups > (kMaxInt - elements) / 2) return -1;
  return elements + 2 * groups;
}

// Kv_cache.Layout.create_heterogeneous, attention layers only (lib/kv_cache.ml:80-166).
int llmopt_op_kv_layout(const llmopt_op_kv_layer *layers, size_t layer_count, llmopt_op_kv_region *regions,
                        int64_t *token_elements, int64_t *bytes_per_token) {
  if (layers == nullptr && layer_count != 0) return fail(LLMOPT_ERR_INVALID, "KV layout needs its attention layers");
  for (size_t i = 0; i < layer_count; ++i) {  // Attention_layer.create, :33-38
    if (layers[i].kv_heads <= 0) return fail(LLMOPT_ERR_FAILURE, "attention KV layer requires positive kv_heads");
    if (layers[i].head_dim <= 0) return fail(LLMOPT_ERR_FAILURE, "attention KV layer requires positive head_dim");
  }
  for (size_t i = 0; i < layer_count; ++i)
    if (layers[i].head_dim % 64 != 0)
      return fail(LLMOPT_ERR_FAILURE, "Q8 KV group_size must divide each attention head dimension");
  int64_t offset = 0;
  for (size_t i = 0; i < layer_count; ++i) {
    if (layers[i].kv_heads > kMaxInt / layers[i].head_dim)
      return fail(LLMOPT_ERR_FAILURE, "attention KV layer element count overflows");
    const int64_t elements = layers[i].kv_heads * layers[i].head_dim;
    const int64_t segment_bytes = llmopt_op_kv_bytes_for_elements(elements);
    if (segment_bytes < 0) return fail(LLMOPT_ERR_FAILURE, "attention KV segment byte length overflows");
    if (elements > kMaxInt - offset || elements > kMaxInt - (offset + elements))
      return fail(LLMOPT_ERR_FAILURE, "KV token element count overflows");
    if (regions != nullptr) regions[i] = {offset, offset + elements, elements, segment_bytes};
    offset += 2 * elements;
  }
  const int64_t bytes = llmopt_op_kv_bytes_for_elements(offset);
  if (bytes < 0) return fail(LLMOPT_ERR_FAILURE, "KV token byte length overflows");
  if (token_elements != nullptr) *token_elements = offset;
  if (bytes_per_token != nullptr) *bytes_per_token = bytes;
  return LLMOPT_OK;
}

const char *llmopt_op_kernel_operation(const char *kernel_name) {
  if (kernel_name == nullptr) return nullptr;
  const llmopt::KernelEntryPoint *entry = llmopt::find_kernel(kernel_name);
  return entry == nullptr ? nullptr : entry->operation;
}

}  // extern "C"
