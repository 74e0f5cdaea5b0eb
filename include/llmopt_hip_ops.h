/*
 * llmopt_hip_ops.h - operator-level entry points above the flat kernel ABI of
 * llmopt_hip.h.
 *
 * The reference reaches its kernels through five `dispatch_*` operators
 * (lib/metal_dispatch_linear.mli, lib/metal_dispatch_attention.mli), which
 * validate tensor metadata, choose the kernel entry, build the parameter block
 * and the Metal grid, and record the dispatch into the current batch.  The
 * functions below are those operators with plain C types: same argument
 * meaning, same kernel choice, same parameter bytes, same error strings.  They
 * are written only in terms of llmopt_hip.h, so an OCaml host can equally keep
 * its own lib/metal_dispatch_*.ml and bind llmopt_hip.h alone.
 *
 * Every function returns LLMOPT_OK or a negative status with the message in
 * llmopt_hip_last_error() (the reference returns `Error message`).
 */
#ifndef LLMOPT_HIP_OPS_H
#define LLMOPT_HIP_OPS_H

#include "llmopt_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Ir.Dtype tags used on this path. */
enum llmopt_op_dtype {
  LLMOPT_F16 = 0,
  LLMOPT_F32 = 1,
  LLMOPT_U8 = 2,
  LLMOPT_I32 = 3,
  LLMOPT_I64 = 4,
  LLMOPT_BOOL = 5
};

/* An Ir.Value bound to its buffer: what Metal_execution_state.find_value
 * resolves (logical shape, dtype, device buffer). */
typedef struct llmopt_op_value {
  llmopt_hip_buffer *buffer;
  int32_t dtype;
  uint32_t rank;
  int64_t dims[8];
} llmopt_op_value;

/* Metal_execution_state.context: the library, the open batch (NULL = dispatch
 * immediately and wait) and the per-batch scratch the operators cache
 * (swiglu_normalized, swiglu_product, candidates_buffer;
 * lib/metal_execution_state.ml:80-101). */
typedef struct llmopt_op_context llmopt_op_context;
int llmopt_op_context_create(llmopt_hip_context *context, llmopt_hip_library *library,
                             llmopt_op_context **out);
void llmopt_op_context_release(llmopt_op_context *context);
/* Sets / clears the batch that subsequent operators record into. */
int llmopt_op_context_set_batch(llmopt_op_context *context, llmopt_hip_batch *batch);
/* Names of the kernels the last operator call dispatched, '\n'-separated (the
 * `string list` the reference operators return). */
const char *llmopt_op_last_kernels(llmopt_op_context *context);

/* dispatch_w4a16_linear ctx st ~m ~n ~k ~has_bias values out
 * (lib/metal_dispatch_linear.ml:938-982).  values = [input; weight; scale]
 * (+ [bias] when has_bias); a bias of m*n elements is a residual (row stride n). */
int llmopt_op_w4a16_linear(llmopt_op_context *context, int64_t m, int64_t n, int64_t k, int has_bias,
                           const llmopt_op_value *values, size_t value_count,
                           const llmopt_op_value *output);

/* dispatch_w4a16_qkv_linear_command ctx st ~m ~k ~n_q ~n_k ~n_v ~extra_outputs values out
 * (lib/metal_dispatch_linear.ml:398-455).  values = [input; qW; qS; kW; kS; vW; vS];
 * output = Q, extra_outputs = [K; V]. */
int llmopt_op_w4a16_qkv_linear(llmopt_op_context *context, int64_t m, int64_t k, int64_t n_q,
                               int64_t n_k, int64_t n_v, const llmopt_op_value *values,
                               size_t value_count, const llmopt_op_value *output,
                               const llmopt_op_value *extra_outputs, size_t extra_count);

/* dispatch_w4a16_swiglu_ffn_command ctx st ~m ~n ~k ~epsilon values out
 * (lib/metal_dispatch_linear.ml:252-396).  values = [activation; residual; gateW; gateS;
 * upW; upS; downW; downS; norm_weight]; three launches. */
int llmopt_op_w4a16_swiglu_ffn(llmopt_op_context *context, int64_t m, int64_t n, int64_t k,
                               double epsilon, const llmopt_op_value *values, size_t value_count,
                               const llmopt_op_value *output);

/* dispatch_w4a16_lm_head_argmax_command ctx st ~m ~n ~k ~epsilon ~extra_outputs values out
 * (lib/metal_dispatch_linear.ml:570-721).  values = [input; norm_weight; weight; scale];
 * output = token ids [m]; at most one extra output (logits f16 [m, n]). */
int llmopt_op_w4a16_lm_head_argmax(llmopt_op_context *context, int64_t m, int64_t n, int64_t k,
                                   double epsilon, const llmopt_op_value *values, size_t value_count,
                                   const llmopt_op_value *output,
                                   const llmopt_op_value *extra_outputs, size_t extra_count);

/* Ir.Paged_attention_q8 config (lib/ir.ml) as dispatch_paged_attention_q8 reads it. */
typedef struct llmopt_op_paged_attention_config {
  int64_t token_elements, key_offset, value_offset, group_size, token_stride;
  double scale;
  int64_t window; /* 0 = none */
} llmopt_op_paged_attention_config;

/* dispatch_paged_attention_q8 ctx st ~config ~query ~current_key ~current_value ~pool ~slots
 * ~mask_values ~output (lib/metal_dispatch_attention.ml:104-217).  past_length is the
 * length of `slots`; mask_count is 0 or 1. */
int llmopt_op_paged_attention_q8(llmopt_op_context *context,
                                 const llmopt_op_paged_attention_config *config,
                                 const llmopt_op_value *query, const llmopt_op_value *current_key,
                                 const llmopt_op_value *current_value, const llmopt_op_value *pool,
                                 const llmopt_op_value *slots, const llmopt_op_value *mask_values,
                                 size_t mask_count, const llmopt_op_value *output);

/* ---- pure helpers (no GPU) --------------------------------------------------- */

/* Paged_attention_tactic.kernel_name (lib/metal_dispatch_common.ml:41-57). */
/* dispatch_attention ctx st ~config ~query ~key ~value ~mask ~output
 * (lib/metal_dispatch_attention.ml:6-102): dense fp16 attention (prefill).  query [b,h,q,d],
 * key [b,kvh,L,d], value [b,kvh,L,d] or [b,L,kvh,d], mask NULL or [mb,mh,q,L] (BOOL or F16),
 * output [b,h,q,d], [b,q,h,d] or [b,q,h*d]; past_length = max(0, L - q). */
int llmopt_op_attention(llmopt_op_context *context, double scale, int causal,
                        const llmopt_op_value *query, const llmopt_op_value *key,
                        const llmopt_op_value *value, const llmopt_op_value *mask,
                        const llmopt_op_value *output);

const char *llmopt_op_paged_attention_kernel_name(int experimental_gqa3_split8, int split8,
                                                  int64_t query_heads, int64_t kv_heads,
                                                  int64_t head_dimension);
/* linear_f16_grid / simd_rows_grid (lib/metal_dispatch_common.ml:64-80): -1 on overflow. */
int64_t llmopt_op_linear_f16_grid(int64_t columns);
int64_t llmopt_op_simd_rows_grid(int64_t rows);
/* Parameters.paged_attention_q8 (lib/metal_parameters.ml:119-140): writes 64 bytes. */
int llmopt_op_parameters_paged_attention_q8(uint8_t out[64], int64_t batches, int64_t query_heads,
                                            int64_t kv_heads, int64_t past_length,
                                            int64_t head_dimension, int64_t mask_batches,
                                            int64_t mask_heads, int64_t token_elements,
                                            int64_t key_offset, int64_t value_offset,
                                            int64_t group_size, int64_t token_stride, double scale,
                                            int64_t mask_dtype, int64_t query_length, int64_t window);
/* Kv_cache.Format.bytes_for_elements (lib/kv_cache.ml:16-21): `elements` int8 values plus one
 * f16 scale per group of 64 (the last group may be partial); -1 for a negative count or on
 * overflow (the reference raises Invalid_argument). */
int64_t llmopt_op_kv_bytes_for_elements(int64_t elements);

/* Kv_cache.Layout.Attention_layer (lib/kv_cache.ml:27-42) and the region Layout.create_heterogeneous
 * gives it (lib/kv_cache.ml:44-50,126-152). */
typedef struct llmopt_op_kv_layer {
  int64_t kv_heads, head_dim;
} llmopt_op_kv_layer;
typedef struct llmopt_op_kv_region {
  int64_t key_offset, value_offset, segment_elements, segment_bytes;
} llmopt_op_kv_region;
/* Kv_cache.Layout.create_heterogeneous for attention layers (lib/kv_cache.ml:80-166): every
 * token's pool slot holds each layer's keys, then its values, layers side by side, then all
 * f16 group scales.  Writes the per-layer regions (regions may be NULL), token_elements and
 * bytes_per_token (the slot stride).  Same checks and messages: positive kv_heads / head_dim,
 * "Q8 KV group_size must divide each attention head dimension", "... overflows". */
int llmopt_op_kv_layout(const llmopt_op_kv_layer *layers, size_t layer_count, llmopt_op_kv_region *regions,
                        int64_t *token_elements, int64_t *bytes_per_token);

/* Kernel_abi.Operation.to_string of an entry name this library implements
 * (lib/kernel_abi.ml:37-70), NULL for an unknown name. */
const char *llmopt_op_kernel_operation(const char *kernel_name);

#ifdef __cplusplus
}
#endif

#endif /* LLMOPT_HIP_OPS_H */
