// Host-visible launch interface of the HIP kernels.  Plain structs and raw
// device pointers; every launcher is asynchronous on the given stream and
// assumes the caller has validated shapes and buffer sizes.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llmopt {

// One packed W4 matrix: weight u8 [n, k/2] row-major, scale f16 [n, k/64].
struct W4Matrix {
  const uint8_t *weight;
  const uint16_t *scale;
};

// y[r, c] = half(sum_k x[r,k] * q[c,k] * s[c,k/64] (+ addend[r*addend_row_stride + c]))
// Semantics of llmopt_w4a16_linear_f16_g64{,_m4,_m8}
// (lib/metal_w4a16_source.ml:8-194): addend is a bias when the stride is 0 and a
// residual when it is n.
struct W4LinearArgs {
  const uint16_t *x;  // f16 [m, k]
  W4Matrix w;
  const uint16_t *addend;  // may be null when has_addend == 0
  uint32_t has_addend;
  uint32_t addend_row_stride;
  uint16_t *y;  // f16 [m, n]; may be null when only y_f32 is wanted
  uint32_t m, n, k;
  // Optional float32 copy of the output before rounding to half (decode path
  // only, m <= kGemvMaxRows): the LM head takes its argmax over these.
  float *y_f32;
  // Optional scratch for the decode path when m x k exceeds the LDS budget and the
  // K range is split over workgroups: fp32 partial sums and one arrival counter per
  // 16-row tile (zero before the first launch; the kernel leaves them zero).
  void *workspace;
  size_t workspace_bytes;
  uint32_t *counters;
  uint32_t counter_count;
};

// Bytes of workspace the decode path wants for this shape (0 when it does not split K).
size_t w4a16_gemv_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);
// The same for the prefill GEMM (m > kGemvMaxRows), which splits K over workgroups when its
// tiles would leave half the CUs idle; without the workspace and the counters it does not split.
size_t w4a16_gemm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);

// Optional RMS normalisation of the activation rows on their way into a decode kernel
// (weight == nullptr: none): the kernel multiplies by half(x * gain * r) (weight_first) or
// half(x * r * gain), r = rsqrt(mean(x^2) + epsilon) in float32 - the values
// llmopt_rms_norm_f16_simd / llmopt_w4a16_swiglu_rms_f16_g64 would have written for it to read.
// Only where w4a16_norm_in_kernel() says so.
struct W4Norm {
  const uint16_t *weight;  // f16 [k]
  float epsilon;
  uint32_t weight_first;
};
// True when launch_w4a16_qkv / launch_w4a16_dual_swiglu with these sizes run a kernel that can
// normalise its activation itself (`columns` = all outputs of the launch).
bool w4a16_norm_in_kernel(uint32_t m, uint64_t columns, uint32_t k);

// Three projections of one activation in one launch
// (llmopt_w4a16_qkv_linear_f16_g64*, lib/metal_w4a16_source.ml:218-480).
struct W4QkvArgs {
  const uint16_t *x;  // f16 [m, k]
  W4Matrix w[3];
  uint16_t *y[3];  // f16 [m, n[i]]
  uint32_t n[3];
  uint32_t m, k;
  W4Norm norm;
};

// product[r, c] = half(silu(gate[r,c]) * up[r,c]) with gate, up fp32
// (llmopt_w4a16_dual_swiglu_f16_g64*, lib/metal_w4a16_source.ml:533-577).
struct W4DualSwigluArgs {
  const uint16_t *x;  // f16 [m, k]
  W4Matrix gate, up;  // each [n, k/2]
  uint16_t *product;  // f16 [m, n]
  uint32_t m, n, k;
  W4Norm norm;
};

hipError_t launch_w4a16_linear(const W4LinearArgs &args, hipStream_t stream);
hipError_t launch_w4a16_qkv(const W4QkvArgs &args, hipStream_t stream);
hipError_t launch_w4a16_dual_swiglu(const W4DualSwigluArgs &args, hipStream_t stream);

// ---- fused decode-step launches (no reference kernels; small activations: k <= 2048) ----------
//
// A decode step at small batch is bound by the number of its launches, not by their bytes: these
// kernels do in one launch what several reference kernels do in a row, with the same arithmetic
// at every rounding point.

// The residual stream of a layer arrives as x plus, when partial_count != 0, the pending partial
// sums of the previous layer's down projection: row r of the stream is
// half(sum_p partials[p][r][:] (p ascending, float32) + float(x[r][:])), the value
// llmopt_w4a16_down_add_f16_g64 would have stored.  Every workgroup forms the rows it needs; the
// first writes them to x_out (may be null).
struct FusedResidual {
  const uint16_t *x;      // f16 [m, k]
  const float *partials;  // f32 [partial_count, m, k], may be null when partial_count == 0
  uint32_t partial_count;
  uint16_t *x_out;        // f16 [m, k]
};
// (and at most 32 per thread of the reader: a reader whose rows leave it one group of threads takes 32)
constexpr uint32_t kFusedMaxPartials = 48;
constexpr uint32_t kFusedMaxWidth = 2048;

// llmopt_rms_norm_f16_simd + llmopt_w4a16_qkv_linear_f16_g64 + llmopt_rotary_qk_f16_simd_h64 +
// llmopt_cache_pack_attention_q8_pair_simd for one new token per sequence, heads of 64: a
// workgroup owns one head of one sequence - both halves of every rotation pair and the whole
// Q8 group - so nothing is handed over between workgroups.
struct FusedQkvArgs {
  FusedResidual in;
  W4Norm norm;              // weight_first = 0
  W4Matrix w[3];            // q, k, v
  uint32_t n[3];            // multiples of 64
  const uint16_t *cosine, *sine;  // f16 [m, 64]
  uint16_t *q_out, *k_out;  // rotated, f16 [m, n[0]], [m, n[1]]
  uint16_t *v_out;          // f16 [m, n[2]]
  const uint32_t *slots;    // [m]: pool slot of every sequence's new token
  uint8_t *pool;
  uint32_t m, k;
  uint32_t key_offset, value_offset, token_elements, token_stride;
};
bool fused_qkv_ok(const FusedQkvArgs &args);
hipError_t launch_fused_qkv(const FusedQkvArgs &args, hipStream_t stream);

// llmopt_w4a16_swiglu_rms_f16_g64 + llmopt_w4a16_dual_swiglu_f16_g64 + the contraction of
// llmopt_w4a16_down_add_f16_g64: workgroup j owns the 64 intermediate columns [64 j, 64 j + 64),
// computes product = half(silu(gate) * up) for them and multiplies it into the down projection's
// partial sum over those 64 columns, partials[j][r][:] (float32, scale applied).  The sums over j
// and the residual are taken by the launch that reads the stream next (FusedResidual).
struct FusedFfnArgs {
  FusedResidual in;    // the stream: rows plus pending partial sums (e.g. of the projecting attention merge)
  W4Norm norm;         // weight_first = 1
  W4Matrix gate, up;   // [n, k/2]
  W4Matrix down;       // [k, n/2]
  float *partials;     // f32 [n / slice, m, k]
  uint32_t m, n, k;
  uint32_t slice = 64;  // columns of the intermediate per workgroup and partial sum: 64 or 32
};
// pending: the input arrives with partial sums to add (their staging takes 8 KiB of the workgroup's memory)
bool fused_ffn_ok(uint32_t m, uint32_t n, uint32_t k, bool pending = false, uint32_t slice = 64);
hipError_t launch_fused_ffn(const FusedFfnArgs &args, hipStream_t stream);

// The product kernels' own nibble decoders run over a whole matrix, as float32 [n, k]:
// decoder 0 = w4_decode_pairs and 1 = w4_decode_biased (minus its bias), each times the float32
// scale, i.e. the exact q * s of python/llmopt_backend/quantization.py:91-121; decoder 2 = the
// prefill GEMM's staged operand half(q * s) (one fp16 rounding).
hipError_t launch_w4_dequant_f32(const W4Matrix &w, float *out, uint32_t n, uint32_t k, uint32_t decoder,
                                 hipStream_t stream);
// The attention kernels' int8 decoders over `count` bytes (a multiple of 4), as float32:
// decoder 0 = int8x4_to_h2, 1 = int8x4_to_h2_biased minus its bias.
hipError_t launch_q8_decode_f32(const uint8_t *bytes, float *out, uint32_t count, uint32_t decoder,
                                hipStream_t stream);

// ---- grouped-Q8 KV cache -----------------------------------------------------

// AttentionCacheParams / AttentionCachePairParams
// (lib/metal_cache_source.ml:9-34).  For the single-segment kernels only
// source[0] / segment_offset[0] are used; the pair kernel packs K and V.
struct Q8PackArgs {
  const uint16_t *source[2];  // f16 head-major [heads, source_items, head_dim]
  const uint32_t *slots;      // [items]
  uint8_t *pool;
  uint32_t items;
  uint32_t segment_offset[2];
  uint32_t heads, head_dim;
  uint32_t token_elements, token_stride;
  uint32_t source_items, source_offset;
  // Extension for batched decode: the sources are [items, heads, head_dim]
  // (one new token per sequence, as the K/V projections leave them) instead of
  // head-major; source_items / source_offset are then unused.
  uint32_t item_major;
};

struct Q8UnpackArgs {
  const uint8_t *pool;
  const uint32_t *slots;
  uint16_t *destination;  // f16 head-major [heads, items, head_dim]
  uint32_t items;
  uint32_t segment_offset;
  uint32_t heads, head_dim;
  uint32_t token_elements, token_stride;
};

hipError_t launch_q8_pack(const Q8PackArgs &args, bool pair, hipStream_t stream);
hipError_t launch_q8_unpack(const Q8UnpackArgs &args, hipStream_t stream);

// llmopt_cache_{pack,unpack}_checkpoint_q8* (lib/metal_cache_source.ml:245-343,
// CheckpointCacheParams :36-44): one layer's flat f16 state of layer_elements values to or from
// checkpoint slot `checkpoint` of a pool of checkpoint_stride-byte slots, the same group-64
// quantiser as the attention cache (int8 values of all layers, then their f16 scales).
// device_checkpoint, when not null, holds the slot index instead (a retained plan writes it per
// step); it is held to max_checkpoint, the last slot the pool has room for.
struct Q8CheckpointArgs {
  const uint16_t *source;  // pack
  uint16_t *destination;   // unpack
  uint8_t *pool;
  const uint32_t *device_checkpoint;
  uint32_t checkpoint, max_checkpoint, layer, layer_elements, checkpoint_elements, checkpoint_stride;
};
hipError_t launch_q8_checkpoint_pack(const Q8CheckpointArgs &args, hipStream_t stream);
hipError_t launch_q8_checkpoint_unpack(const Q8CheckpointArgs &args, hipStream_t stream);

// Q8PagedAttentionParams (lib/metal_cache_source.ml:352-369) plus the
// per-sequence extension: when past_lengths is not null, sequence b attends to
// past_lengths[b] pool tokens whose slot indices start at
// slots[slot_offsets[b]]; otherwise all sequences share slots[0..past_length)
// as in the reference kernels (:391,:429).
struct Q8AttentionArgs {
  const uint16_t *query;          // f16 [b, h, q, D]
  const uint16_t *current_key;    // f16 [b, kvh, q, D]
  const uint16_t *current_value;  // f16 [b, kvh, q, D]
  const uint8_t *pool;
  size_t pool_bytes;  // 0 if unknown; below 4 GiB enables 32-bit slot offsets
  const uint32_t *slots;
  const uint8_t *mask;  // may be null
  uint16_t *output;     // f16 token-major [b, q, h, D]
  const uint32_t *past_lengths;  // extension, may be null
  const uint32_t *slot_offsets;  // extension, may be null
  uint32_t batches, query_heads, kv_heads, past_length, head_dim;
  uint32_t mask_batches, mask_heads, token_elements, key_offset, value_offset;
  uint32_t token_stride;
  float scale;
  uint32_t query_length, mask_dtype, window;
  uint32_t max_past_length;  // >= every past length (bounds the split grid)
  void *workspace;           // split-context partials
  size_t workspace_bytes;
  // Optional (no reference kernel; split-context launches with heads of 64 only, see
  // q8_attention_can_project): instead of storing the output rows, every (sequence, head) row -
  // rounded to half, as it would have been stored - is multiplied into that head's 64 columns of the
  // W4 output projection `projection` [projected_width, query_heads * 64 / 2], and the float32
  // partial sums go to projected[head][sequence][projected_width] (group scale applied).  The sum over
  // heads and the residual are taken by the launch that reads the stream next (FusedResidual);
  // `output` may then be null.
  W4Matrix projection = {nullptr, nullptr};
  float *projected = nullptr;
  uint32_t projected_width = 0;
};
// True when launch_q8_attention can take args.projected for these arguments.
bool q8_attention_can_project(const Q8AttentionArgs &args);

// The longest context the split-context kernels take (longer ones run the row-serial kernel).
constexpr uint32_t kQ8AttentionSplitTokens = 128 * 1024;
// Bytes of workspace launch_q8_attention needs for these arguments (0 when the
// row-serial kernel is used).
size_t q8_attention_workspace_bytes(const Q8AttentionArgs &args);
hipError_t launch_q8_attention(const Q8AttentionArgs &args, hipStream_t stream);

// ---- dense fp16 attention -------------------------------------------------------

// llmopt_attention_f16 / llmopt_attention_f16_simd_h<D>
// (lib/metal_attention_source.ml:239-347; AttentionParams :251-256).
struct DenseAttentionArgs {
  const uint16_t *query;  // f16 [b, h, q, D]
  const uint16_t *key;    // f16 [b, kvh, L, D]
  const uint16_t *value;  // f16 [b, kvh, L, D], or [b, L, kvh, D] with token_first_value
  const uint8_t *mask;    // [mb, mh, q, L] bool or f16; null or mask_batches == 0: none
  uint16_t *output;       // f16 [b, h, q, D], or [b, q, h, D] with token_first_output
  uint32_t batches, heads, query_length, key_length, head_dim, mask_batches, mask_heads, causal;
  float scale;
  uint32_t kv_heads, token_first_output, past_length, token_first_value, mask_dtype;
  uint32_t cus_per_xcd = 0;  // set by the launcher (workgroup order of the causal launch)
  // Scratch for masked launches (may be null: every stage of keys is then walked): one byte per
  // (mask batch, mask head, slab of query rows, stage of keys) that says whether the mask allows
  // anything there, written by a pass over the mask ahead of the attention kernel.
  uint8_t *stage_map = nullptr;
  size_t stage_map_bytes = 0;
  // Set by the launcher: the same pass also leaves the mask as one bit per (mask row, key) behind the
  // map, mask_words_per_row dwords a row, which is what the attention kernel then reads.
  const uint32_t *mask_bits = nullptr;
  uint32_t mask_words_per_row = 0;
};
size_t dense_attention_workspace_bytes(const DenseAttentionArgs &args);
hipError_t launch_dense_attention(const DenseAttentionArgs &args, hipStream_t stream);

// The mask of llmopt_attention_tree_speculative_f16 (llmopt_speculative_tree_allowed,
// lib/metal_attention_source.ml:361-381) as bytes [query_length, key_length]: every key before
// past_length is visible; draft key i (key past_length + i, i < query_length) is visible to query
// token q when bit i of tree_masks[q] is set (q < 8; later query tokens see the past only).
hipError_t launch_tree_mask(uint8_t *mask, uint32_t query_length, uint32_t key_length, uint32_t past_length,
                            const uint32_t tree_masks[8], hipStream_t stream);

// ---- decode glue ---------------------------------------------------------------

// out[row, i] = half(x[row, i] * rsqrt(mean(x[row]^2) + eps) * w[i]), one wave per row.
// weight_first selects the fp32 product order of llmopt_w4a16_swiglu_rms_*
// (x * w * inverse, lib/metal_w4a16_source.ml:525) instead of that of
// llmopt_rms_norm_f16_simd (x * inverse * w, lib/metal_normalization_source.ml:90).
struct RmsNormArgs {
  const void *input;  // f16 or f32 [rows, width]
  bool input_f32;
  const uint16_t *weight;  // f16 [width]
  uint16_t *output;        // f16 [rows, width]
  uint32_t rows, width;
  float epsilon;
  bool weight_first;
};
hipError_t launch_rms_norm(const RmsNormArgs &args, hipStream_t stream);
// x * w * inverse kept to float32 accuracy as two fp16 rows per input row: output
// [2 * rows, width], row 2r = half(v), row 2r + 1 = half(v - float(half(v))).
hipError_t launch_rms_norm_split(const RmsNormArgs &args, hipStream_t stream);

// llmopt_rotary_qk_f16_simd_h64 (lib/metal_normalization_source.ml:765-802):
// token-major [b, t, heads, width] in, head-major [b, heads, t, width] out,
// rotate-half with every product and the sum rounded to half.
struct RotaryQkArgs {
  const uint16_t *q_input, *k_input, *cosine, *sine;
  uint16_t *q_output, *k_output;
  uint32_t batches, tokens, q_heads, k_heads, width, half_dimension, trig_batches;
};
hipError_t launch_rotary_qk(const RotaryQkArgs &args, hipStream_t stream);

// The rotation (token-major in, head-major out; one token per sequence in a decode step, a
// prompt's tokens in a prefill) and, in the same launch, the Q8 quantisation of the rotated keys
// and of the values (pack.source[1], token-major) into the pool slot of every (sequence, token);
// pack.item_major is set and pack.items = batches * tokens.  Same arithmetic as the separate launches.
struct RotaryPackArgs {
  RotaryQkArgs rotary;
  Q8PackArgs pack;
};
hipError_t launch_rotary_qk_pack(const RotaryPackArgs &args, hipStream_t stream);

// llmopt_embedding_f16 (lib/metal_tensor_source.ml:306-320): row gather, rows
// outside [0, vocabulary) give zeros.
struct EmbeddingArgs {
  const int64_t *indices;
  const uint16_t *weight;
  uint16_t *output;
  uint32_t tokens, vocabulary, width;
};
hipError_t launch_embedding(const EmbeddingArgs &args, hipStream_t stream);

// PointwiseParams of llmopt_add_f16 (lib/metal_tensor_source.ml:1007-1032): numpy-style
// broadcasting over up to 8 axes, or a scalar operand.
struct PointwiseArgs {
  const uint16_t *left, *right;
  uint16_t *output;
  uint32_t count, rank, left_scalar, right_scalar;
  uint32_t output_shape[8], left_shape[8], right_shape[8];
  float left_f32, right_f32;
};
hipError_t launch_add_f16(const PointwiseArgs &args, hipStream_t stream);

hipError_t launch_copy_bytes(void *destination, const void *source, size_t bytes, hipStream_t stream);
// One small launch that sets a retained plan's per-step state: *token = *chain_from (when not
// null; int32 widened) or `value` (token may be null), and past[0..past_count) = past_value.
hipError_t launch_plan_state(int64_t *token, int64_t value, const int32_t *chain_from, uint32_t *past,
                             uint32_t past_value, uint32_t past_count, uint32_t *checkpoint, uint32_t checkpoint_value,
                             hipStream_t stream);

// Sets *found (device memory) to 1 when [data, data + bytes) holds a NaN, read as fp16 words or
// (f32) as float32 words; leaves it alone otherwise.
hipError_t launch_nan_scan(const void *data, size_t bytes, bool f32, uint32_t *found, hipStream_t stream);

// Argmax over float32 logits [rows, n] in two steps with the reference's
// candidate layout (W4A16LmHeadCandidate {f32 value, u32 index}, 256 per row,
// lib/metal_w4a16_source.ml:1287-1319); ties go to the lowest index.
// pairs: logits is [2 * rows, n], output row r = rows 2r + (2r + 1) (see launch_rms_norm_split);
// half_logits, when not null, receives half(logit) [rows, n].
hipError_t launch_argmax_candidates(const float *logits, void *candidates, uint32_t rows, uint32_t n, bool pairs,
                                    uint16_t *half_logits, hipStream_t stream);
hipError_t launch_argmax_reduce(const void *candidates, uint32_t *token_ids, uint32_t rows,
                                hipStream_t stream);

// The largest m the streaming GEMV path takes; above it the MFMA GEMM runs.
constexpr uint32_t kGemvMaxRows = 8;
// Up to this m the GEMV uses v_dot2 on the vector ALUs, above it the matrix cores.
constexpr uint32_t kGemvDotRows = 2;

}  // namespace llmopt
