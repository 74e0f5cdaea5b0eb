/*
 * CPU oracle for the quantized-inference hot path of tungd/llmopt.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against; nothing in the shipped library links, loads or calls it.
 *
 * It restates, in plain C, the reference's CPU path and the arithmetic its
 * device kernels define where the CPU path has no counterpart:
 *
 *   oracle_w4a16_linear       lib/cpu.ml:128-152          (Cpu.w4a16_linear)
 *   oracle_add                lib/cpu.ml:154-170          (Cpu.add)
 *   oracle_silu / _silu_mul   lib/cpu.ml:226,239          (pointwise)
 *   oracle_attention          lib/cpu.ml:606-717          (Cpu.attention)
 *   oracle_q8_pack            lib/metal_cache_source.ml:46-81   (Q8 quantizer)
 *   oracle_q8_unpack          lib/metal_cache_source.ml:184-211 (Q8 dequant)
 *   oracle_paged_attention_q8 lib/metal_cache_source.ml:382-401 (dequant +
 *                             index arithmetic) and :493-583 (key range, mask,
 *                             window, GQA head map, token-major output),
 *                             evaluated with Cpu.attention's three passes in
 *                             fp64 (lib/cpu.ml:665-716)
 *   oracle_rms_norm           lib/metal_normalization_source.ml:70-91
 *   oracle_rotary_h           lib/metal_normalization_source.ml:765-802
 *   oracle_argmax             lib/metal_w4a16_source.ml:1116-1117 (tie rule)
 *
 * The OCaml original cannot be compiled in this environment (no OCaml
 * toolchain), so there is no build of the reference itself beside this file.
 * Every function here is pinned by the reference's own golden vectors and by
 * exact-arithmetic cross-checks in tests/test_oracle_*.py.
 *
 * Tensors are held as the reference CPU path holds them: float32 arrays
 * (fp16 values are exactly representable), arithmetic in double, results
 * stored back to float32.  Packed bytes are plain uint8_t here; the
 * reference's "byte carried as a float, recovered with Float.round"
 * (lib/cpu.ml:137) is the identity on 0..255.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- fp16 --- */

/* IEEE binary16 -> binary32, exact. */
float oracle_f16_to_f32(uint16_t bits) {
  uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
  uint32_t exponent = (bits >> 10) & 0x1fu;
  uint32_t mantissa = bits & 0x3ffu;
  uint32_t out;
  if (exponent == 0) {
    if (mantissa == 0) {
      out = sign;
    } else {
      int shift = 0;
      while ((mantissa & 0x400u) == 0) {
        mantissa <<= 1;
        shift++;
      }
      mantissa &= 0x3ffu;
      out = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (mantissa << 13);
    }
  } else if (exponent == 31) {
    out = sign | 0x7f800000u | (mantissa << 13);
  } else {
    out = sign | ((exponent + 127 - 15) << 23) | (mantissa << 13);
  }
  float value;
  memcpy(&value, &out, sizeof value);
  return value;
}

/* IEEE binary32 -> binary16, round to nearest even (what `half(x)` does). */
uint16_t oracle_f32_to_f16(float value) {
  uint32_t bits;
  memcpy(&bits, &value, sizeof bits);
  uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
  uint32_t magnitude = bits & 0x7fffffffu;
  if (magnitude >= 0x7f800000u) {
    if (magnitude > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    return (uint16_t)(sign | 0x7c00u);
  }
  if (magnitude >= 0x477ff000u) {
    /* >= 65520 rounds to infinity */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (magnitude < 0x33000001u) {
    /* <= 2^-25 rounds to zero (tie at exactly 2^-25 goes to even = 0) */
    return sign;
  }
  int32_t exponent = (int32_t)(magnitude >> 23) - 127;
  uint32_t mantissa = (magnitude & 0x7fffffu) | 0x800000u;
  uint32_t shift;
  uint32_t half_exponent;
  if (exponent < -14) {
    shift = (uint32_t)(13 + (-14 - exponent));
    half_exponent = 0;
  } else {
    shift = 13;
    half_exponent = (uint32_t)(exponent + 15);
  }
  uint32_t kept = mantissa >> shift;
  uint32_t remainder = mantissa & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (remainder > halfway || (remainder == halfway && (kept & 1u))) kept++;
  uint32_t out;
  if (half_exponent == 0) {
    out = kept; /* subnormal; a carry into 0x400 is the smallest normal */
  } else {
    out = ((half_exponent - 1) << 10) + kept; /* kept carries the hidden bit */
  }
  return (uint16_t)(sign | out);
}

/* ------------------------------------------------------- W4A16 linear --- */

/* lib/cpu.ml:131 */
static int signed_nibble(int nibble) {
  return (nibble & 0x8) == 0 ? nibble : nibble - 16;
}

/* Signed int4 weight at logical (col, inner): low nibble = even K
 * (lib/cpu.ml:139; python/llmopt_backend/quantization.py:72-88). */
int oracle_w4_unpack(const uint8_t *packed, int64_t k, int64_t col,
                     int64_t inner) {
  int byte = packed[col * (k / 2) + inner / 2];
  int nibble = (inner & 1) == 0 ? (byte & 0xF) : ((byte >> 4) & 0xF);
  return signed_nibble(nibble);
}

/* Dequantised logical weight [N,K] in float32: q * scale with both operands
 * promoted to float32 (python/llmopt_backend/quantization.py:110-121).  The
 * product has at most 15 significant bits, so it is exact. */
void oracle_w4_dequant(const uint8_t *packed, const float *scale, float *out,
                       int64_t n, int64_t k) {
  int64_t groups = k / 64;
  for (int64_t col = 0; col < n; col++)
    for (int64_t inner = 0; inner < k; inner++)
      out[col * k + inner] =
          (float)oracle_w4_unpack(packed, k, col, inner) *
          scale[col * groups + inner / 64];
}

/* lib/cpu.ml:128-152.  input [M,K], packed [N,K/2], scale [N,K/64],
 * bias [1,N] or NULL (broadcast over rows only), output [M,N].
 * The accumulator is a double starting at 0.0, terms are added for
 * inner = 0..K-1 in order, each term is (x * weight) * group_scale. */
void oracle_w4a16_linear(const float *input, const uint8_t *packed,
                         const float *scale, const float *bias, float *output,
                         int64_t m, int64_t n, int64_t k) {
  int64_t groups = k / 64;
  for (int64_t row = 0; row < m; row++) {
    for (int64_t col = 0; col < n; col++) {
      double accumulator = 0.0;
      for (int64_t inner = 0; inner < k; inner++) {
        double weight = (double)oracle_w4_unpack(packed, k, col, inner);
        double group_scale = (double)scale[col * groups + inner / 64];
        accumulator += ((double)input[row * k + inner] * weight) * group_scale;
      }
      double value = bias ? accumulator + (double)bias[col] : accumulator;
      output[row * n + col] = (float)value;
    }
  }
}

/* lib/cpu.ml:154-170 with Shape.Same / Shape.Row broadcast: a one-row operand
 * is repeated over rows. */
void oracle_add(const float *left, int64_t left_rows, const float *right,
                int64_t right_rows, float *output, int64_t rows, int64_t cols) {
  for (int64_t row = 0; row < rows; row++) {
    int64_t left_row = left_rows == 1 ? 0 : row;
    int64_t right_row = right_rows == 1 ? 0 : row;
    for (int64_t col = 0; col < cols; col++)
      output[row * cols + col] = (float)((double)left[left_row * cols + col] +
                                         (double)right[right_row * cols + col]);
  }
}

/* lib/cpu.ml:226 */
void oracle_silu(const float *input, float *output, int64_t count) {
  for (int64_t i = 0; i < count; i++) {
    double value = (double)input[i];
    output[i] = (float)(value / (1.0 + exp(-value)));
  }
}

/* lib/cpu.ml:239 */
void oracle_silu_mul(const float *left, const float *right, float *output,
                     int64_t count) {
  for (int64_t i = 0; i < count; i++) {
    double l = (double)left[i];
    double r = (double)right[i];
    output[i] = (float)((l / (1.0 + exp(-l))) * r);
  }
}

/* ----------------------------------------------------------- attention --- */

/* lib/cpu.ml:606-717.  query/output [b,h,q,d], key/value [b,h,L,d] (the
 * reference requires key_heads = heads; a GQA caller expands first),
 * mask [mb,mh,q,L] with nonzero = allowed.  Three passes per row: maximum,
 * denominator, weighted sum.  The reference recomputes score() inside every
 * pass; score() is a pure function, so computing it once per key gives the
 * same doubles. */
void oracle_attention(const float *query, const float *key, const float *value,
                      const float *mask, float *output, int64_t batches,
                      int64_t heads, int64_t query_length, int64_t key_length,
                      int64_t head_dimension, int64_t mask_batches,
                      int64_t mask_heads, double scale, int causal) {
  double *scores = (double *)malloc(sizeof(double) * (size_t)key_length);
  unsigned char *allowed = (unsigned char *)malloc((size_t)key_length);
  for (int64_t batch = 0; batch < batches; batch++) {
    for (int64_t head = 0; head < heads; head++) {
      for (int64_t qp = 0; qp < query_length; qp++) {
        int64_t mask_batch = mask_batches == 1 ? 0 : batch;
        int64_t mask_head = mask_heads == 1 ? 0 : head;
        const float *q_row =
            query + (((batch * heads) + head) * query_length + qp) *
                        head_dimension;
        double maximum = -INFINITY;
        int found = 0;
        for (int64_t kp = 0; kp < key_length; kp++) {
          int64_t mask_index =
              (((mask_batch * mask_heads) + mask_head) * query_length + qp) *
                  key_length +
              kp;
          allowed[kp] = (unsigned char)(mask[mask_index] != 0.0f &&
                                        (!causal || kp <= qp));
          if (!allowed[kp]) continue;
          const float *k_row =
              key + (((batch * heads) + head) * key_length + kp) *
                        head_dimension;
          double accumulator = 0.0;
          for (int64_t d = 0; d < head_dimension; d++)
            accumulator += (double)q_row[d] * (double)k_row[d];
          scores[kp] = accumulator * scale;
          found = 1;
          maximum = fmax(maximum, scores[kp]);
        }
        double denominator = 0.0;
        if (found)
          for (int64_t kp = 0; kp < key_length; kp++)
            if (allowed[kp]) denominator += exp(scores[kp] - maximum);
        float *o_row = output + (((batch * heads) + head) * query_length + qp) *
                                    head_dimension;
        for (int64_t d = 0; d < head_dimension; d++) {
          double result = 0.0;
          if (denominator != 0.0)
            for (int64_t kp = 0; kp < key_length; kp++)
              if (allowed[kp]) {
                double probability = exp(scores[kp] - maximum) / denominator;
                result += probability *
                          (double)value[(((batch * heads) + head) * key_length +
                                         kp) *
                                            head_dimension +
                                        d];
              }
          o_row[d] = (float)result;
        }
      }
    }
  }
  free(scores);
  free(allowed);
}

/* ------------------------------------------------------------ Q8 cache --- */

/* Parameters of one cache segment, as lib/metal_cache_source.ml:9-20. */
typedef struct {
  uint32_t items;          /* tokens to pack/unpack */
  uint32_t segment_offset; /* element offset of this K or V segment in a token */
  uint32_t heads;          /* kv heads of the layer */
  uint32_t head_dim;
  uint32_t group_size; /* 64 */
  uint32_t token_elements;
  uint32_t token_groups;
  uint32_t token_stride; /* bytes per pool slot */
  uint32_t source_items; /* tokens per head in the f16 source */
  uint32_t source_offset;
} oracle_cache_params;

/* lib/metal_cache_source.ml:46-81.  source is head-major f16
 * [heads, source_items, head_dim] given as raw binary16 bits; the arithmetic
 * is float32 throughout: maximum of |x| over the group, stored scale =
 * half(maximum / 127) or 1.0 for an all-zero group, q = clamp(rint(x /
 * float(stored scale)), -127, 127) with rint = round half to even. */
void oracle_q8_pack(const uint16_t *source, const uint32_t *slots,
                    uint8_t *pool, const oracle_cache_params *p) {
  uint32_t groups_per_head = p->head_dim / p->group_size;
  uint32_t segment_groups = p->heads * groups_per_head;
  for (uint32_t item = 0; item < p->items; item++) {
    for (uint32_t local_group = 0; local_group < segment_groups;
         local_group++) {
      uint32_t head = local_group / groups_per_head;
      uint32_t group_in_head = local_group - head * groups_per_head;
      size_t source_base =
          ((size_t)head * p->source_items + p->source_offset + item) *
              p->head_dim +
          (size_t)group_in_head * p->group_size;
      float maximum = 0.0f;
      for (uint32_t i = 0; i < p->group_size; i++)
        maximum =
            fmaxf(maximum, fabsf(oracle_f16_to_f32(source[source_base + i])));
      uint16_t stored_scale =
          oracle_f32_to_f16(maximum == 0.0f ? 1.0f : maximum / 127.0f);
      float scale = oracle_f16_to_f32(stored_scale);
      size_t slot_base = (size_t)slots[item] * p->token_stride;
      int8_t *values = (int8_t *)(pool + slot_base);
      uint8_t *scales = pool + slot_base + p->token_elements;
      uint32_t value_base = p->segment_offset + head * p->head_dim +
                            group_in_head * p->group_size;
      for (uint32_t i = 0; i < p->group_size; i++) {
        float ratio = oracle_f16_to_f32(source[source_base + i]) / scale;
        float rounded = rintf(ratio);
        int quantized = rounded > 127.0f    ? 127
                        : rounded < -127.0f ? -127
                                            : (int)rounded;
        values[value_base + i] = (int8_t)quantized;
      }
      size_t scale_index = p->segment_offset / p->group_size + local_group;
      memcpy(scales + 2 * scale_index, &stored_scale, 2);
    }
  }
}

/* float(int8) * float(f16 scale), lib/metal_cache_source.ml:382-401. */
static float q8_value(const uint8_t *pool, size_t slot_base,
                      uint32_t token_elements, uint32_t group_size,
                      uint32_t head_dim, uint32_t segment_offset,
                      uint32_t kv_head, uint32_t dimension) {
  uint32_t groups_per_head = head_dim / group_size;
  const int8_t *values = (const int8_t *)(pool + slot_base);
  const uint8_t *scales = pool + slot_base + token_elements;
  uint32_t value_index = segment_offset + kv_head * head_dim + dimension;
  uint32_t scale_index = segment_offset / group_size +
                         kv_head * groups_per_head + dimension / group_size;
  uint16_t scale_bits;
  memcpy(&scale_bits, scales + 2 * (size_t)scale_index, 2);
  return (float)values[value_index] * oracle_f16_to_f32(scale_bits);
}

/* lib/metal_cache_source.ml:184-211: head-major f16 destination
 * [heads, items, head_dim] = half(float(q) * float(scale)). */
void oracle_q8_unpack(const uint8_t *pool, const uint32_t *slots,
                      uint16_t *destination, const oracle_cache_params *p) {
  for (uint32_t item = 0; item < p->items; item++)
    for (uint32_t head = 0; head < p->heads; head++)
      for (uint32_t d = 0; d < p->head_dim; d++) {
        float value = q8_value(pool, (size_t)slots[item] * p->token_stride,
                               p->token_elements, p->group_size, p->head_dim,
                               p->segment_offset, head, d);
        destination[((size_t)head * p->items + item) * p->head_dim + d] =
            oracle_f32_to_f16(value);
      }
}

/* The 64-byte parameter block of lib/metal_cache_source.ml:352-369
 * (host builder lib/metal_parameters.ml:119-140). */
typedef struct {
  uint32_t batches;
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t past_length;
  uint32_t head_dim;
  uint32_t mask_batches;
  uint32_t mask_heads;
  uint32_t token_elements;
  uint32_t key_offset;
  uint32_t value_offset;
  uint32_t group_size;
  uint32_t token_stride;
  float scale;
  uint32_t query_length;
  uint32_t mask_dtype; /* 0 none, 1 bool bytes, 2 f16 additive (>= 0 allowed) */
  uint32_t window;
} oracle_paged_params;

/* Decode attention over a Q8 pool: what
 * llmopt_attention_q8_paged_simd_generic (lib/metal_cache_source.ml:493-583)
 * defines, computed in fp64 with Cpu.attention's three passes
 * (lib/cpu.ml:665-716).
 *
 * query f32 [b,h,q,D]; current_key/current_value f32 [b,kvh,q,D];
 * pool bytes; mask raw bytes (bool) or binary16 bits, or NULL;
 * output f32 token-major [b,q,h,D].
 *
 * Extension beyond the reference operator (which shares one slot table and
 * one past_length across the batch, :391,:429): when past_lengths is not
 * NULL, sequence `batch` has past_lengths[batch] past tokens whose slots
 * start at slots[slot_offsets[batch]].  With both NULL the reference
 * behaviour (slots[key_position], params.past_length) is used. */
void oracle_paged_attention_q8(const float *query, const float *current_key,
                               const float *current_value, const uint8_t *pool,
                               const uint32_t *slots, const uint8_t *mask,
                               float *output, const oracle_paged_params *p,
                               const uint32_t *past_lengths,
                               const uint32_t *slot_offsets) {
  uint32_t q_len = p->query_length == 0 ? 1 : p->query_length;
  uint32_t heads_per_kv = p->query_heads / p->kv_heads;
  uint32_t D = p->head_dim;
  uint32_t max_past = p->past_length;
  if (past_lengths)
    for (uint32_t b = 0; b < p->batches; b++)
      if (past_lengths[b] > max_past) max_past = past_lengths[b];
  size_t max_keys = (size_t)max_past + q_len;
  double *scores = (double *)malloc(sizeof(double) * max_keys);
  unsigned char *allowed = (unsigned char *)malloc(max_keys);
  float *value_row = (float *)malloc(sizeof(float) * max_keys * D);
  for (uint32_t batch = 0; batch < p->batches; batch++) {
    uint32_t past = past_lengths ? past_lengths[batch] : p->past_length;
    const uint32_t *seq_slots = slot_offsets ? slots + slot_offsets[batch] : slots;
    for (uint32_t head = 0; head < p->query_heads; head++) {
      uint32_t kv_head = head / heads_per_kv;
      for (uint32_t q_pos = 0; q_pos < q_len; q_pos++) {
        const float *q_row =
            query + (((size_t)batch * p->query_heads + head) * q_len + q_pos) * D;
        size_t current_base =
            ((size_t)batch * p->kv_heads + kv_head) * q_len * D;
        uint32_t key_length = past + q_pos + 1;
        uint32_t first_key = (p->window == 0 || key_length <= p->window)
                                 ? 0
                                 : key_length - p->window;
        double maximum = -INFINITY;
        int found = 0;
        for (uint32_t kp = first_key; kp < key_length; kp++) {
          allowed[kp] = 1;
          if (mask != NULL && p->mask_batches > 0 && p->mask_dtype != 0) {
            uint32_t mask_batch = p->mask_batches == 1 ? 0 : batch;
            uint32_t mask_head = p->mask_heads == 1 ? 0 : head;
            /* the kernel strides the mask by params.past_length + q_len
             * (lib/metal_cache_source.ml:533) */
            size_t mask_key_stride = (size_t)past + q_len;
            size_t mask_index =
                (((size_t)mask_batch * p->mask_heads + mask_head) * q_len +
                 q_pos) *
                    mask_key_stride +
                kp;
            if (p->mask_dtype == 2) {
              uint16_t bits;
              memcpy(&bits, mask + 2 * mask_index, 2);
              allowed[kp] = oracle_f16_to_f32(bits) >= 0.0f;
            } else {
              allowed[kp] = mask[mask_index] != 0;
            }
          }
          if (!allowed[kp]) continue;
          double accumulator = 0.0;
          for (uint32_t d = 0; d < D; d++) {
            float key_value;
            float v;
            if (kp < past) {
              size_t slot_base = (size_t)seq_slots[kp] * p->token_stride;
              key_value = q8_value(pool, slot_base, p->token_elements,
                                   p->group_size, D, p->key_offset, kv_head, d);
              v = q8_value(pool, slot_base, p->token_elements, p->group_size, D,
                           p->value_offset, kv_head, d);
            } else {
              key_value = current_key[current_base + (size_t)(kp - past) * D + d];
              v = current_value[current_base + (size_t)(kp - past) * D + d];
            }
            value_row[(size_t)kp * D + d] = v;
            accumulator += (double)q_row[d] * (double)key_value;
          }
          /* the kernel multiplies by a float32 scale (params.scale) */
          scores[kp] = accumulator * (double)p->scale;
          found = 1;
          maximum = fmax(maximum, scores[kp]);
        }
        double denominator = 0.0;
        if (found)
          for (uint32_t kp = first_key; kp < key_length; kp++)
            if (allowed[kp]) denominator += exp(scores[kp] - maximum);
        float *o_row =
            output + (((size_t)batch * q_len + q_pos) * p->query_heads + head) * D;
        for (uint32_t d = 0; d < D; d++) {
          double result = 0.0;
          if (denominator != 0.0)
            for (uint32_t kp = first_key; kp < key_length; kp++)
              if (allowed[kp])
                result += (exp(scores[kp] - maximum) / denominator) *
                          (double)value_row[(size_t)kp * D + d];
          o_row[d] = (float)result;
        }
      }
    }
  }
  free(scores);
  free(allowed);
  free(value_row);
}

/* ----------------------------------------------------- decode-step glue --- */

/* x * rsqrt(mean(x^2) + eps) * w per row
 * (lib/metal_normalization_source.ml:70-91), in fp64. */
void oracle_rms_norm(const float *input, const float *weight, float *output,
                     int64_t rows, int64_t width, double epsilon) {
  for (int64_t row = 0; row < rows; row++) {
    double sum = 0.0;
    for (int64_t i = 0; i < width; i++) {
      double v = (double)input[row * width + i];
      sum += v * v;
    }
    double inverse = 1.0 / sqrt(sum / (double)width + epsilon);
    for (int64_t i = 0; i < width; i++)
      output[row * width + i] =
          (float)((double)input[row * width + i] * inverse * (double)weight[i]);
  }
}

/* Rotate-half RoPE (lib/metal_normalization_source.ml:765-802):
 * out[c] = x[c]*cos[c] + (c < h ? -x[c+h] : x[c-h]) * sin[c], token-major
 * input [tokens, heads, d] -> head-major output [heads, tokens, d]; cos/sin
 * tables [tokens, d] already duplicated into both halves. */
void oracle_rotary_h(const float *input, const float *cos_table,
                     const float *sin_table, float *output, int64_t tokens,
                     int64_t heads, int64_t d) {
  int64_t h = d / 2;
  for (int64_t t = 0; t < tokens; t++)
    for (int64_t head = 0; head < heads; head++)
      for (int64_t c = 0; c < d; c++) {
        const float *x = input + (t * heads + head) * d;
        double rotated = c < h ? -(double)x[c + h] : (double)x[c - h];
        output[(head * tokens + t) * d + c] =
            (float)((double)x[c] * (double)cos_table[t * d + c] +
                    rotated * (double)sin_table[t * d + c]);
      }
}

/* Index of the maximum; ties go to the lowest index
 * (lib/metal_w4a16_source.ml:1116-1117). */
int64_t oracle_argmax(const float *values, int64_t count) {
  int64_t best = 0;
  for (int64_t i = 1; i < count; i++)
    if (values[i] > values[best]) best = i;
  return best;
}
