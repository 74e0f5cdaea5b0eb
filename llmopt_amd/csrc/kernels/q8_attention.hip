// Grouped-Q8 KV decode attention for gfx950.
//
// Semantics of llmopt_attention_q8_paged_simd_{generic,h64,h64_gqa3,h256,h512,
// h64_split8,h64_gqa3_split8} (lib/metal_cache_source.ml:352-1247): past keys
// and values are int8 with one fp16 scale per 64-wide head_dim group, read from
// pool slots; the current token's K/V are fp16; softmax in fp32; output fp16,
// token-major [b, q, h, D].
//
// Two kernels:
//
//  * q8_attention_split_kernel (decode fast path: one query token, no mask, no
//    window, D in {64,128}, up to 16 query heads per KV head).  HBM-bound: the
//    context is split into chunks across workgroups, every KV byte is read once
//    per KV head and shared by all query heads of the group through the MFMA
//    column dimension.  int8 -> exact fp16 integers in registers; the fp16
//    group scales are applied in fp32 (K: on the score tile, V: on the
//    probability tile), never folded into fp16 operands.  Partials
//    (max, denominator, O) go to a workspace and q8_attention_merge_kernel
//    folds them together with the current token.
//
//  * q8_attention_rows_kernel: one wave per (batch, head, query position) row,
//    serial over keys with an online softmax.  Covers everything else (mask,
//    window, several query tokens, other head sizes).
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int kSplitThreads = 256;
constexpr int kSplitWaves = 4;
constexpr int kChunkTokens = 256;  // tokens per workgroup
constexpr int kTileTokens = 16;    // tokens per MFMA tile

__device__ __forceinline__ float q8_scale_at(const uint8_t *token, uint32_t token_elements,
                                             uint32_t index) {
  return half_bits_to_float(reinterpret_cast<const uint16_t *>(token + token_elements)[index]);
}

// 4 int8 (already XOR 0x80 -> q + 128) to two h2 of exact integers (b0,b1),(b2,b3).
__device__ __forceinline__ void int8x4_to_h2(uint32_t biased, h2_t &lo, h2_t &hi) {
  const h2_t offset = {(_Float16)1152.0f, (_Float16)1152.0f};  // 1024 + 128
  lo = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04010400u)) - offset;
  hi = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04030402u)) - offset;
}

__device__ __forceinline__ float shfl_xor_f32(float value, int mask) {
  const int lane = __lane_id();
  return __builtin_bit_cast(
      float, __builtin_amdgcn_ds_bpermute(((lane ^ mask) << 2), __builtin_bit_cast(int, value)));
}

struct SplitPartial {
  // layout in the workspace per (batch, kv_head, chunk):
  //   float max[16]; float denominator[16]; float out[G][D];
};

template <int D>
__device__ __forceinline__ size_t partial_floats(uint32_t heads_per_kv) {
  return 32 + (size_t)heads_per_kv * D;
}

template <int D>
__global__ __launch_bounds__(kSplitThreads) void q8_attention_split_kernel(Q8AttentionArgs a,
                                                                           uint32_t chunks_max) {
  constexpr int GROUPS = D / 64;      // scale groups per head
  constexpr int KLOADS = GROUPS;      // 16-byte K loads per lane per tile
  constexpr int VBLOCKS = D / 16;     // PV MFMAs (16 head_dim rows each)
  __shared__ float merge_lds[kSplitWaves][32 + 16 * D];

  const uint32_t chunk = blockIdx.x;
  const uint32_t kv_head = blockIdx.y;
  const uint32_t batch = blockIdx.z;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t col = lane & 15;  // query head within the group / token / d-row
  const uint32_t quad = lane >> 4;
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;

  const uint32_t past = a.past_lengths ? a.past_lengths[batch] : a.past_length;
  const uint32_t chunk_begin = chunk * kChunkTokens;
  if (chunk_begin >= past) return;  // whole workgroup (uniform)
  const uint32_t *slots = a.slot_offsets ? a.slots + a.slot_offsets[batch] : a.slots;
  const uint32_t last_token = past - 1;

  // B operand of the score MFMAs: Q[head = col][d], zero for columns >= G.
  h8_t q_frag[GROUPS][2];
  {
    const uint16_t *q_row =
        a.query + ((size_t)batch * a.query_heads + kv_head * heads_per_kv + col) * D;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (col < heads_per_kv)
          raw = *reinterpret_cast<const uint4 *>(q_row + g * 64 + quad * 16 + j * 8);
        q_frag[g][j] = __builtin_bit_cast(h8_t, raw);
      }
  }

  const uint32_t key_base = a.key_offset + kv_head * D;
  const uint32_t value_base = a.value_offset + kv_head * D;
  const uint32_t key_scale_index = (a.key_offset >> 6) + kv_head * GROUPS;
  const uint32_t value_scale_index = (a.value_offset >> 6) + kv_head * GROUPS;

  float running_max = -INFINITY;  // per head (column), identical in the 4 quads
  float running_sum = 0.0f;       // per lane: this quad's tokens only
  f4_t out_acc[VBLOCKS];
#pragma unroll
  for (int v = 0; v < VBLOCKS; ++v) out_acc[v] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // waves interleave 16-token tiles of the chunk
  for (uint32_t tile = wave; tile < kChunkTokens / kTileTokens; tile += kSplitWaves) {
    const uint32_t token0 = chunk_begin + tile * kTileTokens;
    if (token0 >= past) break;  // wave-uniform

    // ---- K: lane (token = col, quad) holds 16 head_dim values per group ----
    const uint32_t key_token = min(token0 + col, last_token);
    const uint8_t *key_slot = a.pool + (size_t)slots[key_token] * a.token_stride;
    u32x4_t k_raw[KLOADS];
#pragma unroll
    for (int g = 0; g < KLOADS; ++g)
      k_raw[g] = *reinterpret_cast<const u32x4_t *>(key_slot + key_base + g * 64 + quad * 16);

    // ---- V and scales: lane (d-row = col, quad) holds tokens quad*4 + i ----
    uint32_t v_raw[4][GROUPS];
    float k_scale[4][GROUPS], v_scale[4][GROUPS];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t token = min(token0 + quad * 4 + i, last_token);
      const uint8_t *slot = a.pool + (size_t)slots[token] * a.token_stride;
#pragma unroll
      for (int g = 0; g < GROUPS; ++g) {
        v_raw[i][g] = *reinterpret_cast<const uint32_t *>(slot + value_base + g * 64 + col * 4);
        k_scale[i][g] = q8_scale_at(slot, a.token_elements, key_scale_index + g);
        v_scale[i][g] = q8_scale_at(slot, a.token_elements, value_scale_index + g);
      }
    }

    // ---- scores S^T[token][head] = sum_g k_scale[token][g] * (K_g . Q_g) ----
    f4_t score = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      f4_t part = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        h2_t h0, h1, h2, h3;
        int8x4_to_h2(k_raw[g][2 * j] ^ 0x80808080u, h0, h1);
        int8x4_to_h2(k_raw[g][2 * j + 1] ^ 0x80808080u, h2, h3);
        const h8_t k_frag = {h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(k_frag, q_frag[g][j], part, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) score[i] = fmaf(part[i], k_scale[i][g], score[i]);
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool valid = token0 + quad * 4 + i < past;
      score[i] = valid ? score[i] * a.scale : -INFINITY;
      tile_max = fmaxf(tile_max, score[i]);
    }
    tile_max = fmaxf(tile_max, shfl_xor_f32(tile_max, 16));
    tile_max = fmaxf(tile_max, shfl_xor_f32(tile_max, 32));
    // the first token of the tile is valid, so tile_max is finite
    const float new_max = fmaxf(running_max, tile_max);
    const float alpha = __expf(running_max - new_max);  // exp(-inf) = 0 on the first tile
    running_max = new_max;

    float p[4];
    float tile_sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = __expf(score[i] - new_max);
      tile_sum += p[i];
    }
    running_sum = running_sum * alpha + tile_sum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int v = 0; v < VBLOCKS; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) out_acc[v][i] *= alpha;
    }

    // ---- O^T[d][head] += V^T[d][token] * (p * v_scale)[token][head] ----
    // 4x4 byte transposes turn "4 tokens x 4 head_dim" dwords into
    // "4 head_dim x 4 tokens" MFMA A operands.
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      h4_t p_frag;
#pragma unroll
      for (int i = 0; i < 4; ++i) p_frag[i] = (_Float16)(p[i] * v_scale[i][g]);
      const uint32_t a0 = v_raw[0][g] ^ 0x80808080u, a1 = v_raw[1][g] ^ 0x80808080u;
      const uint32_t a2 = v_raw[2][g] ^ 0x80808080u, a3 = v_raw[3][g] ^ 0x80808080u;
      const uint32_t t01_lo = __builtin_amdgcn_perm(a1, a0, 0x05010400u);
      const uint32_t t01_hi = __builtin_amdgcn_perm(a1, a0, 0x07030602u);
      const uint32_t t23_lo = __builtin_amdgcn_perm(a3, a2, 0x05010400u);
      const uint32_t t23_hi = __builtin_amdgcn_perm(a3, a2, 0x07030602u);
      const uint32_t c[4] = {__builtin_amdgcn_perm(t23_lo, t01_lo, 0x05040100u),
                             __builtin_amdgcn_perm(t23_lo, t01_lo, 0x07060302u),
                             __builtin_amdgcn_perm(t23_hi, t01_hi, 0x05040100u),
                             __builtin_amdgcn_perm(t23_hi, t01_hi, 0x07060302u)};
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        h2_t lo, hi;
        int8x4_to_h2(c[jj], lo, hi);
        const h4_t v_frag = {lo[0], lo[1], hi[0], hi[1]};
        out_acc[g * 4 + jj] =
            __builtin_amdgcn_mfma_f32_16x16x16f16(v_frag, p_frag, out_acc[g * 4 + jj], 0, 0, 0);
      }
    }
  }

  // ---- merge the 4 waves, write one partial per (batch, kv_head, chunk) ----
  // out_acc[g*4+jj][i] is O[head = col][d = g*64 + 4*(quad*4 + i) + jj].
  running_sum += shfl_xor_f32(running_sum, 16);
  running_sum += shfl_xor_f32(running_sum, 32);
  float *mine = merge_lds[wave];
  if (quad == 0) {
    mine[col] = running_max;
    mine[16 + col] = running_sum;
  }
#pragma unroll
  for (int v = 0; v < VBLOCKS; ++v)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t d = (v >> 2) * 64 + 4 * (quad * 4 + i) + (v & 3);
      mine[32 + col * D + d] = out_acc[v][i];
    }
  __syncthreads();

  float *partial = reinterpret_cast<float *>(a.workspace) +
                   (((size_t)batch * a.kv_heads + kv_head) * chunks_max + chunk) *
                       partial_floats<D>(heads_per_kv);
  for (uint32_t index = threadIdx.x; index < heads_per_kv * D; index += kSplitThreads) {
    const uint32_t head = index / D;
    float best = -INFINITY;
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w) best = fmaxf(best, merge_lds[w][head]);
    float sum = 0.0f, value = 0.0f;
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w) {
      const float wave_max_value = merge_lds[w][head];
      const float weight = wave_max_value == -INFINITY ? 0.0f : __expf(wave_max_value - best);
      sum += merge_lds[w][16 + head] * weight;
      value += merge_lds[w][32 + index] * weight;
    }
    partial[32 + index] = value;
    if (index == head * D) {
      partial[head] = best;
      partial[16 + head] = sum;
    }
  }
}

// One workgroup of D threads per (batch, query head): folds the chunk partials
// and the current token (fp16 K/V) into the output row.
template <int D>
__global__ __launch_bounds__(D) void q8_attention_merge_kernel(Q8AttentionArgs a,
                                                               uint32_t chunks_max) {
  __shared__ float reduce_lds[D / 64];
  const uint32_t head = blockIdx.x;
  const uint32_t batch = blockIdx.y;
  const uint32_t d = threadIdx.x;
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;
  const uint32_t kv_head = head / heads_per_kv;
  const uint32_t local_head = head - kv_head * heads_per_kv;
  const uint32_t past = a.past_lengths ? a.past_lengths[batch] : a.past_length;
  const uint32_t chunks = (past + kChunkTokens - 1) / kChunkTokens;

  // score of the current token
  const float q = half_bits_to_float(a.query[((size_t)batch * a.query_heads + head) * D + d]);
  const size_t current = ((size_t)batch * a.kv_heads + kv_head) * D + d;
  float dot = wave_sum(q * half_bits_to_float(a.current_key[current]));
  if ((d & 63) == 0) reduce_lds[d >> 6] = dot;
  __syncthreads();
  float score = 0.0f;
#pragma unroll
  for (int w = 0; w < D / 64; ++w) score += reduce_lds[w];
  score *= a.scale;

  float best = score;
  float denominator = 1.0f;
  float value = half_bits_to_float(a.current_value[current]);
  const float *partial = reinterpret_cast<const float *>(a.workspace) +
                         ((size_t)batch * a.kv_heads + kv_head) * chunks_max *
                             partial_floats<D>(heads_per_kv);
  for (uint32_t c = 0; c < chunks; ++c, partial += partial_floats<D>(heads_per_kv)) {
    const float chunk_max = partial[local_head];
    const float chunk_sum = partial[16 + local_head];
    const float chunk_value = partial[32 + local_head * D + d];
    const float new_best = fmaxf(best, chunk_max);
    const float keep = __expf(best - new_best);
    const float take = __expf(chunk_max - new_best);
    denominator = denominator * keep + chunk_sum * take;
    value = value * keep + chunk_value * take;
    best = new_best;
  }
  a.output[((size_t)batch * a.query_heads + head) * D + d] = float_to_half_bits(value / denominator);
}

// ---- row-serial kernel (every other configuration) ---------------------------

constexpr int kMaxFragments = 8;  // head_dim <= 512

__global__ __launch_bounds__(256) void q8_attention_rows_kernel(Q8AttentionArgs a) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const uint32_t rows = a.batches * a.query_heads * q_len;
  if (row >= rows) return;
  const uint32_t q_pos = row % q_len;
  const uint32_t head = (row / q_len) % a.query_heads;
  const uint32_t batch = row / (q_len * a.query_heads);
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;
  const uint32_t kv_head = head / heads_per_kv;
  const uint32_t D = a.head_dim;
  const uint32_t groups_per_head = D >> 6;
  const uint32_t past = a.past_lengths ? a.past_lengths[batch] : a.past_length;
  const uint32_t *slots = a.slot_offsets ? a.slots + a.slot_offsets[batch] : a.slots;
  const size_t query_base = (((size_t)batch * a.query_heads + head) * q_len + q_pos) * D;
  const size_t current_base = ((size_t)batch * a.kv_heads + kv_head) * q_len * D;
  const uint32_t key_length = past + q_pos + 1;
  const uint32_t first_key = a.window == 0 || key_length <= a.window ? 0 : key_length - a.window;
  const uint32_t fragments = D >> 6;  // head_dim is a multiple of 64

  float q[kMaxFragments], result[kMaxFragments];
#pragma unroll
  for (int f = 0; f < kMaxFragments; ++f) {
    result[f] = 0.0f;
    q[f] = (uint32_t)f < fragments ? half_bits_to_float(a.query[query_base + f * 64 + lane]) : 0.0f;
  }
  float maximum = -INFINITY, denominator = 0.0f;
  const bool masked = a.mask != nullptr && a.mask_batches > 0 && a.mask_dtype != 0;

  for (uint32_t key_position = first_key; key_position < key_length; ++key_position) {
    if (masked) {
      const uint32_t mask_batch = a.mask_batches == 1 ? 0 : batch;
      const uint32_t mask_head = a.mask_heads == 1 ? 0 : head;
      const size_t mask_index =
          (((size_t)mask_batch * a.mask_heads + mask_head) * q_len + q_pos) * ((size_t)past + q_len) +
          key_position;
      const bool active = a.mask_dtype == 2
                              ? half_bits_to_float(reinterpret_cast<const uint16_t *>(a.mask)[mask_index]) >= 0.0f
                              : a.mask[mask_index] != 0;
      if (!active) continue;
    }
    float key[kMaxFragments], value[kMaxFragments];
    if (key_position < past) {
      const uint8_t *slot = a.pool + (size_t)slots[key_position] * a.token_stride;
      const int8_t *values = reinterpret_cast<const int8_t *>(slot);
#pragma unroll
      for (int f = 0; f < kMaxFragments; ++f) {
        if ((uint32_t)f >= fragments) break;
        const float ks = q8_scale_at(slot, a.token_elements, (a.key_offset >> 6) + kv_head * groups_per_head + f);
        const float vs = q8_scale_at(slot, a.token_elements, (a.value_offset >> 6) + kv_head * groups_per_head + f);
        key[f] = (float)values[a.key_offset + kv_head * D + f * 64 + lane] * ks;
        value[f] = (float)values[a.value_offset + kv_head * D + f * 64 + lane] * vs;
      }
    } else {
      const size_t base = current_base + (size_t)(key_position - past) * D;
#pragma unroll
      for (int f = 0; f < kMaxFragments; ++f) {
        if ((uint32_t)f >= fragments) break;
        key[f] = half_bits_to_float(a.current_key[base + f * 64 + lane]);
        value[f] = half_bits_to_float(a.current_value[base + f * 64 + lane]);
      }
    }
    float partial_score = 0.0f;
#pragma unroll
    for (int f = 0; f < kMaxFragments; ++f)
      if ((uint32_t)f < fragments) partial_score = fmaf(q[f], key[f], partial_score);
    const float score = wave_sum(partial_score) * a.scale;
    const float next_maximum = fmaxf(maximum, score);
    const float previous_scale = denominator == 0.0f ? 0.0f : __expf(maximum - next_maximum);
    const float current_scale = __expf(score - next_maximum);
#pragma unroll
    for (int f = 0; f < kMaxFragments; ++f)
      if ((uint32_t)f < fragments) result[f] = result[f] * previous_scale + current_scale * value[f];
    denominator = denominator * previous_scale + current_scale;
    maximum = next_maximum;
  }
  const size_t output_base = (((size_t)batch * q_len + q_pos) * a.query_heads + head) * D;
#pragma unroll
  for (int f = 0; f < kMaxFragments; ++f)
    if ((uint32_t)f < fragments)
      a.output[output_base + f * 64 + lane] =
          float_to_half_bits(denominator == 0.0f ? 0.0f : result[f] / denominator);
}

bool use_split_path(const Q8AttentionArgs &a) {
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const bool masked = a.mask != nullptr && a.mask_batches > 0 && a.mask_dtype != 0;
  if (q_len != 1 || masked || a.window != 0) return false;
  if (a.head_dim != 64 && a.head_dim != 128) return false;
  if (a.kv_heads == 0 || a.query_heads % a.kv_heads != 0) return false;
  if (a.query_heads / a.kv_heads > 16) return false;
  // 16-byte K loads and 4-byte V loads from pool slots
  if (a.token_stride % 16 != 0 || a.key_offset % 16 != 0 || a.value_offset % 4 != 0) return false;
  if (a.token_elements % 2 != 0) return false;
  return a.max_past_length >= 64;  // short contexts: one launch of the row kernel is cheaper
}

uint32_t split_chunks(const Q8AttentionArgs &a) {
  return (a.max_past_length + kChunkTokens - 1) / kChunkTokens;
}

}  // namespace

size_t q8_attention_workspace_bytes(const Q8AttentionArgs &a) {
  if (!use_split_path(a)) return 0;
  const size_t per_partial = 32 + (size_t)(a.query_heads / a.kv_heads) * a.head_dim;
  return (size_t)a.batches * a.kv_heads * split_chunks(a) * per_partial * sizeof(float);
}

hipError_t launch_q8_attention(const Q8AttentionArgs &a, hipStream_t stream) {
  if (use_split_path(a)) {
    const uint32_t chunks = split_chunks(a);
    if (a.workspace == nullptr || a.workspace_bytes < q8_attention_workspace_bytes(a))
      return hipErrorInvalidValue;
    const dim3 grid(chunks, a.kv_heads, a.batches);
    const dim3 merge_grid(a.query_heads, a.batches);
    if (a.head_dim == 128) {
      hipLaunchKernelGGL(q8_attention_split_kernel<128>, grid, dim3(kSplitThreads), 0, stream, a, chunks);
      hipLaunchKernelGGL(q8_attention_merge_kernel<128>, merge_grid, dim3(128), 0, stream, a, chunks);
    } else {
      hipLaunchKernelGGL(q8_attention_split_kernel<64>, grid, dim3(kSplitThreads), 0, stream, a, chunks);
      hipLaunchKernelGGL(q8_attention_merge_kernel<64>, merge_grid, dim3(64), 0, stream, a, chunks);
    }
    return hipGetLastError();
  }
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const uint32_t rows = a.batches * a.query_heads * q_len;
  if (rows == 0) return hipSuccess;
  hipLaunchKernelGGL(q8_attention_rows_kernel, dim3((rows + 3) / 4), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace llmopt
