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
#include <type_traits>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int kSplitMaxWaves = 4;   // KV heads per workgroup (one wave each)
constexpr int kMaxChunkTokens = 128;  // context tokens per workgroup: 128, or 64 / 32 when that leaves CUs idle
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

// Same without the subtraction: exact integers q + 1152.  Used for K, where the
// bias becomes a per-head constant 1152 * sum_d(Q[d]) subtracted from the score.
__device__ __forceinline__ void int8x4_to_h2_biased(uint32_t biased, h2_t &lo, h2_t &hi) {
  lo = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04010400u));
  hi = as_h2(__builtin_amdgcn_perm(0x64646464u, biased, 0x04030402u));
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

// OFF32: the pool is smaller than 4 GiB, so slot byte offsets fit 32 bits and the
// loads can use a scalar base plus a 32-bit vector offset.
// Three waves per SIMD: left alone the register allocator takes 209 registers
// (two waves), and the kernel is bound by the latency of each wave's requests.
template <int D, bool OFF32, bool A16>
__global__ __launch_bounds__(kSplitMaxWaves * 64) __attribute__((amdgpu_waves_per_eu(3, 3))) void
q8_attention_split_kernel(Q8AttentionArgs a, uint32_t chunks_max, uint32_t chunk_tokens) {
  constexpr int GROUPS = D / 64;      // scale groups per head
  constexpr int KLOADS = GROUPS;      // 16-byte K loads per lane per tile
  constexpr int VBLOCKS = D / 16;     // PV MFMAs (16 head_dim rows each)
  // One wave per KV head; the waves of a workgroup walk the same tokens, so the
  // cache lines of a token (its heads are adjacent in the pool slot, and all
  // its scales share one line) are fetched into one CU instead of eight XCDs.
  const uint32_t chunk = blockIdx.x;
  const uint32_t batch = blockIdx.z;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t kv_head =
      blockIdx.y * kSplitMaxWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (kv_head >= a.kv_heads) return;  // whole wave; no workgroup barriers below
  const uint32_t col = lane & 15;  // query head within the group / token / d-row
  const uint32_t quad = lane >> 4;
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;

  const uint32_t past = a.past_lengths ? a.past_lengths[batch] : a.past_length;
  const uint32_t chunk_begin = chunk * chunk_tokens;
  if (chunk_begin >= past) return;
  const uint32_t *slots = a.slot_offsets ? a.slots + a.slot_offsets[batch] : a.slots;
  // requests that run ahead of the arithmetic stop at the chunk's last token:
  // what lies beyond belongs to another workgroup and would be fetched twice
  const uint32_t last_token = min(chunk_begin + chunk_tokens, past) - 1;

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

  // 1152 * sum_d Q[head][d] per scale group: the constant the biased K decode
  // adds to every score of this head
  float key_bias[GROUPS];
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) {
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += (float)q_frag[g][j][e];
    sum += shfl_xor_f32(sum, 16);
    sum += shfl_xor_f32(sum, 32);
    key_bias[g] = 1152.0f * sum;
  }
  // softmax runs in base 2: exp(x) = exp2(x * log2(e))
  const float score_scale = a.scale * 1.4426950408889634f;

  const uint32_t key_base = a.key_offset + kv_head * D;
  const uint32_t value_base = a.value_offset + kv_head * D;
  const uint32_t key_scale_index = (a.key_offset >> 6) + kv_head * GROUPS;
  const uint32_t value_scale_index = (a.value_offset >> 6) + kv_head * GROUPS;

  float running_max = -INFINITY;  // per head (column), identical in the 4 quads
  float running_sum = 0.0f;       // per lane: this quad's tokens only
  f4_t out_acc[VBLOCKS];
#pragma unroll
  for (int v = 0; v < VBLOCKS; ++v) out_acc[v] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // Loaded-but-untouched registers of one 16-token tile.  Nothing in here may be
  // used before the tile is processed, or the loads are waited for at once.
  struct TileSlots {
    uint32_t key;       // slot of token (tile0 + col)
    uint32_t value[4];  // slots of tokens (tile0 + quad*4 + i)
  };
  struct TileRaw {
    u32x4_t k[KLOADS];          // lane (token = col, quad): 16 head_dim values per group
    uint32_t v[4][GROUPS];      // lane (d-row = col, quad): tokens quad*4 + i
    uint32_t k_scale[4];        // D = 128: both group scales of the token in one dword
    uint32_t v_scale[4];        // D = 64: the single scale in the low half
  };
  // D = 128 reads the two adjacent fp16 scales of a (token, head) as one dword;
  // the scale index is even because every segment offset is a multiple of 128.
  auto load_slots = [&](uint32_t tile, TileSlots &out) __attribute__((always_inline)) {
    const uint32_t token0 = chunk_begin + tile * kTileTokens;
    out.key = slots[min(token0 + col, last_token)];
#pragma unroll
    for (int i = 0; i < 4; ++i) out.value[i] = slots[min(token0 + quad * 4 + i, last_token)];
  };
  // With OFF32 every address is the scalar pool base plus one 32-bit lane offset
  // and a compile-time displacement, so a load needs no 64-bit vector add.
  // A16 = false: pool slots are only 4-byte aligned (a token stride that is not a
  // multiple of 16, e.g. 11880 bytes); the key loads then carry that alignment.
  typedef uint32_t unaligned_u32x4_t __attribute__((ext_vector_type(4), aligned(4)));
  using KeyVector = typename std::conditional<A16, u32x4_t, unaligned_u32x4_t>::type;
  auto load_raw = [&](const TileSlots &where, TileRaw &out) __attribute__((always_inline)) {
    if (OFF32) {
      const uint32_t key_offset = where.key * a.token_stride + key_base + quad * 16;
#pragma unroll
      for (int g = 0; g < KLOADS; ++g)
        out.k[g] = *reinterpret_cast<const KeyVector *>(a.pool + key_offset + g * 64);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t slot_offset = where.value[i] * a.token_stride;
        const uint32_t value_offset = slot_offset + value_base + col * 4;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g)
          out.v[i][g] = *reinterpret_cast<const uint32_t *>(a.pool + value_offset + g * 64);
        const uint32_t key_scale_offset = slot_offset + a.token_elements + 2 * key_scale_index;
        const uint32_t value_scale_offset = slot_offset + a.token_elements + 2 * value_scale_index;
        if (GROUPS == 2) {
          out.k_scale[i] = *reinterpret_cast<const uint32_t *>(a.pool + key_scale_offset);
          out.v_scale[i] = *reinterpret_cast<const uint32_t *>(a.pool + value_scale_offset);
        } else {
          out.k_scale[i] = *reinterpret_cast<const uint16_t *>(a.pool + key_scale_offset);
          out.v_scale[i] = *reinterpret_cast<const uint16_t *>(a.pool + value_scale_offset);
        }
      }
      return;
    }
    const uint8_t *key_slot = a.pool + (size_t)where.key * a.token_stride;
#pragma unroll
    for (int g = 0; g < KLOADS; ++g)
      out.k[g] = *reinterpret_cast<const KeyVector *>(key_slot + key_base + g * 64 + quad * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint8_t *slot = a.pool + (size_t)where.value[i] * a.token_stride;
#pragma unroll
      for (int g = 0; g < GROUPS; ++g)
        out.v[i][g] = *reinterpret_cast<const uint32_t *>(slot + value_base + g * 64 + col * 4);
      const uint8_t *scales = slot + a.token_elements;
      if (GROUPS == 2) {
        out.k_scale[i] = *reinterpret_cast<const uint32_t *>(scales + 2 * key_scale_index);
        out.v_scale[i] = *reinterpret_cast<const uint32_t *>(scales + 2 * value_scale_index);
      } else {
        out.k_scale[i] = *reinterpret_cast<const uint16_t *>(scales + 2 * key_scale_index);
        out.v_scale[i] = *reinterpret_cast<const uint16_t *>(scales + 2 * value_scale_index);
      }
    }
  };

  auto process = [&](uint32_t tile, const TileRaw &raw) __attribute__((always_inline)) {
    const uint32_t token0 = chunk_begin + tile * kTileTokens;
    // ---- scores S^T[token][head] = sum_g k_scale[token][g] * (K_g . Q_g) ----
    f4_t score = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      f4_t part = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        h2_t h0, h1, h2, h3;
        int8x4_to_h2_biased(raw.k[g][2 * j] ^ 0x80808080u, h0, h1);
        int8x4_to_h2_biased(raw.k[g][2 * j + 1] ^ 0x80808080u, h2, h3);
        const h8_t k_frag = {h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(k_frag, q_frag[g][j], part, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        score[i] = fmaf(part[i] - key_bias[g],
                        half_bits_to_float((uint16_t)(raw.k_scale[i] >> (16 * g))), score[i]);
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool valid = token0 + quad * 4 + i < past;
      score[i] = valid ? score[i] * score_scale : -INFINITY;
      tile_max = fmaxf(tile_max, score[i]);
    }
    tile_max = fmaxf(tile_max, shfl_xor_f32(tile_max, 16));
    tile_max = fmaxf(tile_max, shfl_xor_f32(tile_max, 32));
    // the first token of the tile is valid, so tile_max is finite
    const float new_max = fmaxf(running_max, tile_max);
    const float alpha = __builtin_amdgcn_exp2f(running_max - new_max);  // 0 on the first tile
    running_max = new_max;

    float p[4];
    float tile_sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = __builtin_amdgcn_exp2f(score[i] - new_max);
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
      for (int i = 0; i < 4; ++i)
        p_frag[i] = (_Float16)(p[i] * half_bits_to_float((uint16_t)(raw.v_scale[i] >> (16 * g))));
      const uint32_t a0 = raw.v[0][g] ^ 0x80808080u, a1 = raw.v[1][g] ^ 0x80808080u;
      const uint32_t a2 = raw.v[2][g] ^ 0x80808080u, a3 = raw.v[3][g] ^ 0x80808080u;
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
  };

  // The wave walks the 16-token tiles of the chunk.  Slot indices run two tiles
  // ahead and the K/V bytes one tile ahead of the arithmetic; requests past the
  // last tile are clamped to valid tokens and never used.
  const uint32_t chunk_tiles = (min(past - chunk_begin, chunk_tokens) + kTileTokens - 1) / kTileTokens;
  {
    TileSlots slots_a, slots_b;
    TileRaw raw_a, raw_b;
    load_slots(0, slots_a);
    load_slots(1, slots_b);
    load_raw(slots_a, raw_a);
    // Loads return in issue order, so the small slot loads go out before the
    // K/V loads of the same step: waiting for a slot then never waits for a
    // younger K/V request.
    for (uint32_t tile = 0; tile < chunk_tiles; tile += 2) {
      load_slots(tile + 2, slots_a);
      load_raw(slots_b, raw_b);
      process(tile, raw_a);
      if (tile + 1 >= chunk_tiles) break;
      load_slots(tile + 3, slots_b);
      load_raw(slots_a, raw_a);
      process(tile + 1, raw_b);
    }
  }

  // ---- one partial per (batch, kv_head, chunk), straight from registers ----
  // out_acc[g*4+jj][i] is O[head = col][d = g*64 + 4*(quad*4 + i) + jj].
  running_sum += shfl_xor_f32(running_sum, 16);
  running_sum += shfl_xor_f32(running_sum, 32);
  float *partial = reinterpret_cast<float *>(a.workspace) +
                   (((size_t)batch * a.kv_heads + kv_head) * chunks_max + chunk) *
                       partial_floats<D>(heads_per_kv);
  if (col < heads_per_kv) {
    if (quad == 0) {
      partial[col] = running_max;
      partial[16 + col] = running_sum;
    }
#pragma unroll
    for (int v = 0; v < VBLOCKS; ++v)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t d = (v >> 2) * 64 + 4 * (quad * 4 + i) + (v & 3);
        partial[32 + col * D + d] = out_acc[v][i];
      }
  }
}

constexpr int kMaxSplitChunks = 1024;  // merge kernel keeps one weight per chunk in LDS

constexpr int kMergeSlices = 4;  // chunk slices summed in parallel per output row

// One workgroup of kMergeSlices * D threads per (batch, query head): folds the
// chunk partials and the current token (fp16 K/V) into the output row.  Phase 1
// finds the global maximum and the per-chunk weights exp2(max_c - max) in
// parallel over chunks; phase 2 is an independent-load weighted sum over a
// quarter of the chunks per thread, finished through LDS.
template <int D>
__global__ __launch_bounds__(kMergeSlices *D) void q8_attention_merge_kernel(Q8AttentionArgs a,
                                                                             uint32_t chunks_max,
                                                                             uint32_t chunk_tokens) {
  constexpr int THREADS = kMergeSlices * D;
  constexpr int WAVES = THREADS / 64;
  __shared__ float reduce_lds[3][WAVES];
  __shared__ float weight_lds[kMaxSplitChunks];
  __shared__ float slice_lds[kMergeSlices][D];
  const uint32_t head = blockIdx.x;
  const uint32_t batch = blockIdx.y;
  const uint32_t tid = threadIdx.x;
  const uint32_t d = tid % D;
  const uint32_t slice = tid / D;
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;
  const uint32_t kv_head = head / heads_per_kv;
  const uint32_t local_head = head - kv_head * heads_per_kv;
  const uint32_t past = a.past_lengths ? a.past_lengths[batch] : a.past_length;
  const uint32_t chunks = (past + chunk_tokens - 1) / chunk_tokens;
  const size_t stride = partial_floats<D>(heads_per_kv);
  const float *partial = reinterpret_cast<const float *>(a.workspace) +
                         ((size_t)batch * a.kv_heads + kv_head) * chunks_max * stride;

  // score of the current token (slice 0 holds the dot product) and the largest chunk maximum
  const size_t current = ((size_t)batch * a.kv_heads + kv_head) * D + d;
  float dot = 0.0f;
  if (slice == 0)
    dot = half_bits_to_float(a.query[((size_t)batch * a.query_heads + head) * D + d]) *
          half_bits_to_float(a.current_key[current]);
  dot = wave_sum(dot);
  float chunk_best = -INFINITY;
  for (uint32_t c = tid; c < chunks; c += THREADS)
    chunk_best = fmaxf(chunk_best, partial[c * stride + local_head]);
  chunk_best = wave_max(chunk_best);
  if ((tid & 63) == 0) {
    reduce_lds[0][tid >> 6] = dot;
    reduce_lds[1][tid >> 6] = chunk_best;
  }
  __syncthreads();
  float score = 0.0f, best = -INFINITY;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    score += reduce_lds[0][w];
    best = fmaxf(best, reduce_lds[1][w]);
  }
  score *= a.scale * 1.4426950408889634f;  // the partial maxima are in base-2 units
  best = fmaxf(best, score);

  // weights and denominator
  float denominator_part = 0.0f;
  for (uint32_t c = tid; c < chunks; c += THREADS) {
    const float weight = __builtin_amdgcn_exp2f(partial[c * stride + local_head] - best);
    weight_lds[c] = weight;
    denominator_part += weight * partial[c * stride + 16 + local_head];
  }
  denominator_part = wave_sum(denominator_part);
  if ((tid & 63) == 0) reduce_lds[2][tid >> 6] = denominator_part;
  __syncthreads();
  const float current_weight = __builtin_amdgcn_exp2f(score - best);
  float denominator = current_weight;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) denominator += reduce_lds[2][w];

  float value = slice == 0 ? current_weight * half_bits_to_float(a.current_value[current]) : 0.0f;
  const float *column = partial + 32 + local_head * D + d;
  uint32_t c = slice;
  for (; c + 3 * kMergeSlices < chunks; c += 4 * kMergeSlices) {
    const float v0 = column[(c + 0 * kMergeSlices) * stride], v1 = column[(c + 1 * kMergeSlices) * stride];
    const float v2 = column[(c + 2 * kMergeSlices) * stride], v3 = column[(c + 3 * kMergeSlices) * stride];
    value += weight_lds[c] * v0 + weight_lds[c + kMergeSlices] * v1 +
             weight_lds[c + 2 * kMergeSlices] * v2 + weight_lds[c + 3 * kMergeSlices] * v3;
  }
  for (; c < chunks; c += kMergeSlices) value += weight_lds[c] * column[c * stride];
  slice_lds[slice][d] = value;
  __syncthreads();
  if (slice == 0) {
    float total = 0.0f;
#pragma unroll
    for (int s = 0; s < kMergeSlices; ++s) total += slice_lds[s][d];
    a.output[((size_t)batch * a.query_heads + head) * D + d] = float_to_half_bits(total / denominator);
  }
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
  // 4-byte aligned K and V loads from pool slots (16-byte aligned K loads when the stride allows)
  if (a.token_stride % 4 != 0 || a.key_offset % 4 != 0 || a.value_offset % 4 != 0) return false;
  if ((reinterpret_cast<uintptr_t>(a.pool) & 3) != 0) return false;
  if (a.token_elements % 2 != 0) return false;
  // D = 128 reads the two group scales of a head as one aligned dword
  if (a.head_dim == 128 && (a.key_offset % 128 != 0 || a.value_offset % 128 != 0)) return false;
  if (a.max_past_length > (uint32_t)kMaxChunkTokens * kMaxSplitChunks) return false;
  return a.max_past_length >= 64;  // short contexts: one launch of the row kernel is cheaper
}

// A wave is bound by the latency of its tiles, one after the other: when 128-token
// chunks give fewer waves than the device holds, shorter chunks finish sooner.
uint32_t split_chunk_tokens(const Q8AttentionArgs &a) {
  const uint64_t waves = (uint64_t)a.batches * a.kv_heads * ((a.max_past_length + 127) / 128);
  uint32_t tokens = waves >= 1024 ? 128 : waves >= 512 ? 64 : 32;
  while ((a.max_past_length + tokens - 1) / tokens > (uint32_t)kMaxSplitChunks) tokens *= 2;
  return tokens;
}

uint32_t split_chunks(const Q8AttentionArgs &a) {
  const uint32_t tokens = split_chunk_tokens(a);
  return (a.max_past_length + tokens - 1) / tokens;
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
    const uint32_t chunk_tokens = split_chunk_tokens(a);
    if (a.workspace == nullptr || a.workspace_bytes < q8_attention_workspace_bytes(a))
      return hipErrorInvalidValue;
    const uint32_t waves = std::min<uint32_t>(a.kv_heads, kSplitMaxWaves);
    const dim3 grid(chunks, (a.kv_heads + kSplitMaxWaves - 1) / kSplitMaxWaves, a.batches);
    const dim3 block(waves * 64);
    const dim3 merge_grid(a.query_heads, a.batches);
    const bool small_pool = a.pool_bytes > 0 && a.pool_bytes <= 0xffffffffull;
    const bool aligned16 = a.token_stride % 16 == 0 && a.key_offset % 16 == 0 &&
                           (reinterpret_cast<uintptr_t>(a.pool) & 15) == 0;
    const auto launch_split = [&](auto dim_tag) {
      constexpr int D = decltype(dim_tag)::value;
      if (small_pool && aligned16)
        hipLaunchKernelGGL((q8_attention_split_kernel<D, true, true>), grid, block, 0, stream, a, chunks, chunk_tokens);
      else if (small_pool)
        hipLaunchKernelGGL((q8_attention_split_kernel<D, true, false>), grid, block, 0, stream, a, chunks, chunk_tokens);
      else if (aligned16)
        hipLaunchKernelGGL((q8_attention_split_kernel<D, false, true>), grid, block, 0, stream, a, chunks, chunk_tokens);
      else
        hipLaunchKernelGGL((q8_attention_split_kernel<D, false, false>), grid, block, 0, stream, a, chunks, chunk_tokens);
      hipLaunchKernelGGL(q8_attention_merge_kernel<D>, merge_grid, dim3(kMergeSlices * D), 0, stream, a, chunks,
                         chunk_tokens);
    };
    if (a.head_dim == 128)
      launch_split(std::integral_constant<int, 128>{});
    else
      launch_split(std::integral_constant<int, 64>{});
    return hipGetLastError();
  }
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const uint32_t rows = a.batches * a.query_heads * q_len;
  if (rows == 0) return hipSuccess;
  hipLaunchKernelGGL(q8_attention_rows_kernel, dim3((rows + 3) / 4), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace llmopt
