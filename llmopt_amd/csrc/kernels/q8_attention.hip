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
//  * q8_attention_split_kernel (decode fast path: one query token, no mask, with or
//    without a sliding window, D in {64,128,256}, up to 16 query heads per KV head).  HBM-bound: the
//    context is split into chunks across workgroups, every KV byte is read once
//    per KV head and shared by all query heads of the group through the MFMA
//    column dimension.  int8 -> exact fp16 integers in registers; the fp16
//    group scales are applied in fp32 (K: on the score tile, V: on the
//    probability tile), never folded into fp16 operands.  Partials
//    (max, denominator, O) go to a workspace and q8_attention_merge_kernel
//    folds them together with the current token.
//
//  * q8_attention_general_kernel: one wave per (batch, head, query position) row,
//    64 keys at a time, one key per lane for the scores and one value row per
//    group of lanes for the weighted sum.  Covers everything else (masks,
//    several query tokens, other head sizes, unaligned pools, contexts under 64 tokens).
#include <algorithm>
#include <type_traits>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"
#include "w4_piece.h"

namespace llmopt {
namespace {

constexpr int kSplitMaxWaves = 4;   // KV heads per workgroup (one wave each)
constexpr int kMaxChunkTokens = 128;  // context tokens per workgroup: 128, or 64 / 32 when that leaves CUs idle
constexpr int kTileTokens = 16;    // tokens per MFMA tile
constexpr int kMaxSplitChunks = 1024;  // chunks per sequence: the merge kernel keeps one weight per chunk in LDS
static_assert((uint32_t)kMaxChunkTokens * kMaxSplitChunks == kQ8AttentionSplitTokens, "kernels.h states the limit");

__device__ __forceinline__ float q8_scale_at(const uint8_t *token, uint32_t token_elements,
                                             uint32_t index) {
  return half_bits_to_float(reinterpret_cast<const uint16_t *>(token + token_elements)[index]);
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

// Context length of sequence b.  Lengths in device memory may change between replays of a
// captured launch; they are held to max_past_length, which sized the grid, the partial results
// and the host's check of the slot table.
__device__ __forceinline__ uint32_t sequence_past(const Q8AttentionArgs &a, uint32_t b) {
  return a.past_lengths ? min(a.past_lengths[b], a.max_past_length) : a.past_length;
}

// Pool tokens the split kernels read for sequence b: with a sliding window the last window - 1
// cached tokens (the window counts the current token: first_key = key_length - window,
// lib/metal_cache_source.ml:430-431), i.e. a shorter context that starts `first` entries into
// the sequence's slot table.
struct PoolSpan {
  uint32_t first, length;
};
__device__ __forceinline__ PoolSpan sequence_span(const Q8AttentionArgs &a, uint32_t b) {
  const uint32_t past = sequence_past(a, b);
  const uint32_t first = (a.window == 0 || past < a.window) ? 0 : past + 1 - a.window;
  return {first, past - first};
}

// ---- balanced split --------------------------------------------------------------------
// With chunks of a fixed size the number of workgroups is whatever the contexts give, and the
// device runs them in rounds: 1028 chunks on 768 resident workgroups take two rounds, the
// second a third full.  Here the launch has a fixed number of chunk slots (what the device
// holds at once) and every sequence gets a share of them in proportion to its context, i.e.
// its own chunk size: one round, every workgroup with about the same number of tokens.
// The shares depend on the context lengths, which live in device memory, so every wave works
// them out for itself, one sequence per lane: share = 1 + floor(past * (slots - batches) / total)
// chunks of ceil(past / share) tokens rounded up to whole tiles.  The split and
// the merge kernel run the same instructions on the same inputs and so agree on the layout.
struct SplitPlan {
  uint32_t batch, first, chunks, tokens, past, slot_offset;
  bool found;
};

// Inclusive prefix sum over the 64 lanes with DPP: shifts inside the 16-lane rows, then the
// last lane of a row broadcast into the rows above it.  Lanes a shift has nothing for add 0.
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t value) {
  int v = (int)value;
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return (uint32_t)v;
}

// BY_INDEX: the sequence that owns chunk slot `key`; else sequence `key` itself.
constexpr int kPlanBlocks = 4;  // 64 sequences each: the balanced split serves batches up to 256

template <bool BY_INDEX>
__device__ __forceinline__ SplitPlan split_plan(const Q8AttentionArgs &a, uint32_t slots, uint32_t key) {
  const uint32_t lane = __lane_id();
  // every request goes out before the first result is used: one trip to memory
  uint32_t past[kPlanBlocks], slot_offset[kPlanBlocks];
#pragma unroll
  for (int k = 0; k < kPlanBlocks; ++k) {
    const uint32_t b = k * 64 + lane;
    const PoolSpan span = b < a.batches ? sequence_span(a, b) : PoolSpan{0, 0};
    past[k] = span.length;
    slot_offset[k] = (BY_INDEX && a.slot_offsets != nullptr && b < a.batches ? a.slot_offsets[b] : 0) + span.first;
  }
  uint32_t total = 0;
#pragma unroll
  for (int k = 0; k < kPlanBlocks; ++k) total += past[k];
  total = (uint32_t)__builtin_amdgcn_readlane((int)wave_inclusive_sum(total), 63);
  // a hair below (slots - batches) / total: the shares then add up to slots at most whatever the
  // float roundings do (a chunk beyond the last slot would have no workgroup)
  const float ratio =
      total != 0 ? __fmul_rn(__fdiv_rn((float)(slots - a.batches), (float)total), 0.999999f) : 0.0f;
  // a wave is bound by the latency of its tiles, one after the other, and every chunk costs a
  // partial result: 128-token chunks at least, shorter ones only when those leave the device idle
  const uint32_t waves = ((total + 127) >> 7) * a.kv_heads;
  const uint32_t least = waves >= 1024 ? 128 : waves >= 512 ? 64 : 32;
  SplitPlan plan = {0, 0, 0, 32, 0, 0, false};
  uint32_t carry = 0;
#pragma unroll
  for (int k = 0; k < kPlanBlocks; ++k) {
    if ((uint32_t)k * 64 >= a.batches) break;
    const uint32_t b = k * 64 + lane;
    const uint32_t share = min(1 + (uint32_t)__fmul_rn((float)past[k], ratio), (uint32_t)kMaxSplitChunks);
    const uint32_t tokens =
        max(least, ((past[k] + share - 1) / share + kTileTokens - 1) & ~(uint32_t)(kTileTokens - 1));
    const uint32_t chunks = (past[k] + tokens - 1) / tokens;
    const uint32_t inclusive = wave_inclusive_sum(chunks);
    const uint32_t first = carry + inclusive - chunks;
    const bool hit = b < a.batches && (BY_INDEX ? (key >= first && key < first + chunks) : b == key);
    const uint64_t hits = __builtin_amdgcn_ballot_w64(hit);
    if (hits != 0 && !plan.found) {
      const int source = __builtin_ctzll(hits);
      plan.batch = k * 64 + source;
      plan.first = (uint32_t)__builtin_amdgcn_readlane((int)first, source);
      plan.chunks = (uint32_t)__builtin_amdgcn_readlane((int)chunks, source);
      plan.tokens = (uint32_t)__builtin_amdgcn_readlane((int)tokens, source);
      plan.past = (uint32_t)__builtin_amdgcn_readlane((int)past[k], source);
      plan.slot_offset = (uint32_t)__builtin_amdgcn_readlane((int)slot_offset[k], source);
      plan.found = true;
    }
    carry += (uint32_t)__builtin_amdgcn_readlane((int)inclusive, 63);
  }
  return plan;
}

// OFF32: the pool is smaller than 4 GiB, so slot byte offsets fit 32 bits and the
// loads can use a scalar base plus a 32-bit vector offset.
// Three waves per SIMD: left alone the register allocator takes 209 registers
// (two waves), and the kernel is bound by the latency of each wave's requests.  (Heads of 256:
// two waves; a tile's lines, operands and the 64 output registers do not fit a third.)
template <int D>
constexpr int split_waves_wanted() {
  return D <= 128 ? 3 : 2;
}

template <int D, bool OFF32, bool A16>
__global__ __launch_bounds__(kSplitMaxWaves * 64)
    __attribute__((amdgpu_waves_per_eu(split_waves_wanted<D>(), split_waves_wanted<D>()))) void
q8_attention_split_kernel(Q8AttentionArgs a, uint32_t chunks_max, uint32_t fixed_chunk_tokens,
                          uint32_t balanced_slots) {
  constexpr int GROUPS = D / 64;      // scale groups per head
  constexpr int SW = (GROUPS + 1) / 2;  // dwords that hold a (token, head)'s fp16 group scales
  constexpr int KLOADS = GROUPS;      // 16-byte K loads per lane per tile
  constexpr int VBLOCKS = D / 16;     // PV MFMAs (16 head_dim rows each)
  // One wave per KV head; the waves of a workgroup walk the same tokens, so the
  // cache lines of a token (its heads are adjacent in the pool slot, and all
  // its scales share one line) are fetched into one CU instead of eight XCDs.
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t kv_head =
      blockIdx.y * kSplitMaxWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (kv_head >= a.kv_heads) return;  // whole wave; no workgroup barriers below
  const uint32_t col = lane & 15;  // query head within the group / token / d-row
  const uint32_t quad = lane >> 4;
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;

  // balanced_slots != 0: blockIdx.x is a chunk slot of the balanced split; else chunks of a
  // fixed size, blockIdx.x the chunk and blockIdx.z the sequence
  uint32_t chunk = blockIdx.x, batch = blockIdx.z, chunk_tokens = fixed_chunk_tokens, past, slot_offset;
  size_t partial_index;
  if (balanced_slots != 0) {
    const SplitPlan plan = split_plan<true>(a, balanced_slots, blockIdx.x);
    if (!plan.found) return;
    batch = plan.batch;
    chunk = blockIdx.x - plan.first;
    chunk_tokens = plan.tokens;
    past = plan.past;
    slot_offset = plan.slot_offset;
    partial_index = (size_t)kv_head * balanced_slots + blockIdx.x;
  } else {
    const PoolSpan span = sequence_span(a, batch);
    past = span.length;
    slot_offset = (a.slot_offsets ? a.slot_offsets[batch] : 0) + span.first;
    partial_index = ((size_t)batch * a.kv_heads + kv_head) * chunks_max + chunk;
  }
  const uint32_t chunk_begin = chunk * chunk_tokens;
  if (chunk_begin >= past) return;
  const uint32_t *slots = a.slots + slot_offset;
  // requests that run ahead of the arithmetic stop at the chunk's last token:
  // what lies beyond belongs to another workgroup and would be fetched twice
  const uint32_t last_token = min(chunk_begin + chunk_tokens, past) - 1;

  // B operand of the score MFMAs: Q[head = col][d], zero for columns >= G, and
  // 1152 * sum_d Q[head][d] per scale group: the constant the biased K decode
  // adds to every score of this head.  Both are filled in below, behind the first requests for
  // the context: a wave's start is a chain of trips to memory (context lengths, slot table, K/V
  // rows), and the query rows must not add theirs to it.
  h8_t q_frag[GROUPS][2];
  float key_bias[GROUPS];
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

  // ---- requests: whole lines ------------------------------------------------------------
  // A (token, head) row of K or V is D contiguous bytes.  D / 16 neighbouring lanes read one
  // row with 16 bytes each, so a load instruction covers 64 / (D / 16) tokens with whole
  // lines and a 16-token tile takes kTileTokens * D / 1024 instructions per operand - in MFMA
  // operand order the same bytes took 2 + 8 instructions whose lane quads each touched other
  // lines, and the kernel was bound by the number of requests, not by their bytes.  The
  // (key, value) scales of token lane % 16 ride in one more dword per lane (lanes 0..15 key,
  // 16..31 value).  The tile then passes through a wave-private LDS patch to reach operand
  // order (the LDS unit serves one wave's accesses in order: no barrier).
  constexpr int LPT = D / 16;            // lanes per (token, head) row
  constexpr int TPI = 64 / LPT;          // tokens per load instruction
  constexpr int KL = kTileTokens / TPI;  // load instructions per tile and operand
  constexpr int ROW = D + 32;            // LDS row stride: conflict-free 16-byte reads down the tokens
  const uint32_t line_token = lane / LPT, line_piece = lane % LPT;
  __shared__ __attribute__((aligned(16))) uint8_t turn_lds[kSplitMaxWaves][2 * kTileTokens * ROW + 128 * SW];
  uint8_t *key_patch = turn_lds[threadIdx.x >> 6];
  uint8_t *value_patch = key_patch + kTileTokens * ROW;
  uint32_t *scale_patch = reinterpret_cast<uint32_t *>(key_patch + 2 * kTileTokens * ROW);

  struct TileSlots {
    uint32_t line[KL];  // slot of token (tile0 + n * TPI + line_token)
    uint32_t scale;     // slot of token (tile0 + lane % 16)
  };
  // A16 = false: pool slots are only 4-byte aligned (a token stride that is not a
  // multiple of 16, e.g. 11880 bytes); the vector loads then carry that alignment.
  typedef uint32_t unaligned_u32x4_t __attribute__((ext_vector_type(4), aligned(4)));
  using KeyVector = typename std::conditional<A16, u32x4_t, unaligned_u32x4_t>::type;
  // Loaded-but-untouched registers of one 16-token tile.  Nothing in here may be
  // used before the tile is processed, or the loads are waited for at once.
  struct TileLine {
    u32x4_t k[KL], v[KL];
    uint32_t scale[SW];  // two group scales of the token per dword (D = 64: one scale in the low half)
  };
  struct TileRaw {              // the same tile in operand order
    u32x4_t k[KLOADS];          // lane (token = col, quad): 16 head_dim values per group
    uint32_t v[4][GROUPS];      // lane (d-row = col, quad): tokens quad*4 + i
    uint32_t k_scale[4][SW];    // tokens quad*4 + i
    uint32_t v_scale[4][SW];
  };
  auto load_slots = [&](uint32_t tile, TileSlots &out) __attribute__((always_inline)) {
    const uint32_t token0 = chunk_begin + tile * kTileTokens;
#pragma unroll
    for (int n = 0; n < KL; ++n) out.line[n] = slots[min(token0 + n * TPI + line_token, last_token)];
    out.scale = slots[min(token0 + col, last_token)];
  };
  // With OFF32 every address is the scalar pool base plus one 32-bit lane offset.
  // D = 128 reads the two adjacent fp16 scales of a (token, head) as one dword;
  // the scale index is even because every segment offset is a multiple of 128.
  const uint32_t scale_byte = a.token_elements + 2 * ((quad & 1) ? value_scale_index : key_scale_index);
  auto load_line = [&](const TileSlots &where, TileLine &out) __attribute__((always_inline)) {
    if (OFF32) {
#pragma unroll
      for (int n = 0; n < KL; ++n) {
        const uint32_t row = where.line[n] * a.token_stride + line_piece * 16;
        out.k[n] = *reinterpret_cast<const KeyVector *>(a.pool + row + key_base);
        out.v[n] = *reinterpret_cast<const KeyVector *>(a.pool + row + value_base);
      }
      const uint32_t scale_offset = where.scale * a.token_stride + scale_byte;
      if (GROUPS >= 2) {
#pragma unroll
        for (int w = 0; w < SW; ++w) out.scale[w] = *reinterpret_cast<const uint32_t *>(a.pool + scale_offset + 4 * w);
      } else {
        out.scale[0] = *reinterpret_cast<const uint16_t *>(a.pool + scale_offset);
      }
      return;
    }
#pragma unroll
    for (int n = 0; n < KL; ++n) {
      const uint8_t *row = a.pool + (size_t)where.line[n] * a.token_stride + line_piece * 16;
      out.k[n] = *reinterpret_cast<const KeyVector *>(row + key_base);
      out.v[n] = *reinterpret_cast<const KeyVector *>(row + value_base);
    }
    const uint8_t *scale_at = a.pool + (size_t)where.scale * a.token_stride + scale_byte;
    if (GROUPS >= 2) {
#pragma unroll
      for (int w = 0; w < SW; ++w) out.scale[w] = *reinterpret_cast<const uint32_t *>(scale_at + 4 * w);
    } else {
      out.scale[0] = *reinterpret_cast<const uint16_t *>(scale_at);
    }
  };
  auto turn = [&](const TileLine &line, TileRaw &raw) __attribute__((always_inline)) {
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int n = 0; n < KL; ++n) {
      const uint32_t at = (n * TPI + line_token) * ROW + line_piece * 16;
      *reinterpret_cast<u32x4_t *>(key_patch + at) = line.k[n];
      *reinterpret_cast<u32x4_t *>(value_patch + at) = line.v[n];
    }
    if (lane < 32) {
#pragma unroll
      for (int w = 0; w < SW; ++w) scale_patch[w * 32 + lane] = line.scale[w];
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int g = 0; g < GROUPS; ++g)
      raw.k[g] = *reinterpret_cast<const u32x4_t *>(key_patch + col * ROW + g * 64 + quad * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int g = 0; g < GROUPS; ++g)
        raw.v[i][g] = *reinterpret_cast<const uint32_t *>(value_patch + (quad * 4 + i) * ROW + g * 64 + col * 4);
#pragma unroll
    for (int w = 0; w < SW; ++w) {
      const u32x4_t key_scales = *reinterpret_cast<const u32x4_t *>(scale_patch + w * 32 + quad * 4);
      const u32x4_t value_scales = *reinterpret_cast<const u32x4_t *>(scale_patch + w * 32 + 16 + quad * 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        raw.k_scale[i][w] = key_scales[i];
        raw.v_scale[i][w] = value_scales[i];
      }
    }
    __builtin_amdgcn_wave_barrier();
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
                        half_bits_to_float((uint16_t)(raw.k_scale[i][g >> 1] >> (16 * (g & 1)))), score[i]);
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
        p_frag[i] = (_Float16)(p[i] * half_bits_to_float((uint16_t)(raw.v_scale[i][g >> 1] >> (16 * (g & 1)))));
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
    TileLine line_a, line_b;
    TileRaw raw;
    load_slots(0, slots_a);
    load_slots(1, slots_b);
    __builtin_amdgcn_sched_barrier(0);
    // the query rows go out behind the slot requests and ahead of the first K/V rows: loads return
    // in issue order, so waiting for the slots does not wait for them, and they have landed when
    // the first tile has.  Every lane reads (lanes of columns >= G read the group's last head and
    // drop it): a load under a branch is waited for where it stands.
    uint4 q_raw[GROUPS][2];
    {
      const uint16_t *q_row =
          a.query + ((size_t)batch * a.query_heads + kv_head * heads_per_kv + min(col, heads_per_kv - 1)) * D;
#pragma unroll
      for (int g = 0; g < GROUPS; ++g)
#pragma unroll
        for (int j = 0; j < 2; ++j) q_raw[g][j] = *reinterpret_cast<const uint4 *>(q_row + g * 64 + quad * 16 + j * 8);
    }
    __builtin_amdgcn_sched_barrier(0);
    load_line(slots_a, line_a);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        q_frag[g][j] = __builtin_bit_cast(h8_t, col < heads_per_kv ? q_raw[g][j] : make_uint4(0, 0, 0, 0));
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += (float)q_frag[g][j][e];
      }
      sum += shfl_xor_f32(sum, 16);
      sum += shfl_xor_f32(sum, 32);
      key_bias[g] = 1152.0f * sum;
    }
    // Loads return in issue order, so the small slot loads go out before the
    // K/V loads of the same step: waiting for a slot then never waits for a
    // younger K/V request.
    for (uint32_t tile = 0; tile < chunk_tiles; tile += 2) {
      load_slots(tile + 2, slots_a);
      load_line(slots_b, line_b);
      turn(line_a, raw);
      process(tile, raw);
      if (tile + 1 >= chunk_tiles) break;
      load_slots(tile + 3, slots_b);
      load_line(slots_a, line_a);
      turn(line_b, raw);
      process(tile + 1, raw);
    }
  }

  // ---- one partial per (batch, kv_head, chunk), straight from registers ----
  // out_acc[g*4+jj][i] is O[head = col][d = g*64 + 4*(quad*4 + i) + jj].
  running_sum += shfl_xor_f32(running_sum, 16);
  running_sum += shfl_xor_f32(running_sum, 32);
  float *partial = reinterpret_cast<float *>(a.workspace) + partial_index * partial_floats<D>(heads_per_kv);
  if (col < heads_per_kv) {
    if (quad == 0) {
      partial[col] = running_max;
      partial[16 + col] = running_sum;
    }
    // a lane's sixteen values of a scale group are consecutive in d: four 16-byte stores
#pragma unroll
    for (int g = 0; g < GROUPS; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const f4_t four = {out_acc[g * 4][i], out_acc[g * 4 + 1][i], out_acc[g * 4 + 2][i], out_acc[g * 4 + 3][i]};
        *reinterpret_cast<f4_t *>(partial + 32 + col * D + g * 64 + 4 * (quad * 4 + i)) = four;
      }
  }
}

constexpr int kMergeSlices = 4;  // chunk slices summed in parallel per output row

// One workgroup of kMergeSlices * D threads per (batch, query head): folds the
// chunk partials and the current token (fp16 K/V) into the output row.  Phase 1
// finds the global maximum and the per-chunk weights exp2(max_c - max) in
// parallel over chunks; phase 2 is an independent-load weighted sum over a
// quarter of the chunks per thread, finished through LDS.
// PASSES > 0 (D = 64): the row is not stored but multiplied into the head's 64 columns of an output
// projection (Q8AttentionArgs::projection): lane pair p of pass i owns output column p + 128 i and
// the two 16-byte pieces of that weight row that belong to this head (one scale group); the requests
// for them go out first and land while the partial results are being merged.
template <int D, int PASSES = 0>
__global__ __launch_bounds__(kMergeSlices *D) void q8_attention_merge_kernel(Q8AttentionArgs a,
                                                                             uint32_t chunks_max,
                                                                             uint32_t chunk_tokens,
                                                                             uint32_t balanced_slots) {
  constexpr int THREADS = kMergeSlices * D;
  constexpr int WAVES = THREADS / 64;
  static_assert(PASSES == 0 || D == 64, "a head's columns are one 64-wide scale group of the projection");
  __shared__ float reduce_lds[3][WAVES];
  __shared__ float weight_lds[kMaxSplitChunks];
  __shared__ float slice_lds[kMergeSlices][D];
  __shared__ __attribute__((aligned(16))) uint16_t row_lds[D];
  const uint32_t head = blockIdx.x;
  const uint32_t batch = blockIdx.y;
  const uint32_t tid = threadIdx.x;
  u32x4_t projection_weights[PASSES > 0 ? PASSES : 1];
  uint16_t projection_scales[PASSES > 0 ? PASSES : 1];
  if constexpr (PASSES > 0) {
    const uint32_t row_bytes = a.query_heads * (D / 2);
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const size_t column = min((tid >> 1) + (uint32_t)(THREADS / 2) * i, a.projected_width - 1);
      projection_weights[i] =
          *reinterpret_cast<const u32x4_t *>(a.projection.weight + column * row_bytes + head * (D / 2) + (tid & 1) * 16);
      projection_scales[i] = a.projection.scale[column * a.query_heads + head];
    }
  }
  const uint32_t d = tid % D;
  const uint32_t slice = tid / D;
  const uint32_t heads_per_kv = a.query_heads / a.kv_heads;
  const uint32_t kv_head = head / heads_per_kv;
  const uint32_t local_head = head - kv_head * heads_per_kv;
  const size_t stride = partial_floats<D>(heads_per_kv);
  // The current token's operands depend on the workgroup's indices only: they are requested before
  // the context lengths, by every thread (a load under a branch is waited for where it stands, which
  // made them a trip to memory of their own, after the partial results had landed).
  const size_t current = ((size_t)batch * a.kv_heads + kv_head) * D + d;
  const uint16_t current_value_bits = a.current_value[current];
  const uint16_t current_key_bits = a.current_key[current];
  const uint16_t query_bits = a.query[((size_t)batch * a.query_heads + head) * D + d];
  uint32_t chunks;
  const float *partial = reinterpret_cast<const float *>(a.workspace);
  if (balanced_slots != 0) {
    const SplitPlan plan = split_plan<false>(a, balanced_slots, batch);
    chunks = plan.chunks;
    partial += ((size_t)kv_head * balanced_slots + plan.first) * stride;
  } else {
    const uint32_t past = sequence_span(a, batch).length;
    chunks = (past + chunk_tokens - 1) / chunk_tokens;
    partial += ((size_t)batch * a.kv_heads + kv_head) * chunks_max * stride;
  }

  // Every request goes out before the first result is used - the chunk maxima and denominators
  // (chunk tid, tid + THREADS, ...), the first kAhead chunks of this thread's slice of the
  // weighted sum, the current token - so the kernel waits for memory once, not once per phase.
  constexpr int PER = kMaxSplitChunks / THREADS;  // chunks of phase 1 per thread
  // (heads of 64: sixteen, so that the 64 chunks of a lone sequence of 2048 tokens are one trip to memory, not two)
  constexpr int kAhead = D <= 64 ? 16 : 8;
  static_assert(PER * THREADS == kMaxSplitChunks, "phase 1 covers every chunk once");
  float chunk_max[PER], chunk_denominator[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const uint32_t c = tid + i * THREADS;
    chunk_max[i] = c < chunks ? partial[c * stride + local_head] : -INFINITY;
    chunk_denominator[i] = c < chunks ? partial[c * stride + 16 + local_head] : 0.0f;
  }
  const float *column = partial + 32 + local_head * D + d;
  float ahead[kAhead];
#pragma unroll
  for (int i = 0; i < kAhead; ++i) {
    const uint32_t c = slice + i * kMergeSlices;
    ahead[i] = c < chunks ? column[c * stride] : 0.0f;
  }
  // score of the current token (slice 0 holds the dot product) and the largest chunk maximum
  const float current_value = slice == 0 ? half_bits_to_float(current_value_bits) : 0.0f;
  float dot = slice == 0 ? half_bits_to_float(query_bits) * half_bits_to_float(current_key_bits) : 0.0f;
  dot = wave_sum(dot);
  float chunk_best = -INFINITY;
#pragma unroll
  for (int i = 0; i < PER; ++i) chunk_best = fmaxf(chunk_best, chunk_max[i]);
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
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const uint32_t c = tid + i * THREADS;
    if (c < chunks) {
      const float weight = __builtin_amdgcn_exp2f(chunk_max[i] - best);
      weight_lds[c] = weight;
      denominator_part += weight * chunk_denominator[i];
    }
  }
  denominator_part = wave_sum(denominator_part);
  if ((tid & 63) == 0) reduce_lds[2][tid >> 6] = denominator_part;
  __syncthreads();
  const float current_weight = __builtin_amdgcn_exp2f(score - best);
  float denominator = current_weight;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) denominator += reduce_lds[2][w];

  float value = current_weight * current_value;
#pragma unroll
  for (int i = 0; i < kAhead; ++i) {
    const uint32_t c = slice + i * kMergeSlices;
    if (c < chunks) value += weight_lds[c] * ahead[i];
  }
  uint32_t c = slice + kAhead * kMergeSlices;
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
    const uint16_t stored = float_to_half_bits(total / denominator);
    if constexpr (PASSES == 0)
      a.output[((size_t)batch * a.query_heads + head) * D + d] = stored;
    else
      row_lds[d] = stored;
  }
  if constexpr (PASSES > 0) {
    __syncthreads();
    Held<1> held;
    hold_rows<1>(held, row_lds, D, tid & 1, true);
    float *out = a.projected + ((size_t)head * a.batches + batch) * a.projected_width;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      float share[1];
      piece_dot<1>(projection_weights[i], half_bits_to_float(projection_scales[i]), held, share);
      const float total = share[0] + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                                         0, __builtin_bit_cast(int, share[0]), 0xB1, 0xF, 0xF, false));
      const uint32_t column = (tid >> 1) + (uint32_t)(THREADS / 2) * i;
      if ((tid & 1) == 0 && column < a.projected_width) out[column] = total;
    }
  }
}

// ---- general kernel (every other configuration) -------------------------------------------
// Masks (bool / f16), sliding windows, several query tokens, head sizes up to 512, unaligned
// pools.  One wave per output row (batch, head, query position), keys in tiles of 64 with
// **one key per lane** for the scores: a lane walks its key's row (16-byte requests, the next
// ones hit the line the first brought in), decodes int8 to exact halves and multiplies against
// the query row, which every lane reads from the same LDS address (a broadcast).  No reduction
// across lanes per key: the softmax statistics of 64 keys take one wave maximum and one wave
// sum.  For the weighted sum of the values the lanes change roles - `lanes_per_key` lanes share
// a value row, four (eight at D = 512) head_dim values each, 64 / lanes_per_key keys per request
// - and take each key's probability x group scale and row address from a small LDS table the
// score phase left; the keys that shared a lane's head_dim slice are added at the end.
constexpr int kGeneralWaves = 4;
constexpr int kGeneralLdsWords = 512 / 2 + 8 * 64 + 64 * 2 + 64;  // query (half2), weight[8][64], row address, kind

struct GeneralRow {
  uint32_t batch, head, q_pos, kv_head, past, key_length, first_key;
};

// ALIGNED: pool rows can be read as dwords (pool address, token stride and segment offsets are
// multiples of four); otherwise byte by byte.
template <bool ALIGNED>
__global__ __launch_bounds__(kGeneralWaves * 64) void q8_attention_general_kernel(Q8AttentionArgs a) {
  __shared__ __attribute__((aligned(16))) uint32_t general_lds[kGeneralWaves][kGeneralLdsWords];
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * kGeneralWaves + (threadIdx.x >> 6);
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const uint32_t rows = a.batches * a.query_heads * q_len;
  if (row >= rows) return;  // whole wave; no workgroup barriers below
  uint32_t *lds = general_lds[threadIdx.x >> 6];
  uint32_t *query_lds = lds;                                      // D / 2 half pairs
  float *weight_lds = reinterpret_cast<float *>(lds + 256);       // [group][key]: probability x value scale
  uint64_t *address_lds = reinterpret_cast<uint64_t *>(lds + 256 + 512);  // value row of every key of the tile
  uint32_t *kind_lds = lds + 256 + 512 + 128;                     // 1: int8 pool row, 0: fp16 current token

  const uint32_t D = a.head_dim, groups = D >> 6;
  GeneralRow r;
  r.q_pos = row % q_len;
  r.head = (row / q_len) % a.query_heads;
  r.batch = row / (q_len * a.query_heads);
  r.kv_head = r.head / (a.query_heads / a.kv_heads);
  r.past = sequence_past(a, r.batch);
  r.key_length = r.past + r.q_pos + 1;  // causal over the query tokens
  r.first_key = a.window == 0 || r.key_length <= a.window ? 0 : r.key_length - a.window;
  const uint32_t *slots = a.slot_offsets ? a.slots + a.slot_offsets[r.batch] : a.slots;
  const uint16_t *query = a.query + (((size_t)r.batch * a.query_heads + r.head) * q_len + r.q_pos) * D;
  const size_t current_base = ((size_t)r.batch * a.kv_heads + r.kv_head) * q_len * D;
  const bool masked = a.mask != nullptr && a.mask_batches > 0 && a.mask_dtype != 0;
  const size_t mask_row =
      masked ? (((size_t)(a.mask_batches == 1 ? 0 : r.batch) * a.mask_heads + (a.mask_heads == 1 ? 0 : r.head)) * q_len +
                r.q_pos) * ((size_t)r.past + q_len)
             : 0;
  const uint32_t key_scale_index = (a.key_offset >> 6) + r.kv_head * groups;
  const uint32_t value_scale_index = (a.value_offset >> 6) + r.kv_head * groups;

  for (uint32_t i = lane; i < D / 2; i += 64) query_lds[i] = reinterpret_cast<const uint32_t *>(query)[i];
  __builtin_amdgcn_wave_barrier();

  // value phase geometry
  const uint32_t per_lane = D > 256 ? 8 : 4;                 // head_dim values per lane
  const uint32_t lanes_per_key = D / per_lane;               // 16, 32, 48 or 64
  const uint32_t keys_per_request = 64 / lanes_per_key;      // 4, 2, 1, 1
  const uint32_t key_sub = lane / lanes_per_key, d0 = (lane % lanes_per_key) * per_lane;
  const bool value_lane = key_sub < keys_per_request;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float maximum = -INFINITY, denominator = 0.0f;

  // A wave's tile is a chain of trips to memory (slot table, key rows, value rows), one tile after
  // the other, and a load under a branch is waited for where it stands.  So: the slot of the next
  // tile's key is requested a tile ahead; the pool requests of a tile go out for every lane, at a
  // clamped valid address, and what a lane has no use for is dropped afterwards.
  const uint32_t last_past = r.past == 0 ? 0 : r.past - 1;
  uint32_t next_slot = r.past != 0 ? slots[min(r.first_key + lane, last_past)] : 0;
  for (uint32_t base = r.first_key; base < r.key_length; base += 64) {
    // ---- scores: lane = key ----
    const uint32_t key_position = base + lane;
    const bool in_range = key_position < r.key_length;
    const bool is_past = key_position < r.past;
    bool active = in_range;
    if (masked && in_range) {
      const size_t at = mask_row + key_position;
      active = a.mask_dtype == 2 ? half_bits_to_float(reinterpret_cast<const uint16_t *>(a.mask)[at]) >= 0.0f
                                 : a.mask[at] != 0;
    }
    // (lanes without a pool key read slot `next_slot` of a valid key of the sequence, or the pool's first token)
    const uint8_t *slot = a.pool + (size_t)next_slot * a.token_stride;
    if (r.past != 0) next_slot = slots[min(key_position + 64, last_past)];
    float score = 0.0f;
    if (r.past != 0 && base < r.past) {
      const uint8_t *key_row = slot + a.key_offset + r.kv_head * D;
      float key_scale[8];
#pragma unroll
      for (int g = 0; g < 8; ++g)
        key_scale[g] = q8_scale_at(slot, a.token_elements, key_scale_index + min((uint32_t)g, groups - 1));
      auto load_group = [&](uint32_t g, uint32_t (&words)[16]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (ALIGNED) {
            const u32x4_t loaded = *reinterpret_cast<const u32x4_t __attribute__((aligned(4))) *>(key_row + g * 64 + j * 16);
            words[4 * j] = loaded[0], words[4 * j + 1] = loaded[1], words[4 * j + 2] = loaded[2], words[4 * j + 3] = loaded[3];
          } else {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              const uint8_t *b = key_row + g * 64 + j * 16 + w * 4;
              words[4 * j + w] = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24);
            }
          }
        }
      };
      auto dot_group = [&](uint32_t g, const uint32_t (&words)[16]) __attribute__((always_inline)) {
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint4 q_lo = *reinterpret_cast<const uint4 *>(query_lds + (g * 64 + j * 16) / 2);
          const uint4 q_hi = *reinterpret_cast<const uint4 *>(query_lds + (g * 64 + j * 16) / 2 + 4);
          const uint32_t q_pairs[8] = {q_lo.x, q_lo.y, q_lo.z, q_lo.w, q_hi.x, q_hi.y, q_hi.z, q_hi.w};
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            h2_t lo, hi;
            int8x4_to_h2(words[4 * j + w] ^ 0x80808080u, lo, hi);
            part = __builtin_amdgcn_fdot2(lo, as_h2(q_pairs[2 * w]), part, false);
            part = __builtin_amdgcn_fdot2(hi, as_h2(q_pairs[2 * w + 1]), part, false);
          }
        }
        return part;
      };
      auto scale_of = [&](uint32_t g) __attribute__((always_inline)) {
        float scale = key_scale[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) scale = g == (uint32_t)e ? key_scale[e] : scale;
        return scale;
      };
      if (groups <= 2) {
        // the whole key row (64 or 128 bytes) in one trip
        uint32_t first[16], second[16];
        load_group(0, first);
        load_group(groups - 1, second);
        score = dot_group(0, first) * key_scale[0];
        if (groups == 2) score = fmaf(dot_group(1, second), key_scale[1], score);
      } else {
        // four scale groups (256 bytes of the key row) per trip
        for (uint32_t g = 0; g < groups; g += 4) {
          uint32_t words[4][16];
#pragma unroll
          for (int e = 0; e < 4; ++e) load_group(min(g + e, groups - 1), words[e]);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (g + e < groups) score = fmaf(dot_group(g + e, words[e]), scale_of(g + e), score);
        }
      }
    }
    if (in_range && !is_past) {
      score = 0.0f;
      const uint16_t *key_row = a.current_key + current_base + (size_t)(key_position - r.past) * D;
      for (uint32_t i = 0; i < D / 2; ++i)
        score = __builtin_amdgcn_fdot2(as_h2((uint32_t)key_row[2 * i] | ((uint32_t)key_row[2 * i + 1] << 16)),
                                       as_h2(query_lds[i]), score, false);
    }
    score = active ? score * a.scale : -INFINITY;
    const float tile_maximum = wave_max(score);
    if (tile_maximum == -INFINITY) continue;  // no key of this tile is allowed (the same for every lane)
    const float next_maximum = fmaxf(maximum, tile_maximum);
    const float previous_scale = __expf(maximum - next_maximum);  // 0 for the first tile with a key
    const float probability = active ? __expf(score - next_maximum) : 0.0f;
    denominator = denominator * previous_scale + wave_sum(probability);
    maximum = next_maximum;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= previous_scale;
    // ---- hand the tile to the value phase ----
    const uint8_t *value_row = reinterpret_cast<const uint8_t *>(a.current_value + current_base);  // a valid address for idle keys
    if (in_range && is_past) value_row = slot + a.value_offset + r.kv_head * D;
    else if (in_range) value_row = reinterpret_cast<const uint8_t *>(a.current_value + current_base + (size_t)(key_position - r.past) * D);
    address_lds[lane] = reinterpret_cast<uint64_t>(value_row);
    kind_lds[lane] = in_range && is_past ? 1u : 0u;
    for (uint32_t g = 0; g < groups; ++g)
      weight_lds[g * 64 + lane] =
          in_range && is_past ? probability * q8_scale_at(slot, a.token_elements, value_scale_index + g) : probability;
    __builtin_amdgcn_wave_barrier();
    // ---- values: lanes_per_key lanes share a key's row ----
    const uint32_t tile_keys = min(64u, r.key_length - base);
    const uint32_t pool_keys = base < r.past ? min(tile_keys, r.past - base) : 0;  // the tile's first keys
    if (value_lane) {
      // pool rows, sixteen requests on the way at a time: every slot of the tile's table holds a valid
      // address, so the requests go out whether or not the key counts, and its weight decides
      constexpr int AHEAD = 16;
      for (uint32_t k0 = 0; k0 < pool_keys; k0 += keys_per_request * AHEAD) {
        uint32_t word[AHEAD][2];
        float weight[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
          const uint32_t wanted = k0 + u * keys_per_request + key_sub;
          const uint32_t k = min(wanted, 63u);
          weight[u] = wanted < pool_keys ? weight_lds[(d0 >> 6) * 64 + k] : 0.0f;
          const uint8_t *b = reinterpret_cast<const uint8_t *>(address_lds[k]) + d0;
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            const uint8_t *at = b + (per_lane == 8 ? 4 * w : 0);
            if (ALIGNED)
              word[u][w] = *reinterpret_cast<const uint32_t *>(at);
            else
              word[u][w] = (uint32_t)at[0] | ((uint32_t)at[1] << 8) | ((uint32_t)at[2] << 16) | ((uint32_t)at[3] << 24);
          }
        }
#pragma unroll
        for (int u = 0; u < AHEAD; ++u)
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            h2_t lo, hi;
            int8x4_to_h2(word[u][w] ^ 0x80808080u, lo, hi);
            const float share = (w == 0 || per_lane == 8) ? weight[u] : 0.0f;
            acc[4 * w + 0] = fmaf(share, (float)lo[0], acc[4 * w + 0]);
            acc[4 * w + 1] = fmaf(share, (float)lo[1], acc[4 * w + 1]);
            acc[4 * w + 2] = fmaf(share, (float)hi[0], acc[4 * w + 2]);
            acc[4 * w + 3] = fmaf(share, (float)hi[1], acc[4 * w + 3]);
          }
      }
      // the query tokens' own fp16 rows (the last keys; at most query_length of them in all)
      for (uint32_t k0 = pool_keys; k0 < tile_keys; k0 += keys_per_request) {
        const uint32_t k = min(k0 + key_sub, 63u);
        const float weight = k0 + key_sub < tile_keys ? weight_lds[(d0 >> 6) * 64 + k] : 0.0f;
        const uint16_t *halves = reinterpret_cast<const uint16_t *>(address_lds[k]) + d0;
        for (uint32_t e = 0; e < per_lane; ++e) acc[e] = fmaf(weight, half_bits_to_float(halves[e]), acc[e]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // keys that shared this lane's head_dim slice (keys_per_request = 4: lanes 16 apart; 2: 32 apart)
  if (keys_per_request >= 2)
    for (int e = 0; e < 4; ++e) acc[e] += shfl_xor_f32(acc[e], 32);
  if (keys_per_request == 4)
    for (int e = 0; e < 4; ++e) acc[e] += shfl_xor_f32(acc[e], 16);
  if (lane < lanes_per_key) {
    uint16_t *out = a.output + (((size_t)r.batch * q_len + r.q_pos) * a.query_heads + r.head) * D + d0;
    for (uint32_t e = 0; e < per_lane; ++e)
      out[e] = float_to_half_bits(denominator == 0.0f ? 0.0f : acc[e] / denominator);
  }
}

// ---- several query tokens: a half-precision copy of the context and the dense tile kernel ----
//
// The reference prefills a suffix over cached tokens with this entry (query_length new tokens, a
// byte mask that is causal over them: suffix_causal_mask, lib/serving_engine.ml:1194-1201).  A wave
// per output row re-reads the context once per row; with sixteen query tokens or more (or two, over
// at least 256 keys) the context of the layer is instead written out once as halves - pool tokens as half(float(int8) *
// float(scale)), the new tokens' K and V copied behind them - and the dense kernel, which shares
// every K / V tile among 128 query rows on the matrix cores, runs over that copy with the same
// mask, the causal limit over the new tokens and token-major output.  The copy rounds a cached
// value once more (2^-11 relative at most), where the row kernel multiplies int8 by scale in
// float32: within the tolerance the path's results are held to.
__global__ __launch_bounds__(256) void q8_context_as_halves_kernel(Q8AttentionArgs a, uint16_t *key16, uint16_t *value16) {
  const uint32_t q_len = a.query_length, L = a.past_length + q_len, D = a.head_dim, pieces = D / 8;
  const uint64_t index = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (index >= (uint64_t)a.batches * a.kv_heads * L * pieces) return;
  const bool is_value = blockIdx.y != 0;
  const uint32_t piece = (uint32_t)(index % pieces), token = (uint32_t)(index / pieces % L);
  const uint32_t kv_head = (uint32_t)(index / pieces / L % a.kv_heads), batch = (uint32_t)(index / pieces / L / a.kv_heads);
  uint16_t *destination =
      (is_value ? value16 : key16) + (((size_t)batch * a.kv_heads + kv_head) * L + token) * D + piece * 8;
  uint4 halves;
  if (token < a.past_length) {
    const uint8_t *slot = a.pool + (size_t)a.slots[token] * a.token_stride;
    const uint32_t element = (is_value ? a.value_offset : a.key_offset) + kv_head * D + piece * 8;
    const float scale = q8_scale_at(slot, a.token_elements, element >> 6);
    const uint8_t *bytes = slot + element;
    uint32_t packed[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float low = (float)(int8_t)bytes[2 * e] * scale, high = (float)(int8_t)bytes[2 * e + 1] * scale;
      packed[e] = (uint32_t)float_to_half_bits(low) | ((uint32_t)float_to_half_bits(high) << 16);
    }
    halves = make_uint4(packed[0], packed[1], packed[2], packed[3]);
  } else {
    const uint16_t *source = (is_value ? a.current_value : a.current_key) +
                             (((size_t)batch * a.kv_heads + kv_head) * q_len + (token - a.past_length)) * D + piece * 8;
    halves = *reinterpret_cast<const uint4 *>(source);
  }
  *reinterpret_cast<uint4 *>(destination) = halves;
}

bool use_dense_copy_path(const Q8AttentionArgs &a) {
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  // sixteen query tokens or more; from two on when the context is long enough for the copy to pay
  // (3 new tokens after 2048 of the 9/3 x 64 model: 93 -> 47 us; after 100: the row kernel's 11 us stand)
  if (q_len < 2 || (q_len < 16 && (uint64_t)a.past_length + q_len < 256)) return false;
  if (a.window != 0 || a.past_lengths != nullptr || a.slot_offsets != nullptr) return false;
  if (a.head_dim != 64 && a.head_dim != 128 && a.head_dim != 256) return false;
  if (a.kv_heads == 0 || a.query_heads % a.kv_heads != 0) return false;
  if (!(a.scale > 0.0f && a.scale < INFINITY)) return false;
  if ((uint64_t)a.past_length + q_len > 0x7fffffffull) return false;
  // 16-byte copies of the new tokens' rows; what the dense tile kernel asks of its operands
  return ((reinterpret_cast<uintptr_t>(a.query) | reinterpret_cast<uintptr_t>(a.current_key) |
           reinterpret_cast<uintptr_t>(a.current_value)) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(a.output) & 7) == 0;
}

// Where the copy and the dense kernel's own scratch lie in the workspace, and the dense launch.
struct DenseCopyPlan {
  size_t operand_bytes;  // one of K, V as halves (a multiple of 256)
  size_t map_bytes, total_bytes;
  DenseAttentionArgs dense;
};

DenseCopyPlan dense_copy_plan(const Q8AttentionArgs &a, void *workspace) {
  DenseCopyPlan plan = {};
  const uint32_t q_len = a.query_length, L = a.past_length + q_len;
  plan.operand_bytes = ((size_t)a.batches * a.kv_heads * L * a.head_dim * 2 + 255) & ~(size_t)255;
  // (sizing without a workspace yet: any address with the workspace's alignment gives the same answer)
  uint8_t *base = workspace != nullptr ? static_cast<uint8_t *>(workspace) : reinterpret_cast<uint8_t *>((uintptr_t)4096);
  const bool masked = a.mask != nullptr && a.mask_batches > 0 && a.mask_dtype != 0;
  DenseAttentionArgs &d = plan.dense;
  d.query = a.query;
  d.key = reinterpret_cast<const uint16_t *>(base);
  d.value = reinterpret_cast<const uint16_t *>(base + plan.operand_bytes);
  d.mask = masked ? a.mask : nullptr;
  d.output = a.output;
  d.batches = a.batches, d.heads = a.query_heads, d.query_length = q_len, d.key_length = L, d.head_dim = a.head_dim;
  d.mask_batches = masked ? a.mask_batches : 0, d.mask_heads = masked ? a.mask_heads : 0;
  d.causal = 1;  // key_length of query token q is past_length + q + 1 (lib/metal_cache_source.ml:429)
  d.scale = a.scale;
  d.kv_heads = a.kv_heads, d.token_first_output = 1, d.past_length = a.past_length, d.token_first_value = 0;
  d.mask_dtype = masked ? a.mask_dtype : 0;
  plan.map_bytes = dense_attention_workspace_bytes(d);
  plan.total_bytes = 2 * plan.operand_bytes + plan.map_bytes;
  if (plan.map_bytes > 0) {
    d.stage_map = base + 2 * plan.operand_bytes;
    d.stage_map_bytes = plan.map_bytes;
  }
  return plan;
}

// The longest span of pool tokens a sequence of the launch can have (see sequence_span).
uint32_t longest_span(const Q8AttentionArgs &a) {
  return a.window != 0 && a.max_past_length >= a.window ? a.window - 1 : a.max_past_length;
}

bool use_split_path(const Q8AttentionArgs &a) {
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const bool masked = a.mask != nullptr && a.mask_batches > 0 && a.mask_dtype != 0;
  if (q_len != 1 || masked) return false;
  if (a.head_dim != 64 && a.head_dim != 128 && a.head_dim != 256) return false;
  if (a.kv_heads == 0 || a.query_heads % a.kv_heads != 0) return false;
  if (a.query_heads / a.kv_heads > 16) return false;
  // 4-byte aligned K and V loads from pool slots (16-byte aligned K loads when the stride allows)
  if (a.token_stride % 4 != 0 || a.key_offset % 4 != 0 || a.value_offset % 4 != 0) return false;
  if ((reinterpret_cast<uintptr_t>(a.pool) & 3) != 0) return false;
  if (a.token_elements % 2 != 0) return false;
  // D >= 128 reads the group scales of a head two to an aligned dword
  if (a.head_dim >= 128 && (a.key_offset % 128 != 0 || a.value_offset % 128 != 0)) return false;
  if (longest_span(a) > (uint32_t)kMaxChunkTokens * kMaxSplitChunks) return false;
  return longest_span(a) >= 64;  // short contexts: one launch of the general kernel is cheaper
}

// A wave is bound by the latency of its tiles, one after the other: when 128-token
// chunks give fewer waves than the device holds, shorter chunks finish sooner.
uint32_t split_chunk_tokens(const Q8AttentionArgs &a) {
  const uint64_t waves = (uint64_t)a.batches * a.kv_heads * ((longest_span(a) + 127) / 128);
  uint32_t tokens = waves >= 1024 ? 128 : waves >= 512 ? 64 : 32;
  while ((longest_span(a) + tokens - 1) / tokens > (uint32_t)kMaxSplitChunks) tokens *= 2;
  return tokens;
}

uint32_t split_chunks(const Q8AttentionArgs &a) {
  const uint32_t tokens = split_chunk_tokens(a);
  return (longest_span(a) + tokens - 1) / tokens;
}

// Waves of the split kernel a SIMD holds at once, from the registers the compiler gave it
// (512 vector registers per SIMD lane, allocated in blocks of 8).
template <int D>
uint32_t split_waves_per_simd() {
  static uint32_t cached = 0;
  if (cached == 0) {
    hipFuncAttributes attributes;
    uint32_t waves = 3;
    if (hipFuncGetAttributes(&attributes, reinterpret_cast<const void *>(&q8_attention_split_kernel<D, true, true>)) ==
            hipSuccess &&
        attributes.numRegs > 0)
      waves = std::max(1, std::min(8, 512 / ((attributes.numRegs + 7) / 8 * 8)));
    else
      (void)hipGetLastError();
    cached = waves;
  }
  return cached;
}

// Chunk slots of the balanced split (0 = fixed chunks): the chunks the device holds at once
// (whole workgroups of one wave per KV head and chunk), times the number of rounds that gives a
// sequence about sixteen chunks - with few, rounding the shares down leaves slots unused, and
// 128 sequences of 2048 tokens measured 2.72 ms per decode step with 16 chunks of 128 tokens
// each against 2.77 with 12 longer ones.  One sequence has
// nothing to balance, and every wave scans the context lengths, so this is for batches a wave
// covers in a few passes.
uint32_t balanced_split_slots(const Q8AttentionArgs &a) {
  if (a.batches < 2 || a.batches > 64 * kPlanBlocks) return 0;
  const uint32_t per_simd = a.head_dim == 256   ? split_waves_per_simd<256>()
                            : a.head_dim == 128 ? split_waves_per_simd<128>()
                                                : split_waves_per_simd<64>();
  // whole workgroups: one wave per KV head, at most kSplitMaxWaves of them
  const uint32_t waves = std::min<uint32_t>(a.kv_heads, kSplitMaxWaves);
  const uint32_t head_groups = (a.kv_heads + kSplitMaxWaves - 1) / kSplitMaxWaves;
  // Eight waves keep a CU as busy as twelve do (the kernel is bound by the CU's own work per byte,
  // not by its requests), and the launch takes as long as the CU with the most workgroups: the
  // same number on every CU, and no more than that takes - fewer, longer chunks leave fewer
  // partial results.  Measured at 16 sequences of 512..8192 tokens, 8 KV heads of 128: 256 slots
  // (two workgroups per CU) 37.6 us, 384 (three) 39.0, 288 or 320 (two on some CUs, three on
  // others) 42-44, 192 (one or two) 42.3.
  const uint32_t per_cu = std::max<uint32_t>(1, std::min(4 * per_simd / waves, (8 + waves - 1) / waves));
  const uint32_t resident = std::max<uint32_t>(1, (uint32_t)device_compute_units() * per_cu / head_groups);
  const uint32_t rounds = std::max<uint32_t>(1, (16 * a.batches + resident - 1) / resident);
  return resident * rounds;
}

}  // namespace

size_t q8_attention_workspace_bytes(const Q8AttentionArgs &a) {
  if (use_dense_copy_path(a)) return dense_copy_plan(a, nullptr).total_bytes;
  if (!use_split_path(a)) return 0;
  const size_t per_partial = 32 + (size_t)(a.query_heads / a.kv_heads) * a.head_dim;
  const uint32_t slots = balanced_split_slots(a);
  if (slots != 0) return (size_t)a.kv_heads * slots * per_partial * sizeof(float);
  return (size_t)a.batches * a.kv_heads * split_chunks(a) * per_partial * sizeof(float);
}

bool q8_attention_can_project(const Q8AttentionArgs &a) {
  return a.head_dim == 64 && !use_dense_copy_path(a) && use_split_path(a) && a.projected_width != 0 &&
         a.projected_width <= 1024 && a.projection.weight != nullptr && a.projection.scale != nullptr &&
         (reinterpret_cast<uintptr_t>(a.projection.weight) & 15) == 0;
}

hipError_t launch_q8_attention(const Q8AttentionArgs &a, hipStream_t stream) {
  if (a.projected != nullptr && !q8_attention_can_project(a)) return hipErrorInvalidValue;
  if (use_dense_copy_path(a)) {
    if (a.batches == 0 || a.query_heads == 0) return hipSuccess;
    const DenseCopyPlan plan = dense_copy_plan(a, a.workspace);
    // (a workspace that is not 16-byte aligned - none the runtime hands out is - sends the dense launch to its row kernel)
    if (a.workspace == nullptr || a.workspace_bytes < plan.total_bytes) return hipErrorInvalidValue;
    const uint64_t threads = (uint64_t)a.batches * a.kv_heads * plan.dense.key_length * (a.head_dim / 8);
    if ((threads + 255) / 256 > 0x7fffffffull) return hipErrorInvalidValue;
    uint8_t *base = static_cast<uint8_t *>(a.workspace);
    hipLaunchKernelGGL(q8_context_as_halves_kernel, dim3((uint32_t)((threads + 255) / 256), 2), dim3(256), 0, stream, a,
                       reinterpret_cast<uint16_t *>(base), reinterpret_cast<uint16_t *>(base + plan.operand_bytes));
    return launch_dense_attention(plan.dense, stream);
  }
  if (use_split_path(a)) {
    const uint32_t chunks = split_chunks(a);
    const uint32_t chunk_tokens = split_chunk_tokens(a);
    if (a.workspace == nullptr || a.workspace_bytes < q8_attention_workspace_bytes(a))
      return hipErrorInvalidValue;
    const uint32_t waves = std::min<uint32_t>(a.kv_heads, kSplitMaxWaves);
    const uint32_t slots = balanced_split_slots(a);
    const uint32_t head_groups = (a.kv_heads + kSplitMaxWaves - 1) / kSplitMaxWaves;
    const dim3 grid(slots != 0 ? slots : chunks, head_groups, slots != 0 ? 1 : a.batches);
    const dim3 block(waves * 64);
    const dim3 merge_grid(a.query_heads, a.batches);
    const bool small_pool = a.pool_bytes > 0 && a.pool_bytes <= 0xffffffffull;
    const bool aligned16 = a.token_stride % 16 == 0 && a.key_offset % 16 == 0 &&
                           (reinterpret_cast<uintptr_t>(a.pool) & 15) == 0;
    const auto launch_split = [&](auto dim_tag) {
      constexpr int D = decltype(dim_tag)::value;
      if (small_pool && aligned16)
        hipLaunchKernelGGL((q8_attention_split_kernel<D, true, true>), grid, block, 0, stream, a, chunks, chunk_tokens, slots);
      else if (small_pool)
        hipLaunchKernelGGL((q8_attention_split_kernel<D, true, false>), grid, block, 0, stream, a, chunks, chunk_tokens, slots);
      else if (aligned16)
        hipLaunchKernelGGL((q8_attention_split_kernel<D, false, true>), grid, block, 0, stream, a, chunks, chunk_tokens, slots);
      else
        hipLaunchKernelGGL((q8_attention_split_kernel<D, false, false>), grid, block, 0, stream, a, chunks, chunk_tokens, slots);
      if constexpr (D == 64) {
        if (a.projected != nullptr) {
          if (a.projected_width <= 640)
            hipLaunchKernelGGL((q8_attention_merge_kernel<64, 5>), merge_grid, dim3(kMergeSlices * 64), 0, stream, a, chunks,
                               chunk_tokens, slots);
          else
            hipLaunchKernelGGL((q8_attention_merge_kernel<64, 8>), merge_grid, dim3(kMergeSlices * 64), 0, stream, a, chunks,
                               chunk_tokens, slots);
          return;
        }
      }
      hipLaunchKernelGGL(q8_attention_merge_kernel<D>, merge_grid, dim3(kMergeSlices * D), 0, stream, a, chunks,
                         chunk_tokens, slots);
    };
    if (a.head_dim == 256)
      launch_split(std::integral_constant<int, 256>{});
    else if (a.head_dim == 128)
      launch_split(std::integral_constant<int, 128>{});
    else
      launch_split(std::integral_constant<int, 64>{});
    return hipGetLastError();
  }
  const uint32_t q_len = a.query_length == 0 ? 1 : a.query_length;
  const uint32_t rows = a.batches * a.query_heads * q_len;
  if (rows == 0) return hipSuccess;
  const dim3 grid((rows + kGeneralWaves - 1) / kGeneralWaves), block(kGeneralWaves * 64);
  const bool aligned = ((reinterpret_cast<uintptr_t>(a.pool) | a.token_stride | a.key_offset | a.value_offset) & 3) == 0;
  if (aligned)
    hipLaunchKernelGGL(q8_attention_general_kernel<true>, grid, block, 0, stream, a);
  else
    hipLaunchKernelGGL(q8_attention_general_kernel<false>, grid, block, 0, stream, a);
  return hipGetLastError();
}

}  // namespace llmopt
