// Dense fp16 attention (prefill and any other non-paged attention) for gfx950.
//
// Contract: llmopt_attention_f16 / llmopt_attention_f16_simd_h<D>
// (lib/metal_attention_source.ml:239-347, AttentionParams :251-256): query
// [b, h, q, D] head-major, key [b, kvh, L, D] head-major, value head-major or
// token-major [b, L, kvh, D], optional mask [mb, mh, q, L] (bool: nonzero
// allowed; half: >= 0 allowed), causal limit key <= past_length + q, GQA
// kv_head = head / (h / kvh), output head-major [b, h, q, D] or token-major
// [b, q, h, D]; a row with no allowed key is zero.  Scores and softmax in fp32.
//
//  * dense_attention_tile32_kernel<D> (D = 64, 128): 32 x 32 wave tiles on
//    v_mfma_f32_32x32x16_f16 over K / V stages shared through LDS; described at the kernel.
//  * dense_attention_rows_kernel: one wave per output row, serial over the keys
//    (any D up to 512, every option); the direct restatement.
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

__device__ __forceinline__ float lanes_xor_max(float value, int mask) {
  const int lane = (int)(threadIdx.x & 63);
  const float other = __builtin_bit_cast(
      float, __builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __builtin_bit_cast(int, value)));
  return fmaxf(value, other);
}

__device__ __forceinline__ float lanes_xor_sum(float value, int mask) {
  const int lane = (int)(threadIdx.x & 63);
  const float other = __builtin_bit_cast(
      float, __builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __builtin_bit_cast(int, value)));
  return value + other;
}

__device__ __forceinline__ bool mask_allows(const DenseAttentionArgs &a, uint32_t batch, uint32_t head,
                                            uint32_t query_position, uint32_t key_position) {
  const uint32_t mask_batch = a.mask_batches == 1 ? 0 : batch;
  const uint32_t mask_head = a.mask_heads == 1 ? 0 : head;
  const size_t index =
      (((size_t)mask_batch * a.mask_heads + mask_head) * a.query_length + query_position) * a.key_length +
      key_position;
  if (a.mask_dtype == 2) return half_bits_to_float(reinterpret_cast<const uint16_t *>(a.mask)[index]) >= 0.0f;
  return a.mask[index] != 0;
}

constexpr int kWavesPerBlock = 4;  // consecutive 32-row slabs of one head

// ---- 32 x 32 wave tiles ---------------------------------------------------------------------------
//
// The four waves of a workgroup - 128 consecutive query rows of one head - walk the same keys, so
// K and V go global -> LDS once per workgroup, 64 keys a stage and a stage ahead of the
// arithmetic, as direct copies that pass no registers (global_load_lds_dwordx4: 64 lanes x 16
// bytes land at consecutive LDS addresses, i.e. whole K / V rows side by side), one barrier per
// stage.  The 16-byte pieces of a row are stored XOR-swizzled by the key so that operand reads
// (one piece of many different keys per cycle) hit different banks.  The arithmetic runs on
// v_mfma_f32_32x32x16_f16: a wave owns ONE tile of 32 query rows and walks the keys 32 at a time.
//
//  * S^T = K Q^T: A = K (rows = keys), B = Q^T (columns = query rows), D / 16 chained MFMAs.  Lane
//    (j = lane % 32, half = lane / 32) ends with the sixteen scores of query row j and keys
//    (r / 4) * 8 + half * 4 + r % 4, r = 0..15: one row per lane, so the running maximum and sum
//    are per-lane scalars and the two lanes of a row meet once per tile (maximum) and once at the
//    end (sum).
//  * O^T += V^T P^T in two steps of 16 keys: the B operand of step s is the lane's own
//    probabilities r = 8 s .. 8 s + 7 as halves, no exchange between lanes; the A operand row i
//    of block jj is head_dim 32 jj + i: eight keys at one head_dim, i.e. a column of the V tile,
//    which ds_read_b64_tr_b16 delivers straight from the row-major stage.  In that instruction
//    every lane names a 64-bit chunk (four halves) and lane 4 q + c of a group of sixteen receives
//    element c of the chunks named by lanes q, 4 + q, 8 + q, 12 + q of its group: with lane 4 e + q
//    naming (key e, head_dim chunk q) a lane gets four keys of one head_dim, and two reads make an
//    operand.  V rows are stored with their 16-byte pieces XOR-ed by twice the key, so that the
//    four rows a group touches lie in different banks.
//
// Against the 16-key tiles above: the legacy 16x16x16 MFMA of the P V product runs at half the
// rate of the x32 shapes (16 cycles for 8192 flops), and the per-tile bookkeeping of the online
// softmax (exchanges, rescaling, the alpha exponential) is paid once per 32 keys and 32 rows
// instead of four times.
// WAVES x 32 query rows per workgroup, STAGE_KEYS keys per LDS stage (launched as 4 x 64: 64 KB at
// D = 128, two workgroups per CU).
// MASK: 0 no mask, 1 a mask of bytes, 2 of halves, 3 the mask as one bit per (row, key), which the pass over the
// mask ahead of this kernel leaves (every score is then tested; without one the instantiation carries
// nothing of it).
// KEYSPLIT: the four waves of a workgroup share ONE slab of 32 query rows and take a quarter of every
// 128-key stage each; their partial results meet in LDS at the end.  For launches with fewer
// workgroups than CUs, which last as long as one wave's walk over all the keys of the last slab: the
// walk is a quarter as long and there are four times as many workgroups.
template <int D>
constexpr int tile32_waves_per_simd() {
  return D <= 128 ? 2 : 1;
}

// PAIR: two groups of WAVES waves share the slab's query rows and take alternate stages of its keys (each
// group with its own two LDS stages); group 1 hands its maxima, denominators and sums to group 0 through
// LDS at the end.  For launches of one or two workgroups per CU: such a launch lasts as long as its
// longest slab's walk over the keys, wave by wave, and the walk is half as long this way.
template <int D, int WAVES, int STAGE_KEYS, int MASK, bool KEYSPLIT = false, bool PAIR = false>
__global__ __launch_bounds__(WAVES * 64 * (PAIR ? 2 : 1))
    __attribute__((amdgpu_waves_per_eu(tile32_waves_per_simd<D>(), tile32_waves_per_simd<D>()))) void
    dense_attention_tile32_kernel(DenseAttentionArgs a) {
  constexpr bool MASKED = MASK != 0;
  static_assert(!PAIR || !KEYSPLIT, "one way of splitting the keys at a time");
  constexpr int KSTEPS = D / 16;  // score MFMAs per key tile
  constexpr int JJ = D / 32;      // adjacent head_dim values per lane and key = output blocks
  constexpr int ROW_BYTES = D * 2;
  constexpr int PIECES = ROW_BYTES / 16;
  constexpr int KEYS_PER_COPY = 64 / PIECES;
  constexpr int COPIES = STAGE_KEYS / KEYS_PER_COPY / WAVES;
  constexpr int STAGE_BYTES = STAGE_KEYS * ROW_BYTES;
  static_assert(JJ == 2 || JJ == 4 || JJ == 8, "head_dim 64, 128 or 256");
  // V rows are swizzled by twice the key within the row's first sixteen pieces at most: reads 8 and 16 keys
  // further down must find the same swizzle
  constexpr int VMASK = (PIECES < 16 ? PIECES : 16) - 1;
  static_assert((STAGE_KEYS == 128 || STAGE_KEYS == 64 || STAGE_KEYS == 32) && COPIES >= 1 &&
                    COPIES * KEYS_PER_COPY * WAVES == STAGE_KEYS,
                "stage");
  static_assert(!KEYSPLIT || STAGE_KEYS == 32 * WAVES, "a tile of every stage per wave");
  constexpr int ROWS = KEYSPLIT ? 32 : WAVES * 32;  // query rows per workgroup
  extern __shared__ __attribute__((aligned(16))) unsigned char stage_lds[];  // [group][2 stages][K | V]
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave_of_all = threadIdx.x >> 6;
  const uint32_t group = PAIR ? wave_of_all / WAVES : 0;  // which of the two halves of the stages
  const uint32_t wave = PAIR ? wave_of_all % WAVES : wave_of_all;
  unsigned char *group_lds = stage_lds + group * 4 * STAGE_BYTES;
  const uint32_t row_lane = lane & 31;
  const uint32_t half = lane >> 5;
  // Which (row slab, head, batch) this workgroup takes.  The grid is one-dimensional; rank 0.. runs over
  // the slabs from the last (the most keys under a causal limit) to the first, heads and batches within a
  // slab.  Workgroups go to the XCDs round-robin and, within an XCD, to its CUs in order: XCD x takes
  // ranks x, x + 8, .. (every XCD gets every length), and of each run of two workgroups per CU the second
  // half is taken backwards, so that the CU that got the longest of the run also gets the shortest.
  // Without this a launch of as many workgroups as the device holds - 16 slabs x 32 heads at 2048 tokens -
  // puts the two longest on one CU and all of one length on one XCD, and lasts as long as they do.
  const uint32_t slabs = (a.query_length + ROWS - 1) / ROWS;
  const uint32_t per_slab = a.heads * a.batches;
  uint32_t rank = blockIdx.x;
  // (a mask is taken for a causal one as far as the order goes: later rows see more keys)
  const bool longest_first = a.causal || MASKED;
  if (longest_first && gridDim.x % 8 == 0 && a.cus_per_xcd > 0) {
    const uint32_t xcd = blockIdx.x % 8, position = blockIdx.x / 8, run = 2 * a.cus_per_xcd;
    const uint32_t start = position / run * run, within = position % run;
    uint32_t taken = position;
    // (PAIR: a CU holds one workgroup at a time and takes the next in rank order when it is done)
    if (!PAIR && within >= a.cus_per_xcd && start + run <= gridDim.x / 8)
      taken = start + a.cus_per_xcd + (run - 1 - within);
    rank = taken * 8 + xcd;
  }
  const uint32_t slab = longest_first ? slabs - 1 - rank / per_slab : rank / per_slab;
  const uint32_t head = rank % per_slab % a.heads;
  const uint32_t batch = rank % per_slab / a.heads;
  const uint32_t q0 = KEYSPLIT ? slab * 32 : (slab * WAVES + wave) * 32;
  const bool has_rows = q0 < a.query_length;  // a wave without rows still copies and meets the barriers
  const uint32_t kv_heads = a.kv_heads > 0 ? a.kv_heads : a.heads;
  const uint32_t kv_head = kv_heads < a.heads ? head / (a.heads / kv_heads) : head;
  constexpr bool masked = MASKED;
  const uint32_t L = a.key_length;

  // B operand of the score MFMAs: Q[row = row_lane][d = ks * 16 + half * 8 ..]; rows past the end repeat the last
  h8_t q_frag[KSTEPS];
  {
    const uint32_t row = min(q0 + row_lane, a.query_length - 1);
    const uint16_t *q_row = a.query + (((size_t)batch * a.heads + head) * a.query_length + row) * D;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
      q_frag[ks] = __builtin_bit_cast(h8_t, *reinterpret_cast<const uint4 *>(q_row + ks * 16 + half * 8));
  }
  [[maybe_unused]] const uint16_t *key_base = a.key + ((size_t)batch * kv_heads + kv_head) * L * D;
  [[maybe_unused]] const size_t value_row_stride = a.token_first_value ? (size_t)kv_heads * D : D;
  [[maybe_unused]] const uint16_t *value_base = a.token_first_value
                                   ? a.value + ((size_t)batch * L * kv_heads + kv_head) * D
                                   : a.value + ((size_t)batch * kv_heads + kv_head) * L * D;

  // ---- mask ----
  // A lane's sixteen scores of a tile are four runs of four consecutive keys of one query row.  Their
  // mask values are requested a stage ahead, for every lane at clamped addresses (a load under a
  // per-score test is waited for where it stands: sixteen trips to memory per tile), as one dword
  // (bool) or two (f16) per run when rows of the mask are a multiple of four keys, else element by
  // element; a tile whose 32 x 32 mask values allow nothing is skipped whole.
  constexpr int TILES = KEYSPLIT ? 1 : STAGE_KEYS / 32;  // tiles of a stage this wave works on
  struct MaskRaw {
    uint32_t w[MASK == 2 ? 8 : MASK == 1 ? 4 : 1];  // (bits: the 32 keys of the lane's row in one dword)
  };
  [[maybe_unused]] const size_t mask_row_index =
      masked ? ((size_t)(a.mask_batches == 1 ? 0 : batch) * a.mask_heads + (a.mask_heads == 1 ? 0 : head)) *
                       a.query_length + min(q0 + row_lane, a.query_length - 1)
             : 0;
  [[maybe_unused]] const size_t mask_row = mask_row_index * L;
  [[maybe_unused]] const bool mask_runs =
      masked && L % 4 == 0 && L >= 4 && reinterpret_cast<uintptr_t>(a.mask) % 8 == 0;  // the same for every lane
  [[maybe_unused]] auto mask_request = [&](uint32_t key0, MaskRaw &raw) __attribute__((always_inline)) {
    if constexpr (MASK == 3) {
      raw.w[0] = a.mask_bits[mask_row_index * a.mask_words_per_row + (min(key0, L - 1) >> 5)];
    } else if constexpr (MASK == 2) {
      {
        const uint16_t *row = reinterpret_cast<const uint16_t *>(a.mask) + mask_row;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t key = key0 + g * 8 + half * 4;
          if (mask_runs) {
            const uint2 run = *reinterpret_cast<const uint2 *>(row + min(key, L - 4));
            raw.w[2 * g] = run.x;
            raw.w[2 * g + 1] = run.y;
          } else {
            raw.w[2 * g] = (uint32_t)row[min(key, L - 1)] | ((uint32_t)row[min(key + 1, L - 1)] << 16);
            raw.w[2 * g + 1] = (uint32_t)row[min(key + 2, L - 1)] | ((uint32_t)row[min(key + 3, L - 1)] << 16);
          }
        }
      }
    } else if constexpr (MASK == 1) {
      {
        const uint8_t *row = a.mask + mask_row;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t key = key0 + g * 8 + half * 4;
          if (mask_runs)
            raw.w[g] = *reinterpret_cast<const uint32_t *>(row + min(key, L - 4));
          else
            raw.w[g] = (uint32_t)row[min(key, L - 1)] | ((uint32_t)row[min(key + 1, L - 1)] << 8) |
                       ((uint32_t)row[min(key + 2, L - 1)] << 16) | ((uint32_t)row[min(key + 3, L - 1)] << 24);
        }
      }
    }
  };
  // bit r: the mask allows score r (keys past the end read a clamped element; they fail the range test anyway).
  // With whole runs a run that starts past L - 4 was read from L - 4: its keys are all past the end.
  [[maybe_unused]] auto mask_bits = [&](const MaskRaw &raw) __attribute__((always_inline)) {
    uint32_t bits = 0;
    if constexpr (MASKED) {
      // Most tiles of the masks a prefill builds are allowed as a whole, and their values are all +0.0
      // (halves) or all 1 (bytes): one OR / AND over the lane's words and a vote say so, and only the
      // tiles the mask's edge runs through pay for the value-by-value conversion.
      if constexpr (MASK == 3) {
        // bit k of the dword is key key0 + k of this lane's row; score r is key (r / 4) * 8 + half * 4 + r % 4
        if (__builtin_amdgcn_ballot_w64(raw.w[0] != 0xffffffffu) == 0) return 0xffffu;
#pragma unroll
        for (int g = 0; g < 4; ++g) bits |= ((raw.w[0] >> (8 * g + 4 * half)) & 0xfu) << (4 * g);
        return bits;
      } else {
        bool plain;
        if constexpr (MASK == 2) {
          uint32_t any = 0;
#pragma unroll
          for (int i = 0; i < 8; ++i) any |= raw.w[i];
          plain = any == 0;
        } else {
          plain = raw.w[0] == 0x01010101u && raw.w[1] == 0x01010101u && raw.w[2] == 0x01010101u && raw.w[3] == 0x01010101u;
        }
        if (__builtin_amdgcn_ballot_w64(!plain) == 0) return 0xffffu;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          bool allowed;
          if constexpr (MASK == 2)
            allowed = half_bits_to_float((uint16_t)(raw.w[2 * (r >> 2) + ((r & 3) >> 1)] >> (16 * (r & 1)))) >= 0.0f;
          else
            allowed = ((raw.w[r >> 2] >> (8 * (r & 3))) & 0xffu) != 0;
          bits |= allowed ? (1u << r) : 0u;
        }
      }
    }
    return bits;
  };

  const float score_scale = a.scale * 1.4426950408889634f;  // softmax in base 2
  float running_max = -INFINITY, running_sum = 0.0f;        // of this lane's row; the sum over this lane's keys
  f16x_t out_acc[JJ];  // O^T[d = 32 jj + (r / 4) * 8 + half * 4 + r % 4][row = row_lane]
#pragma unroll
  for (int jj = 0; jj < JJ; ++jj)
#pragma unroll
    for (int r = 0; r < 16; ++r) out_acc[jj][r] = 0.0f;

  uint32_t key_end = has_rows ? L : 0;
  if (a.causal && has_rows) {
    const uint32_t last_row = min(q0 + 32, a.query_length) - 1;
    key_end = min((uint64_t)L, (uint64_t)a.past_length + last_row + 1);
  }
  uint32_t group_key_end = L;
  if (a.causal) {
    const uint32_t group_q0 = slab * ROWS;
    const uint32_t last_row = min(group_q0 + ROWS, a.query_length) - 1;
    group_key_end = min((uint64_t)L, (uint64_t)a.past_length + last_row + 1);
  }
  const uint32_t stages = (group_key_end + STAGE_KEYS - 1) / STAGE_KEYS;
  auto copy_stage = [&](uint32_t stage, uint32_t buffer) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t buffer_base =
        (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)group_lds + buffer * 2 * STAGE_BYTES;
    const uint32_t row_in_copy = lane / PIECES, piece = lane % PIECES;
#pragma unroll
    for (int c = 0; c < COPIES; ++c) {
      const uint32_t copy = wave * COPIES + c;
      const uint32_t local = copy * KEYS_PER_COPY + row_in_copy;    // row within the stage
      const uint32_t key = min(stage * STAGE_KEYS + local, L - 1);  // rows past the end repeat the last one
      const uint16_t *k_src = key_base + (size_t)key * D + ((piece ^ (local & (PIECES - 1))) * 8);
      const uint16_t *v_src = value_base + (size_t)key * value_row_stride + ((piece ^ ((2 * local) & VMASK)) * 8);
      const uint32_t k_dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)(buffer_base + copy * 1024));
      const uint32_t v_dst = k_dst + STAGE_BYTES;
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(k_src), "s"(k_dst) : "memory");
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(v_src), "s"(v_dst) : "memory");
    }
#endif
  };
  auto stage_landed = [&]() __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's copies; the barrier covers the others'
    __syncthreads();
  };
  // What this lane names in a transposing read of V: key (lane / 32) * 4 + (lane % 16) / 4 of the
  // eight keys of a read, head_dim chunk 8 jj + ((lane / 16) % 2) * 4 + lane % 4 of block jj (the
  // multiples of 16 and 8 keys that steps and reads add leave the swizzle of a row unchanged).
  uint32_t v_lane_offset[JJ];
  {
    const uint32_t group = lane >> 4, p = lane & 15;
    const uint32_t key_in_read = (group >> 1) * 4 + (p >> 2);
    const uint32_t chunk = (group & 1) * 4 + (p & 3);
#pragma unroll
    for (int jj = 0; jj < JJ; ++jj)
      v_lane_offset[jj] = key_in_read * ROW_BYTES +
                          (((jj * 4 + (chunk >> 1)) ^ ((2 * key_in_read) & VMASK)) * 16) + (chunk & 1) * 8;
  }
  // first key of this wave's tile t of a stage
  auto tile_key0 = [&](uint32_t stage, int t) __attribute__((always_inline)) {
    return stage * STAGE_KEYS + (KEYSPLIT ? wave * 32 : (uint32_t)t * 32);
  };
  // With a mask, the stages of keys that have anything for this slab of rows come from a map a pass
  // over the mask left (one byte per mask row group, slab and stage): wave 0 turns the slab's bytes
  // into the list of its live stages, and the loop below walks that list - a stage the mask forbids
  // costs nothing.  Without a map (no scratch given, or more stages than the list holds) every stage
  // is walked and only its arithmetic is skipped.
  constexpr uint32_t kMaxLive = 2048;
  [[maybe_unused]] __shared__ uint16_t live_list[MASKED ? kMaxLive : 1];
  [[maybe_unused]] __shared__ uint32_t live_count_lds;
  bool listed = false;
  uint32_t walk = stages;  // stages to walk
  if constexpr (MASKED) {
    listed = a.stage_map != nullptr && stages <= kMaxLive;
    if (listed) {
      const uint32_t map_stride = (L + STAGE_KEYS - 1) / STAGE_KEYS;  // a byte per stage
      const uint32_t mask_group = (a.mask_batches == 1 ? 0 : batch) * a.mask_heads + (a.mask_heads == 1 ? 0 : head);
      const uint8_t *map = a.stage_map + ((size_t)mask_group * slabs + slab) * map_stride;
      if (wave_of_all == 0) {
        uint32_t count = 0;
        for (uint32_t base = 0; base < stages; base += 64) {
          const uint32_t stage = base + lane;
          const bool live = stage < stages && map[min(stage, stages - 1)] != 0;
          const uint64_t votes = __builtin_amdgcn_ballot_w64(live);
          if (live) live_list[count + __builtin_popcountll(votes & ((1ull << lane) - 1))] = (uint16_t)stage;
          count += (uint32_t)__builtin_popcountll(votes);
        }
        if (lane == 0) live_count_lds = count;
      }
      __syncthreads();
      walk = live_count_lds;
    }
  }
  auto stage_at = [&](uint32_t index) __attribute__((always_inline)) -> uint32_t {
    if constexpr (MASKED) return listed ? (uint32_t)live_list[index] : index;
    return index;
  };
  // step s of the loop below works on entry walk_index(s) of the walk (PAIR: the groups take alternate entries)
  const uint32_t steps = PAIR ? (walk + 1) / 2 : walk;
  auto walk_index = [&](uint32_t step) __attribute__((always_inline)) { return PAIR ? 2 * step + group : step; };
  MaskRaw mask_raw[TILES];
  if (walk > 0) {
    if (walk_index(0) < walk) {
      const uint32_t first = stage_at(walk_index(0));
      if constexpr (MASKED) {
#pragma unroll
        for (int t = 0; t < TILES; ++t) mask_request(tile_key0(first, t), mask_raw[t]);
      }
      copy_stage(first, 0);
    }
    stage_landed();
  }

  // scores of one tile of 32 keys: k_tile = its first row in the stage, local0 = that row's index in the stage
  auto tile_scores = [&](const unsigned char *k_tile, uint32_t local0) __attribute__((always_inline)) {
    f16x_t score;
#pragma unroll
    for (int r = 0; r < 16; ++r) score[r] = 0.0f;
    const uint32_t local = local0 + row_lane;
    const unsigned char *k_row = k_tile + row_lane * ROW_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const h8_t k_frag = __builtin_bit_cast(
          h8_t, *reinterpret_cast<const uint4 *>(k_row + (((ks * 2 + half) ^ (local & (PIECES - 1))) * 16)));
      score = __builtin_amdgcn_mfma_f32_32x32x16_f16(k_frag, q_frag[ks], score, 0, 0, 0);
    }
    return score;
  };
  // softmax update and P V product of one tile from its scores; v_tile = its first V row in the stage
  auto tile_update = [&](uint32_t key0, f16x_t score, const unsigned char *v_tile, uint32_t allowed_bits)
                         __attribute__((always_inline)) {
    // a tile of existing keys, all below the causal limit of the wave's first row, of existing
    // rows and without a mask needs no per-score test.  Maxima are taken over the scores as the MFMAs left them; the
    // scale (positive) goes into the exponent's multiply-add.
    // (with a mask: when it allows all 32 x 32 scores of the tile)
    const bool interior = (!masked || __builtin_amdgcn_ballot_w64(allowed_bits != 0xffffu) == 0) && key0 + 32 <= L &&
                          q0 + 32 <= a.query_length && (!a.causal || key0 + 31 <= a.past_length + q0);
    float tile_max = -INFINITY;
    if (interior) {
#pragma unroll
      for (int r = 0; r < 16; ++r) tile_max = fmaxf(tile_max, score[r]);
    } else {
      const uint32_t row = q0 + row_lane;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t key = key0 + (r >> 2) * 8 + half * 4 + (r & 3);
        bool allowed = key < L && row < a.query_length;
        if (a.causal) allowed = allowed && key <= a.past_length + row;
        if constexpr (masked) allowed = allowed && ((allowed_bits >> r) & 1u) != 0;
        score[r] = allowed ? score[r] : -INFINITY;
        tile_max = fmaxf(tile_max, score[r]);
      }
    }
    tile_max = lanes_xor_max(tile_max, 32);
    const float new_max = fmaxf(running_max, tile_max);
    // no allowed key yet: keep every exponent finite (the probabilities are zero anyway)
    const float reference = new_max == -INFINITY ? 0.0f : new_max;
    const float alpha = __builtin_amdgcn_exp2f((running_max - reference) * score_scale);  // 0 while running_max is -inf
    running_max = new_max;
    const float scaled_reference = reference * score_scale;
    h8_t p_frag[2];
    float tile_sum = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float p = __builtin_amdgcn_exp2f(fmaf(score[r], score_scale, -scaled_reference));
      tile_sum += p;
      p_frag[r >> 3][r & 7] = (_Float16)p;
    }
    running_sum = running_sum * alpha + tile_sum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int jj = 0; jj < JJ; ++jj)
#pragma unroll
        for (int r = 0; r < 16; ++r) out_acc[jj][r] *= alpha;
    }
    typedef short s4_t __attribute__((ext_vector_type(4)));
    typedef s4_t __attribute__((address_space(3))) * lds_chunk_t;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int jj = 0; jj < JJ; ++jj) {
        const unsigned char *source = v_tile + v_lane_offset[jj] + s * 16 * ROW_BYTES;
        const s4_t keys_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_chunk_t)source);
        const s4_t keys_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_chunk_t)(source + 8 * ROW_BYTES));
        const h8_t operand = __builtin_bit_cast(
            h8_t, make_uint4(__builtin_bit_cast(uint2, keys_lo).x, __builtin_bit_cast(uint2, keys_lo).y,
                             __builtin_bit_cast(uint2, keys_hi).x, __builtin_bit_cast(uint2, keys_hi).y));
        out_acc[jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(operand, p_frag[s], out_acc[jj], 0, 0, 0);
      }
  };

  // The tiles of a stage.  Two: both score chains go to the matrix pipe first, so the second runs
  // while the vector unit works on the first tile's softmax.
  for (uint32_t step = 0; step < steps; ++step) {
    const uint32_t index = walk_index(step);
    const bool active = index < walk;  // (PAIR: the last step may have an entry for group 0 only)
    const uint32_t stage = active ? stage_at(index) : 0;
    // The mask values of this stage were requested a stage ago and landed with that stage's copies
    // (stage_landed waits for everything): they are turned into bits before anything new is
    // requested, so that no wait for them stands behind the next stage's copies.
    uint32_t allowed_bits[TILES];
    bool live[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      allowed_bits[t] = MASKED ? mask_bits(mask_raw[t]) : 0xffffu;
      live[t] = active && tile_key0(stage, t) < key_end &&
                (!MASKED || __builtin_amdgcn_ballot_w64(allowed_bits[t] != 0) != 0);
    }
    if (walk_index(step + 1) < walk) {
      const uint32_t next = stage_at(walk_index(step + 1));
      copy_stage(next, (step + 1) & 1);  // into the buffer every wave left at the last barrier
      if constexpr (MASKED) {
#pragma unroll
        for (int t = 0; t < TILES; ++t) mask_request(tile_key0(next, t), mask_raw[t]);
      }
    }
    const unsigned char *k_stage = group_lds + (step & 1) * 2 * STAGE_BYTES;
    const unsigned char *v_stage = k_stage + STAGE_BYTES;
    if constexpr (KEYSPLIT) {
      if (live[0])
        tile_update(tile_key0(stage, 0), tile_scores(k_stage + wave * 32 * ROW_BYTES, wave * 32),
                    v_stage + wave * 32 * ROW_BYTES, allowed_bits[0]);
      stage_landed();
      continue;
    }
    const uint32_t key0 = stage * STAGE_KEYS;
    if constexpr (!MASKED && STAGE_KEYS == 64) {
      // (without a mask the second tile exists whenever the first does, except at the very end)
      if (active && key0 < key_end) {
        const f16x_t first_scores = tile_scores(k_stage, 0);
        const bool second = key0 + 32 < key_end;
        f16x_t second_scores = first_scores;
        if (second) second_scores = tile_scores(k_stage + 32 * ROW_BYTES, 32);
        tile_update(key0, first_scores, v_stage, 0xffffu);
        if (second) tile_update(key0 + 32, second_scores, v_stage + 32 * ROW_BYTES, 0xffffu);
      }
    } else if constexpr (STAGE_KEYS == 64) {
      f16x_t first_scores, second_scores;
      if (live[0]) first_scores = tile_scores(k_stage, 0);
      if (live[1]) second_scores = tile_scores(k_stage + 32 * ROW_BYTES, 32);
      if (live[0]) tile_update(key0, first_scores, v_stage, allowed_bits[0]);
      if (live[1]) tile_update(key0 + 32, second_scores, v_stage + 32 * ROW_BYTES, allowed_bits[1]);
    } else {
#pragma unroll
      for (int t = 0; t < TILES; ++t)
        if (live[t])
          tile_update(key0 + t * 32, tile_scores(k_stage + t * 32 * ROW_BYTES, t * 32), v_stage + t * 32 * ROW_BYTES,
                      allowed_bits[t]);
    }
    stage_landed();
  }
  if constexpr (KEYSPLIT) {
    // The waves' shares of the slab meet in LDS (the stages are read to the end: the loop's last
    // barrier): per wave the row maxima and denominators, and O^T as floats [d][row] - a lane's
    // values of one register are 32 neighbouring rows.  Thread t then folds row t % 32, head_dim
    // values (t / 32) * D / 8 .. of the four shares and stores them.
    float *share_out = reinterpret_cast<float *>(stage_lds);                  // [WAVES][D][32]
    float *share_max = share_out + WAVES * D * 32;                            // [WAVES][32]
    float *share_sum = share_max + WAVES * 32;                                // [WAVES][32]
    static_assert((WAVES * D * 32 + 2 * WAVES * 32) * sizeof(float) <= 4 * (size_t)STAGE_BYTES, "the shares fit the stages");
    const float wave_total = lanes_xor_sum(running_sum, 32);
    if (half == 0) {
      share_max[wave * 32 + row_lane] = running_max;
      share_sum[wave * 32 + row_lane] = wave_total;
    }
#pragma unroll
    for (int jj = 0; jj < JJ; ++jj)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        share_out[(wave * D + 32 * jj + (r >> 2) * 8 + half * 4 + (r & 3)) * 32 + row_lane] = out_acc[jj][r];
    __syncthreads();
    constexpr int PER_THREAD = D / 8;  // head_dim values per thread: 32 rows x 8 threads a row
    const uint32_t out_row_index = q0 + (threadIdx.x & 31);
    const uint32_t d0 = (threadIdx.x >> 5) * PER_THREAD;
    float best = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) best = fmaxf(best, share_max[w * 32 + (threadIdx.x & 31)]);
    float weight[WAVES], denominator = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float share = share_max[w * 32 + (threadIdx.x & 31)];
      weight[w] = share == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f((share - best) * score_scale);
      denominator += weight[w] * share_sum[w * 32 + (threadIdx.x & 31)];
    }
    if (out_row_index >= a.query_length) return;
    const float inverse = denominator != 0.0f ? 1.0f / denominator : 0.0f;
    uint16_t *out_row = a.token_first_output
                            ? a.output + (((size_t)batch * a.query_length + out_row_index) * a.heads + head) * D
                            : a.output + (((size_t)batch * a.heads + head) * a.query_length + out_row_index) * D;
#pragma unroll
    for (int e = 0; e < PER_THREAD; e += 4) {
      float value[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w)
          if (weight[w] != 0.0f) sum += weight[w] * share_out[(w * D + d0 + e + i) * 32 + (threadIdx.x & 31)];
        value[i] = sum * inverse;
      }
      uint2 packed;
      packed.x = (uint32_t)float_to_half_bits(value[0]) | ((uint32_t)float_to_half_bits(value[1]) << 16);
      packed.y = (uint32_t)float_to_half_bits(value[2]) | ((uint32_t)float_to_half_bits(value[3]) << 16);
      *reinterpret_cast<uint2 *>(out_row + d0 + e) = packed;
    }
    return;
  }
  if constexpr (PAIR) {
    // Group 1 leaves its share in LDS (the stages are read to the end: the loop's last barrier), register
    // by register with the lanes side by side, and group 0's wave of the same rows folds it into its own:
    // both hold the same (row, head_dim) in the same lane and register.
    float *share = reinterpret_cast<float *>(stage_lds) + wave * (JJ * 16 + 2) * 64;
    static_assert((size_t)WAVES * (JJ * 16 + 2) * 64 * sizeof(float) <= 8 * (size_t)STAGE_BYTES, "the shares fit the stages");
    if (group == 1) {
      share[lane] = running_max;
      share[64 + lane] = running_sum;
#pragma unroll
      for (int jj = 0; jj < JJ; ++jj)
#pragma unroll
        for (int r = 0; r < 16; ++r) share[(2 + jj * 16 + r) * 64 + lane] = out_acc[jj][r];
    }
    __syncthreads();
    if (group == 1) return;
    const float other_max = share[lane], other_sum = share[64 + lane];
    const float best = fmaxf(running_max, other_max);
    const float reference = best == -INFINITY ? 0.0f : best;
    const float own_weight = __builtin_amdgcn_exp2f((running_max - reference) * score_scale);  // 0 for a share without keys
    const float other_weight = __builtin_amdgcn_exp2f((other_max - reference) * score_scale);
    running_sum = running_sum * own_weight + other_sum * other_weight;
#pragma unroll
    for (int jj = 0; jj < JJ; ++jj)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        out_acc[jj][r] = out_acc[jj][r] * own_weight + share[(2 + jj * 16 + r) * 64 + lane] * other_weight;
  }
  if (!has_rows) return;

  const float total = lanes_xor_sum(running_sum, 32);
  const uint32_t row = q0 + row_lane;
  if (row >= a.query_length) return;
  const float inverse = total != 0.0f ? 1.0f / total : 0.0f;
  uint16_t *out_row = a.token_first_output ? a.output + (((size_t)batch * a.query_length + row) * a.heads + head) * D
                                           : a.output + (((size_t)batch * a.heads + head) * a.query_length + row) * D;
#pragma unroll
  for (int jj = 0; jj < JJ; ++jj)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // r = 4 g .. 4 g + 3 are adjacent in head_dim: one 8-byte store
      uint2 packed;
      packed.x = (uint32_t)float_to_half_bits(out_acc[jj][4 * g] * inverse) |
                 ((uint32_t)float_to_half_bits(out_acc[jj][4 * g + 1] * inverse) << 16);
      packed.y = (uint32_t)float_to_half_bits(out_acc[jj][4 * g + 2] * inverse) |
                 ((uint32_t)float_to_half_bits(out_acc[jj][4 * g + 3] * inverse) << 16);
      *reinterpret_cast<uint2 *>(out_row + 32 * jj + g * 8 + half * 4) = packed;
    }
}

// ---- the pass over a mask ahead of the attention kernel ---------------------------------------
//
// Leaves (1) the mask as one bit per (mask row, key), words_per_row dwords a row - what the attention
// kernel reads instead of the bytes or halves: one dword per lane and tile of 32 keys - and (2) one byte
// per (mask row group, slab of query rows, stage of keys) that says whether the mask allows anything
// there.  One workgroup per (two stages, slab, mask row group); a thread takes 64 consecutive keys of
// one row (every request out before the first value is looked at).  (One workgroup per eight stages and
// a bit per stage left three quarters of the CUs without work: 9.8 us for 2048 x 2048 halves.)
// rows_per_slab x stage_keys is the attention launch's geometry: 128 x 64, or 32 x 128 when the keys
// of a slab are split over the waves; the workgroup has rows_per_slab * stage_keys / 32 threads.
__global__ __launch_bounds__(256) void mask_bits_kernel(DenseAttentionArgs a, uint32_t rows_per_slab, uint32_t stage_keys,
                                                         uint32_t map_stride, uint32_t *bits_out, uint32_t words_per_row) {
  __shared__ uint32_t chunk_bits;
  const uint32_t chunk = blockIdx.x, slab = blockIdx.y, group = blockIdx.z;
  const uint32_t L = a.key_length;
  const uint32_t units = stage_keys / 32;  // 64-key units in two stages: 2 or 4
  const uint32_t unit = threadIdx.x % units, row = slab * rows_per_slab + threadIdx.x / units;
  const uint32_t key = chunk * 2 * stage_keys + unit * 64;
  if (threadIdx.x == 0) chunk_bits = 0;
  uint32_t word[2] = {0, 0};  // keys key .. key + 31, key + 32 .. key + 63
  const bool inside = row < a.query_length && key < L;
  if (inside) {
    const size_t first = ((size_t)group * a.query_length + row) * L + key;
    // 16-byte requests at whatever alignment the row has (rows of a suffix's mask start anywhere);
    // only a row's last, partial unit goes element by element
    typedef uint32_t unaligned_u32x4_t __attribute__((ext_vector_type(4), aligned(1)));
    const bool whole = key + 64 <= L;
    if (a.mask_dtype == 2) {
      const uint16_t *values = reinterpret_cast<const uint16_t *>(a.mask) + first;
      if (whole) {
        unaligned_u32x4_t piece[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) piece[i] = reinterpret_cast<const unaligned_u32x4_t *>(values)[i];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t four[4] = {piece[i].x, piece[i].y, piece[i].z, piece[i].w};
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const bool allowed = half_bits_to_float((uint16_t)(four[e >> 1] >> (16 * (e & 1)))) >= 0.0f;
            word[i >> 2] |= allowed ? 1u << ((i & 3) * 8 + e) : 0u;
          }
        }
      } else {
        for (uint32_t e = 0; e < 64 && key + e < L; ++e)
          word[e >> 5] |= half_bits_to_float(values[e]) >= 0.0f ? 1u << (e & 31) : 0u;
      }
    } else {
      const uint8_t *values = a.mask + first;
      if (whole) {
        unaligned_u32x4_t piece[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) piece[i] = reinterpret_cast<const unaligned_u32x4_t *>(values)[i];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t four[4] = {piece[i].x, piece[i].y, piece[i].z, piece[i].w};
#pragma unroll
          for (int e = 0; e < 16; ++e)
            word[i >> 1] |= ((four[e >> 2] >> (8 * (e & 3))) & 0xffu) != 0 ? 1u << ((i & 1) * 16 + e) : 0u;
        }
      } else {
        for (uint32_t e = 0; e < 64 && key + e < L; ++e) word[e >> 5] |= values[e] != 0 ? 1u << (e & 31) : 0u;
      }
    }
    uint32_t *out = bits_out + ((size_t)group * a.query_length + row) * words_per_row + (key >> 5);
    out[0] = word[0];
    out[1] = word[1];
  }
  __syncthreads();
  if ((word[0] | word[1]) != 0) atomicOr(&chunk_bits, 1u << (unit * 64 / stage_keys));
  __syncthreads();
  if (threadIdx.x < 2 && chunk * 2 + threadIdx.x < map_stride)
    a.stage_map[((size_t)group * gridDim.y + slab) * map_stride + chunk * 2 + threadIdx.x] =
        (uint8_t)((chunk_bits >> threadIdx.x) & 1u);
}

// ---- the mask of the speculative tree attention entries ---------------------------------------
struct TreeMaskArgs {
  uint8_t *mask;
  uint32_t query_length, key_length, past_length;
  uint32_t tree_masks[8];
};

__global__ __launch_bounds__(256) void tree_mask_kernel(TreeMaskArgs a) {
  const uint64_t index = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (index >= (uint64_t)a.query_length * a.key_length) return;
  const uint32_t query = (uint32_t)(index / a.key_length), key = (uint32_t)(index % a.key_length);
  bool allowed = key < a.past_length;
  if (!allowed) {
    const uint32_t draft = key - a.past_length;
    uint32_t bits = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) bits = query == (uint32_t)i ? a.tree_masks[i] : bits;
    allowed = draft < a.query_length && draft < 32 && ((bits >> draft) & 1u) != 0;
  }
  a.mask[index] = allowed ? 1 : 0;
}

// ---- row-serial kernel (every other configuration) ---------------------------

constexpr int kMaxFragments = 8;  // head_dim <= 512

__global__ __launch_bounds__(256) void dense_attention_rows_kernel(DenseAttentionArgs a) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row_index = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t rows = a.batches * a.heads * a.query_length;
  if (row_index >= rows) return;
  const uint32_t query_position = row_index % a.query_length;
  const uint32_t head = (row_index / a.query_length) % a.heads;
  const uint32_t batch = row_index / (a.query_length * a.heads);
  const uint32_t kv_heads = a.kv_heads > 0 ? a.kv_heads : a.heads;
  const uint32_t kv_head = kv_heads < a.heads ? head / (a.heads / kv_heads) : head;
  const uint32_t D = a.head_dim;
  const uint32_t fragments = (D + 63) / 64;
  const bool masked = a.mask != nullptr && a.mask_batches > 0;
  const uint16_t *q_row = a.query + (size_t)row_index * D;

  float q[kMaxFragments], result[kMaxFragments];
#pragma unroll
  for (int f = 0; f < kMaxFragments; ++f) {
    result[f] = 0.0f;
    const uint32_t d = f * 64 + lane;
    q[f] = (uint32_t)f < fragments && d < D ? half_bits_to_float(q_row[d]) : 0.0f;
  }
  float maximum = -INFINITY, denominator = 0.0f;
  for (uint32_t key_position = 0; key_position < a.key_length; ++key_position) {
    if (a.causal && key_position > a.past_length + query_position) break;
    if (masked && !mask_allows(a, batch, head, query_position, key_position)) continue;
    const uint16_t *k_row = a.key + (((size_t)batch * kv_heads + kv_head) * a.key_length + key_position) * D;
    const uint16_t *v_row =
        a.token_first_value
            ? a.value + (((size_t)batch * a.key_length + key_position) * kv_heads + kv_head) * D
            : a.value + (((size_t)batch * kv_heads + kv_head) * a.key_length + key_position) * D;
    float partial = 0.0f;
    float value[kMaxFragments];
#pragma unroll
    for (int f = 0; f < kMaxFragments; ++f) {
      if ((uint32_t)f >= fragments) break;
      const uint32_t d = f * 64 + lane;
      const bool inside = d < D;
      partial += inside ? q[f] * half_bits_to_float(k_row[d]) : 0.0f;
      value[f] = inside ? half_bits_to_float(v_row[d]) : 0.0f;
    }
    const float score = wave_sum(partial) * a.scale;
    const float new_max = fmaxf(maximum, score);
    const float alpha = __expf(maximum - new_max);  // 0 for the first allowed key
    const float p = __expf(score - new_max);
    denominator = denominator * alpha + p;
#pragma unroll
    for (int f = 0; f < kMaxFragments; ++f) {
      if ((uint32_t)f >= fragments) break;
      result[f] = result[f] * alpha + p * value[f];
    }
    maximum = new_max;
  }
  const float inverse = denominator != 0.0f ? 1.0f / denominator : 0.0f;
  uint16_t *out_row =
      a.token_first_output
          ? a.output + (((size_t)batch * a.query_length + query_position) * a.heads + head) * D
          : a.output + (size_t)row_index * D;
#pragma unroll
  for (int f = 0; f < kMaxFragments; ++f) {
    if ((uint32_t)f >= fragments) break;
    const uint32_t d = f * 64 + lane;
    if (d < D) out_row[d] = float_to_half_bits(result[f] * inverse);
  }
}

template <int D, int WAVES, int STAGE_KEYS, int MASK, bool KEYSPLIT, bool PAIR = false>
hipError_t launch_tile32_instance(uint32_t grid, const DenseAttentionArgs &a, hipStream_t stream) {
  constexpr size_t bytes = (PAIR ? 2 : 1) * 2 * 2 * (size_t)STAGE_KEYS * D * 2;  // two stages of K and V per group
  auto kernel = &dense_attention_tile32_kernel<D, WAVES, STAGE_KEYS, MASK, KEYSPLIT, PAIR>;
  if constexpr (bytes >= 64 * 1024) {
    static bool configured[kMaxDevices] = {};  // the attribute is per device function and device
    if (hipError_t status = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), (int)bytes, configured)) return status;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(WAVES * 64 * (PAIR ? 2 : 1)), bytes, stream, a);
  return hipGetLastError();
}

// mask: 0 none, 1 bytes, 2 halves, 3 bits
template <int D, int WAVES, int STAGE_KEYS, bool KEYSPLIT, bool PAIR = false>
hipError_t launch_tile32(int mask, uint32_t grid, const DenseAttentionArgs &a, hipStream_t stream) {
  if (mask == 3) return launch_tile32_instance<D, WAVES, STAGE_KEYS, 3, KEYSPLIT, PAIR>(grid, a, stream);
  if (mask == 2) return launch_tile32_instance<D, WAVES, STAGE_KEYS, 2, KEYSPLIT, PAIR>(grid, a, stream);
  if (mask == 1) return launch_tile32_instance<D, WAVES, STAGE_KEYS, 1, KEYSPLIT, PAIR>(grid, a, stream);
  return launch_tile32_instance<D, WAVES, STAGE_KEYS, 0, KEYSPLIT, PAIR>(grid, a, stream);
}

// Which kernel a launch takes and the slabs and stages it works in.
struct Tile32Geometry {
  bool tiled;       // the 32 x 32 tile kernel (else the row-serial one)
  bool key_split;   // 32-row slabs whose keys are split over the waves, 128-key stages
  uint32_t rows_per_slab, stage_keys, slabs;
  uint64_t workgroups;  // of 128 rows
};

Tile32Geometry tile32_geometry(const DenseAttentionArgs &a) {
  Tile32Geometry g = {false, false, 128, 64, 0, 0};
  const bool aligned = reinterpret_cast<uintptr_t>(a.query) % 16 == 0 && reinterpret_cast<uintptr_t>(a.key) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(a.value) % 8 == 0 && reinterpret_cast<uintptr_t>(a.output) % 8 == 0;
  if (!((a.head_dim == 64 || a.head_dim == 128 || a.head_dim == 256) && aligned &&
        (a.query_length >= 16 || (a.query_length >= 2 && a.key_length >= 256))))
    return g;
  // K and V stages are copied as 16-byte pieces of whole rows (16-byte aligned K and V rows), and the
  // maxima are taken before scaling (a positive, finite scale); anything else takes the row kernel
  const size_t value_row_halfs = a.token_first_value ? (size_t)(a.kv_heads > 0 ? a.kv_heads : a.heads) * a.head_dim
                                                     : a.head_dim;
  const bool staged = reinterpret_cast<uintptr_t>(a.value) % 16 == 0 && value_row_halfs % 8 == 0 &&
                      a.scale > 0.0f && a.scale < INFINITY;
  g.workgroups = (uint64_t)((a.query_length + kWavesPerBlock * 32 - 1) / (kWavesPerBlock * 32)) * a.heads * a.batches;
  if (!staged || g.workgroups > 0x7fffffffull) return g;
  g.tiled = true;
  g.key_split = g.workgroups < (uint64_t)device_compute_units() && a.key_length >= 256 && a.head_dim <= 128;
  if (g.key_split) g.rows_per_slab = 32, g.stage_keys = 128;
  g.slabs = (a.query_length + g.rows_per_slab - 1) / g.rows_per_slab;
  return g;
}

bool dense_masked(const DenseAttentionArgs &a) { return a.mask != nullptr && a.mask_batches > 0; }

// bytes of the stage map per (mask row group, slab): one per stage of keys
uint32_t stage_map_stride(const DenseAttentionArgs &a, const Tile32Geometry &g) {
  return (a.key_length + g.stage_keys - 1) / g.stage_keys;
}

// the map comes first in the scratch memory, rounded up so that the bit words behind it are aligned
size_t stage_map_region(const DenseAttentionArgs &a, const Tile32Geometry &g) {
  return ((size_t)a.mask_batches * a.mask_heads * g.slabs * stage_map_stride(a, g) + 255) & ~(size_t)255;
}

uint32_t mask_words_per_row(const DenseAttentionArgs &a) { return 2 * ((a.key_length + 63) / 64); }

}  // namespace

hipError_t launch_tree_mask(uint8_t *mask, uint32_t query_length, uint32_t key_length, uint32_t past_length,
                            const uint32_t tree_masks[8], hipStream_t stream) {
  const uint64_t elements = (uint64_t)query_length * key_length;
  if (elements == 0) return hipSuccess;
  if ((elements + 255) / 256 > 0x7fffffffull) return hipErrorInvalidValue;
  TreeMaskArgs args = {mask, query_length, key_length, past_length, {}};
  for (int i = 0; i < 8; ++i) args.tree_masks[i] = tree_masks[i];
  hipLaunchKernelGGL(tree_mask_kernel, dim3((uint32_t)((elements + 255) / 256)), dim3(256), 0, stream, args);
  return hipGetLastError();
}

size_t dense_attention_workspace_bytes(const DenseAttentionArgs &a) {
  if (!dense_masked(a) || a.batches == 0 || a.heads == 0 || a.query_length == 0 || a.key_length == 0) return 0;
  const Tile32Geometry g = tile32_geometry(a);
  if (!g.tiled) return 0;
  // a few stages only: walking them all (their arithmetic is skipped where the mask forbids it) costs
  // less than another launch ahead of the attention kernel
  if ((a.key_length + g.stage_keys - 1) / g.stage_keys <= 4) return 0;
  return stage_map_region(a, g) + (size_t)a.mask_batches * a.mask_heads * a.query_length * mask_words_per_row(a) * 4;
}

hipError_t launch_dense_attention(const DenseAttentionArgs &a, hipStream_t stream) {
  const uint64_t rows = (uint64_t)a.batches * a.heads * a.query_length;
  if (rows == 0) return hipSuccess;
  if (a.key_length == 0 || a.head_dim == 0 || a.head_dim > 64 * kMaxFragments) return hipErrorInvalidValue;
  const Tile32Geometry geometry = tile32_geometry(a);
  {
    if (geometry.tiled) {
      const uint64_t workgroups = geometry.workgroups;
      const int mask = dense_masked(a) ? (a.mask_dtype == 2 ? 2 : 1) : 0;
      DenseAttentionArgs scheduled = a;
      scheduled.cus_per_xcd = (uint32_t)device_compute_units() / 8;
      // the pass over the mask: which stages of keys each slab of rows has to walk, and the mask as bits
      int mask_kind = mask;
      if (mask != 0 && a.stage_map != nullptr) {
        const uint32_t stride = stage_map_stride(a, geometry);
        const uint64_t groups = (uint64_t)a.mask_batches * a.mask_heads;
        const size_t map_region = stage_map_region(a, geometry);
        const size_t wanted = map_region + (size_t)groups * a.query_length * mask_words_per_row(a) * 4;
        if (a.stage_map_bytes < wanted || geometry.slabs > 65535 || groups > 65535 ||
            (reinterpret_cast<uintptr_t>(a.stage_map) & 3) != 0) {
          scheduled.stage_map = nullptr;
        } else {
          uint32_t *bits = reinterpret_cast<uint32_t *>(a.stage_map + map_region);
          hipLaunchKernelGGL(mask_bits_kernel, dim3((stride + 1) / 2, geometry.slabs, (uint32_t)groups),
                             dim3(geometry.rows_per_slab * geometry.stage_keys / 32), 0, stream, a, geometry.rows_per_slab,
                             geometry.stage_keys, stride, bits, mask_words_per_row(a));
          scheduled.mask_bits = bits;
          scheduled.mask_words_per_row = mask_words_per_row(a);
          mask_kind = 3;
        }
      }
      if (geometry.key_split) {
        const uint32_t grid = (uint32_t)((a.query_length + 31) / 32) * a.heads * a.batches;
        if (a.head_dim == 64) return launch_tile32<64, 4, 128, true>(mask_kind, grid, scheduled, stream);
        return launch_tile32<128, 4, 128, true>(mask_kind, grid, scheduled, stream);
      }
      // 32 x 32 wave tiles over shared LDS stages, four waves and 64 keys a stage.  (Workgroups of two
      // waves with 32-key stages, twice as many and four per CU, so that short causal launches are not
      // as long as their longest workgroup, measured slower: 105.6 against 91.2 us at 32 heads x 2048
      // tokens - one tile per barrier, half the sharing.)  Heads of 256: 128 KB of stages, one
      // workgroup per CU with all of its registers.
      if (a.head_dim == 256) return launch_tile32<256, 4, 64, false>(mask_kind, (uint32_t)workgroups, scheduled, stream);
      // One or two workgroups per CU: two groups of four waves per slab, each with half of the stages (a
      // CU then holds one workgroup at a time, at the same two waves per SIMD): 32 heads x 2048 tokens,
      // 512 workgroups, 72.9 -> 67.6 us.  The groups meet at every stage's barrier, so two of them get
      // less out of a CU than two workgroups of four waves that run side by side freely - launches with
      // enough of those keep them.
      if (workgroups <= 2 * (uint64_t)device_compute_units() && a.key_length >= 256) {
        if (a.head_dim == 64) return launch_tile32<64, 4, 64, false, true>(mask_kind, (uint32_t)workgroups, scheduled, stream);
        return launch_tile32<128, 4, 64, false, true>(mask_kind, (uint32_t)workgroups, scheduled, stream);
      }
      if (a.head_dim == 64) return launch_tile32<64, 4, 64, false>(mask_kind, (uint32_t)workgroups, scheduled, stream);
      return launch_tile32<128, 4, 64, false>(mask_kind, (uint32_t)workgroups, scheduled, stream);
    }
  }
  const uint64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dense_attention_rows_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace llmopt
