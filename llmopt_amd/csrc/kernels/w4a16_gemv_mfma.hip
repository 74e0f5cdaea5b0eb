// W4A16 decode GEMV for a few activation rows (M <= 8) on gfx950 with the
// contraction on the matrix cores and the activation held in registers.
//
// Work split.  A wave owns one 256-wide K range for the whole kernel; the waves
// of a workgroup cover the K extent (16 waves = 4096) and, when K is short,
// several tiles side by side.  A workgroup walks tiles of 16 weight rows; per
// tile a wave reads its 16 rows x 128 bytes, multiplies them with its own
// activation fragment and leaves an 8 x 16 partial sum in LDS; the workgroup
// adds the partial sums of its K ranges every few tiles.  K extents beyond one
// workgroup are split over blockIdx.y: the slices leave fp32 partial sums in a
// workspace and the last workgroup to arrive at a tile (an atomic counter per
// tile) adds them in slice order.
//
// Matrix operands.  One v_mfma_f32_16x16x32_f16 multiplies a 16(m) x 32(k)
// activation block with a 32(k) x 16(n) weight block.  Lane (c = lane % 16,
// h = lane / 16) supplies the B operand of weight row c: the 8 K values of
// dword j of the 16-byte chunk h of a 64-byte half step.  Chunks 0,1 lie in one
// 64-wide scale group, chunks 2,3 in the next, so the activation is laid out
// block-diagonally: A rows 0..7 are x rows 0..7 for chunks 0,1 and zero for
// chunks 2,3, A rows 8..15 the other way round.  D rows 0..7 / 8..15 are then
// the partial sums of the two scale groups, and the 4 D registers of a lane
// (rows 4h..4h+3, column c) belong to the scale group of the weights that lane
// holds: the fp16 group scale is one scalar per lane, applied in fp32.
//
// Loads.  In operand order a lane quad would touch four weight rows (four
// cache lines) per load.  The weight loads therefore use a row-major lane order
// in which eight lanes read one whole 128-byte line (half lines from two
// instructions measured 1.5 us slower per 31 MB), and the tile passes through a
// wave-private LDS patch to reach the operand lanes: two 16-byte writes and two
// reads (a ds_bpermute per dword measured 1.2 us slower).  The scales are read
// as (row lane / 4, group lane % 4) and moved by ds_bpermute.
// The activation fragment is requested first and then a ring of tiles, so that
// all of a workgroup's weights are in flight from the start and a tile can be
// multiplied as soon as it has arrived (loads return in order).
//
// Decode.  Nibbles become fp16 with a bias (q + 1032 or q + 72, one bit
// operation per pair of nibbles); the bias is removed by starting every MFMA
// chain from -(x . bias pattern), which one extra MFMA chain per wave computes
// once from the resident activation fragment.
//
// Same arithmetic contract as llmopt_w4a16_linear_f16_g64{,_m4,_m8},
// llmopt_w4a16_qkv_linear_f16_g64*, llmopt_w4a16_dual_swiglu_f16_g64* and
// llmopt_w4a16_down_add_f16_g64* (lib/metal_w4a16_source.ml:8-966).
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int TN = 16;         // weight rows per tile
constexpr int kStepK = 256;    // K values per wave
constexpr int kMaxWaves = 16;  // per workgroup
constexpr uint32_t kXRowBytes = 33 * 16;           // 32 pieces of 8 activation values + padding
constexpr uint32_t kXStageBytes = 9 * kXRowBytes;  // per wave: 8 rows and a zero row
constexpr uint32_t kTurnRowBytes = 128 + 16;       // a tile's 128-byte row pieces, padded: conflict-free 16-byte reads down the rows
static_assert(16 * kTurnRowBytes <= kXStageBytes, "the weight turn-around reuses the activation staging area");

struct MfmaMatrix {
  const uint8_t *w;
  const uint16_t *s;
  uint16_t *y;
  uint32_t n;
};

struct MfmaGemvParams {
  const uint16_t *x;
  uint32_t m, k;
  MfmaMatrix mat0, mat1, mat2;  // blockIdx.z selects (DUAL: mat0 = gate, mat1 = up)
  const uint16_t *addend;
  uint32_t has_addend;
  uint32_t addend_stride;
  uint32_t k_slice;    // K values per blockIdx.y slice, a multiple of 256
  uint32_t waves_k;    // waves along K (each 256 wide)
  uint32_t waves_t;    // tiles processed side by side
  float *partials;     // [gridDim.y][8][n] fp32, used when gridDim.y > 1
  uint32_t *counters;  // one per tile, zero between launches
  float *y_f32;        // optional float32 copy of mat0's output, may be null
  uint32_t row_groups;  // > 1: blockIdx.y is a group of 8 activation rows instead of a K slice
  W4Norm norm;          // weight != nullptr: RMS-normalise the activation rows first (one K slice only)
};

// NB = tiles in flight per wave (= tiles between two workgroup reductions)
template <int NB, bool DUAL>
__global__ __launch_bounds__(kMaxWaves * 64) void w4a16_gemv_mfma_kernel(MfmaGemvParams p) {
  constexpr int NW = DUAL ? 2 : 1;
  extern __shared__ float red_lds[];  // partial sums [NB][waves_t][NW][waves_k][8][16] | flags | activation staging

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wk = wave % p.waves_k;  // K range of this wave
  const uint32_t wt = wave / p.waves_k;  // tile lane of this wave
  const MfmaMatrix mat = DUAL ? p.mat0 : (blockIdx.z == 0 ? p.mat0 : blockIdx.z == 1 ? p.mat1 : p.mat2);
  const uint32_t tiles = (mat.n + TN - 1) / TN;
  const uint32_t tile_groups = (tiles + p.waves_t - 1) / p.waves_t;
  if (blockIdx.x >= tile_groups) return;  // a shorter matrix of a QKV launch (whole workgroup)
  const uint32_t rounds = (tile_groups - blockIdx.x + gridDim.x - 1) / gridDim.x;

  // blockIdx.y: K slice (long K, at most 8 rows) or group of 8 activation rows (short K, up to 32 rows)
  const uint32_t row0 = p.row_groups > 1 ? blockIdx.y * 8 : 0;
  const uint32_t rows = min(8u, p.m - row0);
  const uint32_t slice = p.row_groups > 1 ? 0 : blockIdx.y;
  const uint32_t slices = p.row_groups > 1 ? 1 : gridDim.y;
  const uint32_t K = p.k;
  const uint32_t groups_total = K >> 6;
  const uint32_t slice_end = min(K, (slice + 1) * p.k_slice);
  const uint32_t k0 = slice * p.k_slice + wk * kStepK;  // first K value of this wave
  const uint32_t valid_groups = k0 >= slice_end ? 0 : min(4u, (slice_end - k0) >> 6);

  // ---- lane roles -----------------------------------------------------------------
  // operand order: weight row c, chunk h
  const uint32_t c = lane & 15, h = lane >> 4;
  // scale load order: weight row lane / 4, scale group lane % 4 (a quad reads 8 contiguous bytes)
  const uint32_t load_row = lane >> 2, load_chunk = lane & 3;
  // weight load order: eight lanes read one whole 128-byte line (row lane / 8 of the tile's rows
  // 0..7 in the first load, 8..15 in the second; piece lane % 8 of 16 bytes)
  const uint32_t line_row = lane >> 3, line_piece = lane & 7;

  struct Raw {  // loaded-but-untouched registers of one tile
    u32x4_t w[NW][2];
    uint32_t s[NW];
  };
  // Loads that have nothing to fetch (past the last tile, a wave without K range)
  // stay unconditional - a skipped load would make the compiler wait for the
  // whole load queue - and read 16 bytes that are this wave's own, so the idle
  // loads of different waves do not meet on one cache line.
  const size_t idle_row = min(blockIdx.x * p.waves_t * TN, mat.n - 1);
  const size_t idle_w_off = idle_row * (K >> 1) + (min(k0, K - 64) >> 1);
  const size_t idle_s_off = idle_row * groups_total + (min(k0, K - 64) >> 6);
  const uint32_t last_group = valid_groups > 0 ? valid_groups - 1 : 0;
  auto load_tile = [&](uint32_t round, Raw &out) __attribute__((always_inline)) {
    const uint32_t tile = (blockIdx.x + round * gridDim.x) * p.waves_t + wt;
    // bitwise on purpose: short-circuit evaluation would turn the loads into branches
    const bool real = (round < rounds) & (tile < tiles) & (valid_groups > 0);
    const uint32_t row = min(tile * TN + load_row, mat.n - 1);
    // a group past the K range is clamped; its scale is zeroed later
    const uint32_t piece_offset = min(line_piece >> 1, last_group) * 32 + (line_piece & 1) * 16;
    const uint32_t row_w[2] = {(uint32_t)min(tile * TN + line_row, mat.n - 1),
                               (uint32_t)min(tile * TN + 8 + line_row, mat.n - 1)};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const size_t w_off = real ? (size_t)row_w[t] * (K >> 1) + (k0 >> 1) + piece_offset : idle_w_off + t * 16;
      out.w[0][t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(mat.w + w_off));
      if (DUAL)
        out.w[NW - 1][t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p.mat1.w + w_off));
    }
    // scale of (row lane / 4, group lane % 4): a quad reads 8 contiguous bytes
    const size_t s_off = real ? (size_t)row * groups_total + (k0 >> 6) + min(load_chunk, last_group) : idle_s_off;
    out.s[0] = mat.s[s_off];
    if (DUAL) out.s[NW - 1] = p.mat1.s[s_off];
  };

  // ---- activation fragment of this wave's K range, in registers ----------------------
  // A operand of lane (row r = lane % 16, quarter h): x row r % 8 if the row half
  // matches the chunk half, else zero.
  // The 8 rows x 256 values are read row-major (half a wave reads 512 contiguous
  // bytes of one row), rearranged into the decoder's pair order and passed through
  // a wave-private LDS area (rows padded to 33 pieces: conflict-free 16-byte reads
  // down the rows) to reach the operand lanes.  Row 8 of the area is zero: it serves
  // the lanes off the block diagonal.
  h8_t a_frag[2][4];
  const uint32_t slot_floats = NW * p.waves_k * 8 * TN;  // partial sums of one tile
  uint32_t *flag_lds = reinterpret_cast<uint32_t *>(red_lds + NB * p.waves_t * slot_floats);
  uint8_t *x_stage = reinterpret_cast<uint8_t *>(flag_lds + ((NB * p.waves_t + 3) & ~3u)) + wave * kXStageBytes;
  uint4 x_loaded[4];  // requested before the weights: loads return in order
  const uint32_t x_piece = lane & 31;
  const bool normalise = p.norm.weight != nullptr;  // the same for every workgroup
  uint4 gain_loaded = make_uint4(0, 0, 0, 0);
  {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t row = 2 * i + (lane >> 5);
      const uint32_t kk = k0 + x_piece * 8;
      x_loaded[i] =
          *reinterpret_cast<const uint4 *>(p.x + (size_t)(row0 + min(row, rows - 1)) * K + min(kk, K - 8));
    }
    if (normalise) gain_loaded = *reinterpret_cast<const uint4 *>(p.norm.weight + min(k0 + x_piece * 8, K - 8));
  }
  // all tiles of the ring go out next
  Raw ring[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) load_tile(b, ring[b]);
  if (normalise) {
    // RMS normalisation of the rows: a wave holds 256 of a row's K values, so the mean squares of
    // the workgroup's waves with the same tiles meet in LDS; then the half values the separate
    // kernel would have stored (float32 products in its order) replace the raw ones.
    float *norm_lds = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(flag_lds + ((NB * p.waves_t + 3) & ~3u)) +
                                                p.waves_k * p.waves_t * kXStageBytes);
    float square[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool keep = k0 + x_piece * 8 < slice_end;
      const h8_t x = __builtin_bit_cast(h8_t, x_loaded[i]);
      float sum = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += (float)x[e] * (float)x[e];
      sum = keep ? sum : 0.0f;
#pragma unroll
      for (int step = 1; step < 32; step *= 2)  // the 32 lanes of one row
        sum += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)((lane ^ step) << 2),
                                                                       __builtin_bit_cast(int, sum)));
      square[i] = sum;
    }
    if (x_piece == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) norm_lds[(wt * p.waves_k + wk) * 8 + 2 * i + (lane >> 5)] = square[i];
    }
    __syncthreads();
    const h8_t gain = __builtin_bit_cast(h8_t, gain_loaded);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float total = 0.0f;
      for (uint32_t w = 0; w < p.waves_k; ++w) total += norm_lds[(wt * p.waves_k + w) * 8 + 2 * i + (lane >> 5)];
      const float inverse = rsqrtf(total / (float)K + p.norm.epsilon);
      const h8_t x = __builtin_bit_cast(h8_t, x_loaded[i]);
      h8_t y;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float value = (float)x[e], g = (float)gain[e];
        y[e] = (_Float16)(p.norm.weight_first ? value * g * inverse : value * inverse * g);
      }
      x_loaded[i] = __builtin_bit_cast(uint4, y);
    }
  }
  {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t row = 2 * i + (lane >> 5);
      const bool keep = (row < rows) & (k0 + x_piece * 8 < slice_end);
      const uint4 ordered = pair_order(x_loaded[i]);
      uint4 value;
      value.x = keep ? ordered.x : 0u;
      value.y = keep ? ordered.y : 0u;
      value.z = keep ? ordered.z : 0u;
      value.w = keep ? ordered.w : 0u;
      *reinterpret_cast<uint4 *>(x_stage + row * kXRowBytes + x_piece * 16) = value;
    }
    if (lane < 33) *reinterpret_cast<uint4 *>(x_stage + 8 * kXRowBytes + lane * 16) = make_uint4(0, 0, 0, 0);
    __builtin_amdgcn_wave_barrier();  // the LDS unit serves one wave's accesses in order
    const bool on_diagonal = (c >= 8) == (h >= 2);
    const uint8_t *mine = x_stage + (on_diagonal ? (c & 7) : 8) * kXRowBytes + (on_diagonal ? h * 64 : 0);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        a_frag[t][j] = __builtin_bit_cast(h8_t, *reinterpret_cast<const uint4 *>(mine + (t * 16 + j) * 16));
  }
  // -(x . decode bias) per half step: pairs (k0,k4) and (k2,k6) carry 1032, (k1,k5) and (k3,k7) carry 72
  f4_t start[2];
  {
    const h8_t bias = {(_Float16)1032.0f, (_Float16)1032.0f, (_Float16)72.0f, (_Float16)72.0f,
                       (_Float16)1032.0f, (_Float16)1032.0f, (_Float16)72.0f, (_Float16)72.0f};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      f4_t sum = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 4; ++j) sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_frag[t][j], bias, sum, 0, 0, 0);
      start[t] = -sum;
    }
  }

  // Multiplies one tile by the fragment and leaves the wave's partial sums in reduction slot `slot`.
  auto consume = [&](const Raw &raw, uint32_t slot) __attribute__((always_inline)) {
    float *out = red_lds + (slot * p.waves_t + wt) * slot_floats;
    uint8_t *turn = x_stage;
#pragma unroll
    for (int v = 0; v < NW; ++v) {
      f4_t acc = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
      // load order -> operand order through the wave's own LDS patch (the activation staging
      // area, free by now; the LDS unit serves one wave's accesses in order): two 16-byte writes
      // and two reads per tile instead of a ds_bpermute per dword
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 2; ++t)
        *reinterpret_cast<u32x4_t *>(turn + (8 * t + line_row) * kTurnRowBytes + line_piece * 16) = raw.w[v][t];
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const u32x4_t words = *reinterpret_cast<const u32x4_t *>(turn + c * kTurnRowBytes + (4 * t + h) * 16);
        const uint32_t group = 2 * t + (h >> 1);
        const uint32_t scale_bits =
            (uint32_t)__builtin_amdgcn_ds_bpermute((int)((4 * c + group) * 4), (int)raw.s[v]);
        f4_t tile = start[t];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const W4Pairs w = w4_decode_biased(words[j]);
          uint4 packed;
          packed.x = as_u32(w.p04);
          packed.y = as_u32(w.p15);
          packed.z = as_u32(w.p26);
          packed.w = as_u32(w.p37);
          tile = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_frag[t][j], __builtin_bit_cast(h8_t, packed), tile, 0, 0, 0);
        }
        const float scale = group < valid_groups ? half_bits_to_float((uint16_t)scale_bits) : 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(tile[i], scale, acc[i]);
      }
      // the two scale groups of a column sit 32 lanes apart
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float total = acc[i] + __shfl_xor(acc[i], 32);
        if (h < 2) out[((v * p.waves_k + wk) * 8 + h * 4 + i) * TN + c] = total;
      }
    }
  };

  // Adds the K ranges of the tiles parked in slots [0, count) and stores them.
  auto flush = [&](uint32_t first_round, uint32_t count) __attribute__((always_inline)) {
    __syncthreads();
    const uint32_t outputs = count * p.waves_t * 8 * TN;
    const bool split = !DUAL && slices > 1;
    for (uint32_t base = 0; base < outputs; base += blockDim.x) {  // uniform trip count
      const uint32_t o = base + threadIdx.x;
      const bool in_range = o < outputs;
      const uint32_t slot_tile = o >> 7;  // slot * waves_t + tile lane
      const uint32_t slot = slot_tile / p.waves_t, lane_t = slot_tile - slot * p.waves_t;
      const uint32_t m = (o >> 4) & 7, col_in_tile = o & 15;
      const uint32_t tile = (blockIdx.x + (first_round + slot) * gridDim.x) * p.waves_t + lane_t;
      const uint32_t col = tile * TN + col_in_tile;
      const bool writer = in_range && tile < tiles && m < rows && col < mat.n;
      // the addend is requested here, by every thread at a clamped address, and used at the store:
      // under the writer's test it would be a trip to memory of its own after the sums are ready
      uint16_t addend_bits = 0;
      if (!DUAL && p.has_addend)
        addend_bits = p.addend[(size_t)(row0 + min(m, rows - 1)) * p.addend_stride + min(col, mat.n - 1)];
      float total[NW];
#pragma unroll
      for (int v = 0; v < NW; ++v) total[v] = 0.0f;
      if (in_range) {
        const float *in = red_lds + slot_tile * slot_floats;
        // four independent sums so that the LDS reads are issued back to back
#pragma unroll
        for (int v = 0; v < NW; ++v) {
          const float *column = in + (v * p.waves_k * 8 + m) * TN + col_in_tile;
          float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
          uint32_t w = 0;
          for (; w + 4 <= p.waves_k; w += 4) {
#pragma unroll
            for (int u = 0; u < 4; ++u) part[u] += column[(w + u) * 8 * TN];
          }
          for (; w < p.waves_k; ++w) part[0] += column[w * 8 * TN];
          total[v] = (part[0] + part[1]) + (part[2] + part[3]);
        }
      }
      bool store = writer;
      if (split) {
        // K split over workgroups: leave the partial sum where every CU sees it
        // (device-scope stores and loads, no cache write-back needed); the last
        // workgroup to arrive at a tile adds the slices in order.
        if (writer)
          __hip_atomic_store(p.partials + ((size_t)slice * 8 + m) * mat.n + col, total[0], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();  // waits for the stores of every wave
        if (in_range && (o & 127) == 0 && tile < tiles) {
          const uint32_t arrived =
              __hip_atomic_fetch_add(p.counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const bool last = arrived == slices - 1;
          if (last) __hip_atomic_store(p.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          flag_lds[slot_tile] = last ? 1u : 0u;
        }
        __syncthreads();
        store = writer && flag_lds[slot_tile] != 0;
        if (store) {
          // four requests at a time (one after the other they cost a trip to L2 each), summed in slice order
          float sum = 0.0f;
          for (uint32_t other = 0; other < slices; other += 4) {
            float part[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
              part[u] = __hip_atomic_load(p.partials + ((size_t)min(other + u, slices - 1) * 8 + m) * mat.n + col,
                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int u = 0; u < 4; ++u) sum += other + u < slices ? part[u] : 0.0f;
          }
          total[0] = sum;
        }
        __syncthreads();  // the flags are free again
      }
      if (store) {
        float value;
        if (DUAL) {
          value = total[0] / (1.0f + __expf(-total[0])) * total[NW - 1];
        } else {
          value = total[0];
          if (p.has_addend) value += half_bits_to_float(addend_bits);
        }
        if (mat.y != nullptr) mat.y[(size_t)(row0 + m) * mat.n + col] = float_to_half_bits(value);
        if (!DUAL && p.y_f32 != nullptr) p.y_f32[(size_t)(row0 + m) * mat.n + col] = value;
      }
    }
    __syncthreads();  // the slots are free again
  };

  // ---- tiles: NB per pass, each buffer refilled as soon as it has been consumed ------
  for (uint32_t first = 0; first < rounds; first += NB) {
    const bool refill = first + NB < rounds;  // nothing is loaded after the last pass
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      consume(ring[b], b);
      if (refill) load_tile(first + NB + b, ring[b]);
    }
    flush(first, min((uint32_t)NB, rounds - first));
  }
}

struct Plan {
  uint32_t slices, k_slice, waves_k, waves_t, blocks, ring;
  size_t lds_bytes;
};

Plan make_plan(uint32_t k, uint32_t max_n, uint32_t matrices, bool dual) {
  Plan plan;
  const uint32_t steps_total = (k + kStepK - 1) / kStepK;
  plan.slices = (steps_total + kMaxWaves - 1) / kMaxWaves;
  plan.waves_k = (steps_total + plan.slices - 1) / plan.slices;
  plan.k_slice = plan.waves_k * kStepK;
  plan.slices = (k + plan.k_slice - 1) / plan.k_slice;
  const uint32_t tiles = (max_n + TN - 1) / TN;
  const uint32_t cus = (uint32_t)device_compute_units();
  // short K: several tiles side by side in one workgroup, once there are more tiles than CUs
  const uint32_t room = std::max<uint32_t>(1, kMaxWaves / plan.waves_k);
  plan.waves_t = std::max<uint32_t>(1, std::min<uint32_t>(room, tiles * plan.slices * matrices / cus));
  const uint32_t tile_groups = (tiles + plan.waves_t - 1) / plan.waves_t;
  const uint32_t waves = plan.waves_k * plan.waves_t;
  const uint32_t per_cu = waves <= 4 ? 4 : waves <= 8 ? 2 : 1;
  const uint32_t resident = std::max<uint32_t>(1, cus * per_cu / (plan.slices * matrices));
  // the same number of tiles for every workgroup: 896 tiles on 256 CUs run as 224 workgroups of
  // four rather than 256 of three or four (10.1 against 10.6 us at 4096 x 14336)
  const uint32_t passes = (tile_groups + resident - 1) / resident;
  plan.blocks = (tile_groups + passes - 1) / passes;
  // tiles in flight per wave: all of a workgroup's tiles when they are few
  const uint32_t rounds = (tile_groups + plan.blocks - 1) / plan.blocks;
  plan.ring = rounds <= 1 ? 1 : (rounds <= 2 || dual) ? 2 : 4;
  const int nw = dual ? 2 : 1;
  plan.lds_bytes = (size_t)plan.ring * plan.waves_t * nw * plan.waves_k * 8 * TN * sizeof(float) +
                   (size_t)((plan.ring * plan.waves_t + 3) & ~3u) * sizeof(uint32_t) + (size_t)waves * kXStageBytes +
                   (size_t)waves * 8 * sizeof(float);  // the last: mean squares of a normalising launch
  return plan;
}

template <int NB, bool DUAL>
hipError_t launch_ring(const MfmaGemvParams &p, uint32_t matrices, const Plan &plan, hipStream_t stream) {
  static bool configured[kMaxDevices] = {};  // the attribute is per device function and device
  if (hipError_t status = allow_dynamic_lds(reinterpret_cast<const void *>(&w4a16_gemv_mfma_kernel<NB, DUAL>), 160 * 1024,
                                            configured))
    return status;
  const dim3 grid(plan.blocks, p.row_groups > 1 ? p.row_groups : plan.slices, matrices);
  hipLaunchKernelGGL((w4a16_gemv_mfma_kernel<NB, DUAL>), grid, dim3(plan.waves_k * plan.waves_t * 64),
                     plan.lds_bytes, stream, p);
  return hipGetLastError();
}

template <bool DUAL>
hipError_t launch(MfmaGemvParams p, uint32_t matrices, const Plan &plan, hipStream_t stream) {
  p.k_slice = plan.k_slice;
  p.waves_k = plan.waves_k;
  p.waves_t = plan.waves_t;
  if (plan.lds_bytes > 160 * 1024) return hipErrorInvalidValue;
  if (plan.ring == 1) return launch_ring<1, DUAL>(p, matrices, plan, stream);
  if (plan.ring == 2) return launch_ring<2, DUAL>(p, matrices, plan, stream);
  if constexpr (DUAL) return hipErrorInvalidValue;
  else return launch_ring<4, false>(p, matrices, plan, stream);
}

}  // namespace

size_t w4a16_gemv_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
  (void)m;
  const uint32_t steps_total = (k + kStepK - 1) / kStepK;
  const uint32_t slices = (steps_total + kMaxWaves - 1) / kMaxWaves;
  return slices > 1 ? (size_t)slices * 8 * n * sizeof(float) : 0;
}

bool w4a16_gemv_mfma_needs_split(uint32_t k) { return (k + kStepK - 1) / kStepK > (uint32_t)kMaxWaves; }

bool w4a16_gemv_mfma_row_groups_ok(uint32_t m, uint64_t columns, uint32_t k) {
  return m > kGemvMaxRows && m <= 128 && !w4a16_gemv_mfma_needs_split(k) && columns * k / 2 <= (4u << 20);
}

hipError_t launch_w4a16_gemv_mfma_linear(const W4LinearArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.w.weight, a.w.scale, a.y, a.n};
  p.mat1 = p.mat0;
  p.mat2 = p.mat0;
  p.addend = a.addend;
  p.has_addend = a.has_addend;
  p.addend_stride = a.addend_row_stride;
  p.row_groups = (a.m + 7) / 8;
  const Plan plan = make_plan(a.k, a.n, p.row_groups, false);
  if (plan.slices > 1) {
    if (p.row_groups > 1) return hipErrorInvalidValue;  // callers check w4a16_gemv_mfma_row_groups_ok
    const uint32_t tiles = (a.n + TN - 1) / TN;
    if (a.workspace == nullptr || a.counters == nullptr || tiles > a.counter_count ||
        a.workspace_bytes < w4a16_gemv_workspace_bytes(a.m, a.n, a.k))
      return hipErrorInvalidValue;
  }
  p.partials = static_cast<float *>(a.workspace);
  p.counters = a.counters;
  p.y_f32 = a.y_f32;
  return launch<false>(p, 1, plan, stream);
}

hipError_t launch_w4a16_gemv_mfma_qkv(const W4QkvArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.w[0].weight, a.w[0].scale, a.y[0], a.n[0]};
  p.mat1 = {a.w[1].weight, a.w[1].scale, a.y[1], a.n[1]};
  p.mat2 = {a.w[2].weight, a.w[2].scale, a.y[2], a.n[2]};
  p.row_groups = (a.m + 7) / 8;
  p.norm = a.norm;
  const Plan plan = make_plan(a.k, std::max(a.n[0], std::max(a.n[1], a.n[2])), 3 * p.row_groups, false);
  if (plan.slices > 1) return hipErrorInvalidValue;  // callers check w4a16_gemv_mfma_needs_split
  return launch<false>(p, 3, plan, stream);
}

hipError_t launch_w4a16_gemv_mfma_dual_swiglu(const W4DualSwigluArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.gate.weight, a.gate.scale, a.product, a.n};
  p.mat1 = {a.up.weight, a.up.scale, a.product, a.n};
  p.mat2 = p.mat0;
  p.row_groups = (a.m + 7) / 8;
  p.norm = a.norm;
  const Plan plan = make_plan(a.k, a.n, p.row_groups, true);
  if (plan.slices > 1) return hipErrorInvalidValue;
  return launch<true>(p, 1, plan, stream);
}

}  // namespace llmopt
