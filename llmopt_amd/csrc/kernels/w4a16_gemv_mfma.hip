// W4A16 decode GEMV for 1 <= M <= 8 activation rows on gfx950 with the
// contraction on the matrix cores.
//
// One v_mfma_f32_16x16x32_f16 multiplies a 16(m) x 32(k) activation block with
// a 32(k) x 16(n) weight block.  Lane (c = lane % 16, h = lane / 16) supplies
// the B operand of weight row c: the 8 K values of dword j of the 16 bytes it
// loaded at byte offset 16 h of a 128-wide K block.  Lanes h = 0,1 therefore
// hold the first 64-wide scale group of the block and lanes h = 2,3 the second.
// The activation is laid out block-diagonally: A rows 0..7 are x rows 0..7 for
// K quarters 0,1 and zero for quarters 2,3, A rows 8..15 the other way round.
// D rows 0..7 then hold the partial sums of the first scale group and rows
// 8..15 those of the second, and the D registers of a lane (rows 4 h .. 4 h + 3,
// column c) belong to exactly the scale group of the weights that lane loaded:
// the fp16 group scale is one scalar per lane, applied in fp32 to the 4
// accumulators.
//
// The nibbles are decoded to fp16 with a bias (q + 1032 or q + 72, one bit
// operation per pair of nibbles).  The bias is removed by starting the MFMA
// accumulation of a scale group from -(1032 sum x_even_pairs + 72 sum
// x_odd_pairs), computed once per workgroup while the activation is staged to
// LDS in the operand order of the decode.
//
// A workgroup of 8 waves streams tiles of 16 weight rows; its waves split the
// K range of the tile in steps of 256 and are reduced through LDS.  When M x K
// does not fit the LDS budget the K range is split over blockIdx.y as well:
// the slices leave fp32 partial sums in a workspace and the last workgroup to
// arrive at a tile (an atomic counter per tile) adds them in slice order.
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

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int TN = 16;        // weight rows per tile
constexpr int kStepK = 256;   // K values one wave consumes per step
constexpr int kZeroVectors = 20;  // per activation row: covers every operand offset of a step
template <bool DUAL>
constexpr int kReduceSlots = DUAL ? 1 : 2;  // DUAL keeps two sets of partial sums per tile

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
  float *partials;     // [gridDim.y][8][n] fp32, used when gridDim.y > 1
  uint32_t *counters;  // one per tile, zero between launches
  float *y_f32;        // optional float32 copy of mat0's output, may be null
};

// MP = activation rows held in LDS (1, 2, 4 or 8, >= m)
template <int MP, bool DUAL>
__global__ __launch_bounds__(kThreads) void w4a16_gemv_mfma_kernel(MfmaGemvParams p) {
  constexpr int NW = DUAL ? 2 : 1;
  constexpr int SPI = DUAL ? 1 : 2;      // steps per work item: 64 bytes per lane in flight per item
  constexpr int RS = kReduceSlots<DUAL>;  // tiles finished between two workgroup reductions
  extern __shared__ uint4 lds[];

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t c = lane & 15;  // weight row of the tile (B column, D column)
  const uint32_t h = lane >> 4;  // K quarter of the B operand; D rows 4h..4h+3
  const MfmaMatrix mat = DUAL ? p.mat0 : (blockIdx.z == 0 ? p.mat0 : blockIdx.z == 1 ? p.mat1 : p.mat2);
  const uint32_t tiles = (mat.n + TN - 1) / TN;
  if (blockIdx.x >= tiles) return;  // a shorter matrix of a QKV launch (whole workgroup)

  const uint32_t K = p.k;
  const uint32_t groups_total = K >> 6;
  const uint32_t k_begin = blockIdx.y * p.k_slice;
  const uint32_t k_len = min(p.k_slice, K - k_begin);
  const uint32_t groups = k_len >> 6;  // scale groups of this slice
  const uint32_t steps = (k_len + kStepK - 1) / kStepK;
  const uint32_t items_per_tile = (steps + kWaves * SPI - 1) / (kWaves * SPI);  // per wave

  // LDS: zero vectors | x in operand order | -bias correction | wave partial sums | flags
  const uint32_t x_vectors = steps * 32 * MP;
  uint4 *x_lds = lds + kZeroVectors * MP;
  float *corr_lds = reinterpret_cast<float *>(x_lds + x_vectors);  // [steps*4][8]
  float *red_lds = corr_lds + steps * 4 * 8;                       // [RS][NW][waves][8][16]
  uint32_t *flag_lds = reinterpret_cast<uint32_t *>(red_lds + RS * NW * kWaves * 8 * TN);  // [RS]

  struct Item {  // raw loaded registers only: conversions at the load would serialise the prefetch
    u32x4_t w[NW][SPI][2];
    uint16_t s[NW][SPI][2];
  };
  // item `index` of a tile covers steps (wave + index*kWaves)*SPI .. +SPI-1
  // `real` = false is the prefetch past the last item: it stays unconditional
  // (a skipped load would make the compiler wait for the whole load queue) but
  // every lane reads the first 16 bytes of the matrix, one cache line per wave.
  auto load_item = [&](uint32_t tile, uint32_t index, bool real, Item &out) __attribute__((always_inline)) {
    const uint32_t row = min(tile * TN + c, mat.n - 1);
    const uint32_t step0 = (wave + index * kWaves) * SPI;
#pragma unroll
    for (int u = 0; u < SPI; ++u) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // clamped past the end of the slice (the scale is zeroed when consumed)
        const uint32_t g = min((step0 + u) * 4 + 2 * t + (h >> 1), groups - 1);
        const size_t w_off = real ? (size_t)row * (K >> 1) + (k_begin >> 1) + g * 32 + (h & 1) * 16 : 0;
        const size_t s_off = real ? (size_t)row * groups_total + (k_begin >> 6) + g : 0;
        out.w[0][u][t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(mat.w + w_off));
        out.s[0][u][t] = mat.s[s_off];
        if (DUAL) {
          out.w[NW - 1][u][t] =
              __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p.mat1.w + w_off));
          out.s[NW - 1][u][t] = p.mat1.s[s_off];
        }
      }
    }
  };

  // first loads go out before the activation is staged
  Item item_a, item_b;
  load_item(blockIdx.x, 0, true, item_a);

  // ---- stage x[:, k_begin .. k_begin + steps*256) and the bias correction ----
  for (uint32_t i = threadIdx.x; i < kZeroVectors * MP; i += kThreads) lds[i] = make_uint4(0, 0, 0, 0);
  {
    constexpr int UNROLL = 4;  // independent loads in flight per thread
    const uint32_t padded = (x_vectors + 63) & ~63u;
    for (uint32_t base = threadIdx.x; base < padded; base += kThreads * UNROLL) {
      uint4 value[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t i = base + u * kThreads;
        const uint32_t m = i & (MP - 1);
        const uint32_t kb = i / MP;  // block of 8 K values within the slice
        value[u] = make_uint4(0, 0, 0, 0);
        if (m < p.m && kb * 8 < k_len)
          value[u] = *reinterpret_cast<const uint4 *>(p.x + (size_t)m * K + k_begin + kb * 8);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t i = base + u * kThreads;
        if (i >= padded) break;  // uniform per wave: padded is a multiple of 64
        const uint32_t m = i & (MP - 1);
        const uint32_t kb = i / MP;
        const uint4 ordered = pair_order(value[u]);
        if (i < x_vectors) x_lds[i] = ordered;
        // pairs .x and .z meet weights decoded as q + 1032, pairs .y and .w as q + 72
        const h2_t a = as_h2(ordered.x), b = as_h2(ordered.y), cc = as_h2(ordered.z), d = as_h2(ordered.w);
        float bias = 1032.0f * (((float)a[0] + (float)a[1]) + ((float)cc[0] + (float)cc[1])) +
                     72.0f * (((float)b[0] + (float)b[1]) + ((float)d[0] + (float)d[1]));
        // the 8 blocks of a scale group sit MP lanes apart
        bias += __shfl_xor(bias, MP);
        bias += __shfl_xor(bias, 2 * MP);
        bias += __shfl_xor(bias, 4 * MP);
        if ((kb & 7) == 0 && i < x_vectors) corr_lds[(kb >> 3) * 8 + m] = -bias;
      }
    }
    if (MP < 8) {
      // rows MP..7 of the correction are read (their D rows are never used): keep them finite
      for (uint32_t i = threadIdx.x; i < steps * 4 * 8; i += kThreads)
        if ((i & 7) >= MP) corr_lds[i] = 0.0f;
    }
  }
  __syncthreads();

  // operand addressing: lanes off the block diagonal read the zero vectors
  const bool on_diagonal = (c >= 8) == (h >= 2);
  const uint32_t m_of_lane = (c & 7) & (MP - 1);
  const uint32_t a_base = on_diagonal ? (kZeroVectors + h * 4) * MP + m_of_lane : 0;  // in vectors
  const uint32_t a_step = on_diagonal ? 32 * MP : 0;
  const uint32_t corr_base = (h >> 1) * 8 + (h & 1) * 4;

  f4_t acc[NW];
#pragma unroll
  for (int v = 0; v < NW; ++v) acc[v] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};

  auto consume = [&](uint32_t index, const Item &cur) __attribute__((always_inline)) {
    const uint32_t step0 = (wave + index * kWaves) * SPI;
#pragma unroll
    for (int u = 0; u < SPI; ++u) {
      const uint32_t step = step0 + u;
      const uint32_t step_l = min(step, steps - 1);
      const uint4 *a_ptr = lds + a_base + a_step * step_l;
      const float *corr_ptr = corr_lds + corr_base + step_l * 32;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const bool ok = step * 4 + 2 * t + (h >> 1) < groups;
        const f4_t start = *reinterpret_cast<const f4_t *>(corr_ptr + t * 16);
        h8_t a_frag[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) a_frag[j] = __builtin_bit_cast(h8_t, a_ptr[(t * 16 + j) * MP]);
#pragma unroll
        for (int v = 0; v < NW; ++v) {
          f4_t tile = start;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const W4Pairs w = w4_decode_biased(cur.w[v][u][t][j]);
            uint4 packed;
            packed.x = as_u32(w.p04);
            packed.y = as_u32(w.p15);
            packed.z = as_u32(w.p26);
            packed.w = as_u32(w.p37);
            tile = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_frag[j], __builtin_bit_cast(h8_t, packed), tile, 0,
                                                          0, 0);
          }
          const float scale = ok ? half_bits_to_float(cur.s[v][u][t]) : 0.0f;
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[v][i] = fmaf(tile[i], scale, acc[v][i]);
        }
      }
    }
  };

  // A finished tile leaves the wave's partial sums in a reduction slot; the
  // workgroup reduces RS tiles at a time.
  uint32_t pending = 0;        // tiles waiting in the slots (uniform)
  uint32_t pending_first = 0;  // tile index of slot 0; slot s holds pending_first + s*gridDim.x
  auto park_tile = [&](uint32_t tile) __attribute__((always_inline)) {
    if (pending == 0) pending_first = tile;
    float *slot = red_lds + pending * (NW * kWaves * 8 * TN);
    // the two scale-group halves of a column sit 32 lanes apart
#pragma unroll
    for (int v = 0; v < NW; ++v) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float total = acc[v][i] + __shfl_xor(acc[v][i], 32);
        if (h < 2) slot[((v * kWaves + wave) * 8 + h * 4 + i) * TN + c] = total;
        acc[v][i] = 0.0f;
      }
    }
    ++pending;
  };
  auto flush = [&]() __attribute__((always_inline)) {
    __syncthreads();
    const uint32_t slot_index = threadIdx.x >> 7;  // 128 outputs per tile
    const uint32_t in_slot = threadIdx.x & 127;
    const uint32_t m = in_slot >> 4, col_in_tile = in_slot & 15;
    const uint32_t tile = pending_first + slot_index * gridDim.x;
    const uint32_t col = tile * TN + col_in_tile;
    const bool active = slot_index < pending;
    const bool writer = active && m < p.m && col < mat.n;
    float total[NW];
    if (active) {
      const float *slot = red_lds + slot_index * (NW * kWaves * 8 * TN);
#pragma unroll
      for (int v = 0; v < NW; ++v) {
        total[v] = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total[v] += slot[((v * kWaves + w) * 8 + m) * TN + col_in_tile];
      }
    }
    bool store = writer;
    if (!DUAL && gridDim.y > 1) {
      // K split over workgroups: leave the partial sum where every CU sees it
      // (device-scope stores and loads, no cache write-back needed); the last
      // workgroup to arrive at a tile adds the slices in order.
      if (writer)
        __hip_atomic_store(p.partials + ((size_t)blockIdx.y * 8 + m) * mat.n + col, total[0], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();  // waits for the stores of every wave
      if (active && in_slot == 0) {
        const uint32_t arrived =
            __hip_atomic_fetch_add(p.counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = arrived == gridDim.y - 1;
        if (last) __hip_atomic_store(p.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        flag_lds[slot_index] = last ? 1u : 0u;
      }
      __syncthreads();
      store = writer && flag_lds[slot_index] != 0;
      if (store) {
        float sum = 0.0f;
        for (uint32_t slice = 0; slice < gridDim.y; ++slice)
          sum += __hip_atomic_load(p.partials + ((size_t)slice * 8 + m) * mat.n + col, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        total[0] = sum;
      }
    }
    if (store) {
      float value;
      if (DUAL) {
        value = total[0] / (1.0f + __expf(-total[0])) * total[NW - 1];
      } else {
        value = total[0];
        if (p.has_addend) value += half_bits_to_float(p.addend[(size_t)m * p.addend_stride + col]);
      }
      if (mat.y != nullptr) mat.y[(size_t)m * mat.n + col] = float_to_half_bits(value);
      if (!DUAL && p.y_f32 != nullptr) p.y_f32[(size_t)m * mat.n + col] = value;
    }
    __syncthreads();  // the slots are free again
    pending = 0;
  };

  // Items of this wave: for each tile of the workgroup, items 0 .. items_per_tile-1.
  // Ping-pong between two register sets with an unconditional prefetch.
  auto advance = [&](uint32_t &tile, uint32_t &index) {
    if (++index == items_per_tile) {
      index = 0;
      tile += gridDim.x;
    }
  };
  uint32_t tile = blockIdx.x, index = 0;
  while (true) {
    uint32_t next_tile = tile, next_index = index;
    advance(next_tile, next_index);
    bool more = next_tile < tiles;
    load_item(next_tile, next_index, more, item_b);
    consume(index, item_a);
    if (index == items_per_tile - 1) {
      park_tile(tile);
      if (pending == RS || !more) flush();
    }
    if (!more) break;
    tile = next_tile;
    index = next_index;
    advance(next_tile, next_index);
    more = next_tile < tiles;
    load_item(next_tile, next_index, more, item_a);
    consume(index, item_b);
    if (index == items_per_tile - 1) {
      park_tile(tile);
      if (pending == RS || !more) flush();
    }
    if (!more) break;
    tile = next_tile;
    index = next_index;
  }
}

constexpr size_t kLdsBudget = 79 * 1024;  // two workgroups per CU (160 KB)

size_t lds_bytes_for(uint32_t mp, uint32_t steps, int nw) {
  const int slots = nw == 2 ? kReduceSlots<true> : kReduceSlots<false>;
  return (size_t)(kZeroVectors * mp + steps * 32 * mp) * 16 + (size_t)steps * 4 * 8 * 4 +
         (size_t)slots * nw * kWaves * 8 * TN * 4 + 16;
}

struct Plan {
  uint32_t mp, slices, k_slice;
  size_t lds_bytes;
};

Plan make_plan(uint32_t m, uint32_t k, int nw, bool may_split) {
  Plan plan;
  plan.mp = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
  const uint32_t steps_total = (k + kStepK - 1) / kStepK;
  plan.slices = 1;
  if (may_split) {
    while (plan.slices < steps_total &&
           lds_bytes_for(plan.mp, (steps_total + plan.slices - 1) / plan.slices, nw) > kLdsBudget)
      ++plan.slices;
  }
  const uint32_t steps = (steps_total + plan.slices - 1) / plan.slices;
  plan.k_slice = steps * kStepK;
  plan.slices = (k + plan.k_slice - 1) / plan.k_slice;
  plan.lds_bytes = lds_bytes_for(plan.mp, steps, nw);
  return plan;
}

template <int MP, bool DUAL>
hipError_t launch_instance(const MfmaGemvParams &p, dim3 grid, size_t lds_bytes, hipStream_t stream) {
  static bool configured = false;  // per instantiation; the attribute is per device function
  if (!configured) {
    hipError_t status = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&w4a16_gemv_mfma_kernel<MP, DUAL>),
        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (status != hipSuccess) return status;
    configured = true;
  }
  hipLaunchKernelGGL((w4a16_gemv_mfma_kernel<MP, DUAL>), grid, dim3(kThreads), lds_bytes, stream, p);
  return hipGetLastError();
}

template <bool DUAL>
hipError_t launch(MfmaGemvParams p, uint32_t matrices, uint32_t max_n, const Plan &plan, hipStream_t stream) {
  p.k_slice = plan.k_slice;
  const uint32_t tiles = (max_n + TN - 1) / TN;
  const uint32_t per_cu = plan.lds_bytes <= kLdsBudget ? 2 : 1;
  const uint32_t resident = (uint32_t)device_compute_units() * per_cu;
  const uint32_t blocks = std::max<uint32_t>(1, std::min<uint32_t>(tiles, resident / (plan.slices * matrices)));
  const dim3 grid(blocks, plan.slices, matrices);
  switch (plan.mp) {
    case 1: return launch_instance<1, DUAL>(p, grid, plan.lds_bytes, stream);
    case 2: return launch_instance<2, DUAL>(p, grid, plan.lds_bytes, stream);
    case 4: return launch_instance<4, DUAL>(p, grid, plan.lds_bytes, stream);
    default: return launch_instance<8, DUAL>(p, grid, plan.lds_bytes, stream);
  }
}

}  // namespace

size_t w4a16_gemv_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
  const Plan plan = make_plan(m, k, 1, true);
  return plan.slices > 1 ? (size_t)plan.slices * 8 * n * sizeof(float) : 0;
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
  const uint32_t tiles = (a.n + TN - 1) / TN;
  const bool may_split = a.workspace != nullptr && a.counters != nullptr && tiles <= a.counter_count &&
                         a.workspace_bytes >= w4a16_gemv_workspace_bytes(a.m, a.n, a.k);
  const Plan plan = make_plan(a.m, a.k, 1, may_split);
  if (plan.lds_bytes > 160 * 1024) return hipErrorInvalidValue;
  p.partials = static_cast<float *>(a.workspace);
  p.counters = a.counters;
  p.y_f32 = a.y_f32;
  return launch<false>(p, 1, a.n, plan, stream);
}

hipError_t launch_w4a16_gemv_mfma_qkv(const W4QkvArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.w[0].weight, a.w[0].scale, a.y[0], a.n[0]};
  p.mat1 = {a.w[1].weight, a.w[1].scale, a.y[1], a.n[1]};
  p.mat2 = {a.w[2].weight, a.w[2].scale, a.y[2], a.n[2]};
  const Plan plan = make_plan(a.m, a.k, 1, false);
  if (plan.lds_bytes > 160 * 1024) return hipErrorInvalidValue;
  return launch<false>(p, 3, std::max(a.n[0], std::max(a.n[1], a.n[2])), plan, stream);
}

hipError_t launch_w4a16_gemv_mfma_dual_swiglu(const W4DualSwigluArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.gate.weight, a.gate.scale, a.product, a.n};
  p.mat1 = {a.up.weight, a.up.scale, a.product, a.n};
  p.mat2 = p.mat0;
  const Plan plan = make_plan(a.m, a.k, 2, false);
  if (plan.lds_bytes > 160 * 1024) return hipErrorInvalidValue;
  return launch<true>(p, 1, a.n, plan, stream);
}

}  // namespace llmopt
