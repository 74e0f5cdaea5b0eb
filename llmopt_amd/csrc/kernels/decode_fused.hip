// Fused launches of a decode step for gfx950 (one new token per sequence, activations of at most
// 2048 values): a 30-layer model at hidden 576 moves under 2 MB of weights per layer, so a step is
// bound by the number of its launches - each costs a kernel boundary and a first trip to memory,
// about 3 us together - and not by their bytes.  Two kernels, each doing in one launch what three or
// four reference kernels do in a row, with the same arithmetic at every rounding point:
//
//  * fused_qkv_kernel: llmopt_rms_norm_f16_simd (lib/metal_normalization_source.ml:70-91),
//    llmopt_w4a16_qkv_linear_f16_g64 (lib/metal_w4a16_source.ml:218-480),
//    llmopt_rotary_qk_f16_simd_h64 (lib/metal_normalization_source.ml:765-802) and
//    llmopt_cache_pack_attention_q8_pair_simd (lib/metal_cache_source.ml:105-182).  A workgroup owns
//    one head of 64 columns for its sequences: both halves of every rotation pair and the whole Q8
//    group are its own, nothing is handed over between workgroups.
//  * fused_ffn_kernel: llmopt_w4a16_swiglu_rms_f16_g64, llmopt_w4a16_dual_swiglu_f16_g64 and the
//    contraction of llmopt_w4a16_down_add_f16_g64 (lib/metal_w4a16_source.ml:496-611).  Workgroup j
//    owns a slice of 64 or 32 columns of the intermediate: gate and up for them, product =
//    half(silu(gate) * up), and that product times its columns of the down matrix - a partial sum of
//    every output, float32.  The sums over j and the residual are taken by whoever reads the stream
//    next (the next layer's fused_qkv_kernel): every workgroup there adds the partial sums in the
//    same fixed order, so the result does not depend on scheduling and no workgroup waits for
//    another.  Its own input may arrive the same way (rows plus the partial sums the projecting
//    attention merge left, one per head).
//
// What bounds a launch like these, measured with time stamps inside the kernels: the first trip to
// memory (about 2 us: argument block, then weights / activations / partial sums, all requested
// together), and then the *instructions* - a kernel's code is fetched cold on every launch (a pass
// over the same code a second time inside one launch runs 2.2 times faster than the first), and
// every vector instruction of a workgroup issues on the four SIMDs of its one CU at about 4.3 cycles
// each.  Hence: the weights go global -> LDS directly (no registers, no unrolled register sets), and
// everything after the one wait is a short loop over whole weight rows - small code, executed many
// times.
//
// Both kernels walk their weight rows the same way: a lane owns one 16-byte piece of a row (32 K
// values, inside one 64-wide scale group) and the matching 32 activations of its sequences, held in
// registers in the decoder's pair order; a wave's step covers as many whole rows as fit its 64 lanes
// (three rows of 576: 54 lanes busy).  Nibbles decode to exact fp16 integers with a bias that a
// per-lane correction removes (w4_common.h), v_dot2_f32_f16 accumulates in float32, the fp16 group
// scale is applied in float32, and the lanes of a row meet in a prefix sum over the wave whose
// differences at the row ends are the row sums.  The rows of the stream are normalised once per
// workgroup and left in LDS as halves.
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"
#include "w4_piece.h"

// Time stamps of one workgroup's phases for a scratch timing program (compiled out of the library).
#ifdef LLMOPT_FUSED_STAMPS
__device__ unsigned long long g_fused_stamps[32];
#define FUSED_STAMP(i)                                                                        \
  do {                                                                                        \
    if (blockIdx.x == LLMOPT_FUSED_STAMPS && blockIdx.y == 0 && threadIdx.x == 0) {           \
      g_fused_stamps[i] = wall_clock64();                                                     \
      g_fused_stamps[16 + i] = clock64();                                                     \
    }                                                                                         \
  } while (0)
#else
#define FUSED_STAMP(i)
#endif

namespace llmopt {
namespace {

#ifndef LLMOPT_FUSED_THREADS
#define LLMOPT_FUSED_THREADS 512
#endif
constexpr int kThreads = LLMOPT_FUSED_THREADS;
constexpr int kWaves = kThreads / 64;
constexpr int kHead = 64;  // columns a workgroup owns: one attention head, one Q8 group, one scale group of down

// Inclusive prefix sum over the 64 lanes (DPP shifts inside the 16-lane rows, then the last lane of a
// row broadcast into the rows above it).
__device__ __forceinline__ float wave_prefix_sum(float value) {
#define LLMOPT_DPP_ADD(control, row_mask)                                                                   \
  value += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), control, \
                                                                 row_mask, 0xF, false))
  LLMOPT_DPP_ADD(0x111, 0xF);  // row_shr:1
  LLMOPT_DPP_ADD(0x112, 0xF);  // row_shr:2
  LLMOPT_DPP_ADD(0x114, 0xF);  // row_shr:4
  LLMOPT_DPP_ADD(0x118, 0xF);  // row_shr:8
  LLMOPT_DPP_ADD(0x142, 0xA);  // row_bcast:15 into rows 1 and 3
  LLMOPT_DPP_ADD(0x143, 0xC);  // row_bcast:31 into rows 2 and 3
#undef LLMOPT_DPP_ADD
  return value;
}

__device__ __forceinline__ float lane_value(float value, uint32_t lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, value), (int)lane));
}

// `bytes` (a multiple of 16) from 16-byte aligned global memory straight into LDS, a KiB per wave
// instruction, no registers in between; piece i of the copy lands at destination + 16 i and comes from
// source(i).  Not waited for here.
template <typename Source>
__device__ __forceinline__ void copy_to_lds(uint8_t *destination, uint32_t bytes, Source source) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)destination;
  for (uint32_t first = wave * 1024; first < bytes; first += kWaves * 1024) {  // the same for a whole wave
    const uint32_t piece = (first >> 4) + lane;
    if (piece * 16 < bytes) {
      const uint8_t *from = source(piece);
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(base + first) : "memory");
    }
  }
#endif
}

__device__ __forceinline__ void wait_for_copies_and_meet() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
  __syncthreads();
}

// How the lanes of a wave share whole weight rows of `pieces` 16-byte pieces: `rows_per_step` rows per
// step (as many as fit, four at most), lane = row_in_step * pieces + piece.
struct RowLanes {
  uint32_t pieces, rows_per_step, row_in_step, piece;
  bool present;
  uint32_t weight_offset, scale_offset;  // of this lane's piece within a step's first row (bytes, halves)
  uint32_t last_lane[4];                 // last lane of row r of a step (wave-uniform)
  __device__ __forceinline__ RowLanes(uint32_t k) {
    const uint32_t lane = threadIdx.x & 63;
    pieces = k >> 5;
    rows_per_step = min(4u, 64u / pieces);
    const uint32_t row = lane / pieces;
    present = row < rows_per_step;
    row_in_step = present ? row : 0;
    piece = present ? lane - row * pieces : 0;
    weight_offset = row_in_step * (k >> 1) + piece * 16;
    scale_offset = row_in_step * (k >> 6) + (piece >> 1);
#pragma unroll
    for (int r = 0; r < 4; ++r) last_lane[r] = __builtin_amdgcn_readfirstlane(min((r + 1) * pieces, 64u) - 1);
  }
};

// Rows [row, row + rows_per_step) of a block of weight rows staged in LDS (rows side by side, their
// scales likewise; `weights_lds` / `scales_lds` at the step's first row) against the held
// activations: lane r < rows_per_step gets the sum of row `row + r` for sequence m in sums[m].  A
// step may reach past the block's last row: what it reads there is other LDS content, and the sums
// of those rows - later in lane order, so they touch no earlier row's prefix - are not used.
template <int M>
__device__ __forceinline__ void rows_dot(const RowLanes &lanes, const Held<M> &held, const uint8_t *weights_lds,
                                         const uint16_t *scales_lds, float (&sums)[M]) {
  const uint32_t lane = threadIdx.x & 63;
  const u32x4_t weights = *reinterpret_cast<const u32x4_t *>(weights_lds + lanes.weight_offset);
  const float scale = lanes.present ? half_bits_to_float(scales_lds[lanes.scale_offset]) : 0.0f;
  float share[M];
  piece_dot<M>(weights, scale, held, share);
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const float prefix = wave_prefix_sum(share[m]);
    const float t0 = lane_value(prefix, lanes.last_lane[0]), t1 = lane_value(prefix, lanes.last_lane[1]);
    const float t2 = lane_value(prefix, lanes.last_lane[2]), t3 = lane_value(prefix, lanes.last_lane[3]);
    sums[m] = lane == 0 ? t0 : lane == 1 ? t1 - t0 : lane == 2 ? t2 - t1 : t3 - t2;
  }
}

// The workgroup's M rows of the residual stream, normalised, into LDS as the halves the RMSNorm
// kernel would have stored (float32 products in its order).  A row is x plus, with PER > 0, the
// pending partial sums: the threads form `groups` groups, group g adds partial sums g, g + groups,
// g + 2 groups, ... (at most PER of them) for four values per thread, the group sums meet in LDS and
// are added in ascending order, then the residual, then one rounding to half - a fixed order, so
// every workgroup that reads the stream forms the same bits.  write_out: this workgroup stores the
// rows to in.x_out.  Barriers inside; every request is out before the first.
template <int M, int PER>
__device__ __forceinline__ void stage_normalised_rows(const FusedResidual &in, const W4Norm &norm, uint32_t rows,
                                                      uint32_t k, uint32_t row0, bool write_out, uint16_t *x_lds,
                                                      f4_t *group_lds, float (*square_lds)[kWaves]) {
  const uint32_t units_per_row = k >> 2;
  const uint32_t units = M * units_per_row;  // at most kThreads
  const uint32_t groups = PER > 0 ? min((uint32_t)kThreads / units, in.partial_count) : 1;
  const uint32_t group = threadIdx.x / units, unit = threadIdx.x - group * units;
  const uint32_t m = unit / units_per_row, column = (unit - m * units_per_row) * 4;
  const bool real = row0 + m < rows;
  const size_t at = (size_t)min(row0 + m, rows - 1) * k + column;
  const size_t partial_stride = (size_t)rows * k;
  uint2 residual = make_uint2(0, 0), gain = make_uint2(0, 0);
  if (group == 0) {
    residual = *reinterpret_cast<const uint2 *>(in.x + at);
    gain = *reinterpret_cast<const uint2 *>(norm.weight + column);
  }
  if constexpr (PER > 0) {
    if (group < groups) {
      f4_t pending[PER];
#pragma unroll
      for (int j = 0; j < PER; ++j)
        pending[j] = *reinterpret_cast<const f4_t *>(in.partials + min(group + j * groups, in.partial_count - 1) * partial_stride + at);
      f4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if (group + j * groups < in.partial_count) sum += pending[j];
      group_lds[group * units + unit] = sum;
    }
    wait_for_copies_and_meet();
  }
  float squares[M];
#pragma unroll
  for (int mm = 0; mm < M; ++mm) squares[mm] = 0.0f;
  float x[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (group == 0) {
    uint2 stored = residual;
    if constexpr (PER > 0) {
      f4_t sum = group_lds[unit];
      for (uint32_t g = 1; g < groups; ++g) sum += group_lds[g * units + unit];
      const h2_t lo = as_h2(residual.x), hi = as_h2(residual.y);
      const h2_t out_lo = {(_Float16)(sum[0] + (float)lo[0]), (_Float16)(sum[1] + (float)lo[1])};
      const h2_t out_hi = {(_Float16)(sum[2] + (float)hi[0]), (_Float16)(sum[3] + (float)hi[1])};
      stored = make_uint2(as_u32(out_lo), as_u32(out_hi));
    }
    if (write_out && real) *reinterpret_cast<uint2 *>(in.x_out + at) = stored;
    const h2_t lo = as_h2(stored.x), hi = as_h2(stored.y);
    x[0] = (float)lo[0], x[1] = (float)lo[1], x[2] = (float)hi[0], x[3] = (float)hi[1];
    const float square = (x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3]);
#pragma unroll
    for (int mm = 0; mm < M; ++mm) squares[mm] = (uint32_t)mm == m ? square : 0.0f;
  }
#pragma unroll
  for (int mm = 0; mm < M; ++mm) {
    const float total = wave_sum(squares[mm]);
    if ((threadIdx.x & 63) == 0) square_lds[mm][threadIdx.x >> 6] = total;
  }
  FUSED_STAMP(1);
  if constexpr (PER > 0) __syncthreads(); else wait_for_copies_and_meet();
  FUSED_STAMP(2);
  if (group == 0) {
    float square_sum = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      float of_wave = square_lds[0][w];
#pragma unroll
      for (int mm = 1; mm < M; ++mm) of_wave = (uint32_t)mm == m ? square_lds[mm][w] : of_wave;
      square_sum += of_wave;
    }
    const float inverse = rsqrtf(square_sum / (float)k + norm.epsilon);
    const h2_t g_lo = as_h2(gain.x), g_hi = as_h2(gain.y);
    const float g[4] = {(float)g_lo[0], (float)g_lo[1], (float)g_hi[0], (float)g_hi[1]};
    _Float16 y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = (_Float16)(norm.weight_first ? x[e] * g[e] * inverse : x[e] * inverse * g[e]);
    const h2_t y_lo = {y[0], y[1]}, y_hi = {y[2], y[3]};
    *reinterpret_cast<uint2 *>(x_lds + m * k + column) = make_uint2(as_u32(y_lo), as_u32(y_hi));
  }
  __syncthreads();
}

// LDS of a workgroup, carved from the dynamic block: everything 16-byte aligned.
struct Carve {
  uint8_t *next;
  __device__ __forceinline__ uint8_t *take(uint32_t bytes) {
    uint8_t *out = next;
    next += (bytes + 15) & ~15u;
    return out;
  }
};

// M: sequences per workgroup; PER: pending partial sums a thread adds on the way in (0: none).
template <int M, int PER>
__global__ __launch_bounds__(kThreads) void fused_qkv_kernel(FusedQkvArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t fused_lds[];
  __shared__ float square_lds[M][kWaves];
  __shared__ float head_lds[M][kHead];
  Carve carve = {fused_lds};
  uint8_t *weights_lds = carve.take(kHead * (a.k >> 1));
  uint16_t *scales_lds = reinterpret_cast<uint16_t *>(carve.take(kHead * (a.k >> 6) * 2));
  uint16_t *x_lds = reinterpret_cast<uint16_t *>(carve.take(M * a.k * 2));
  f4_t *group_lds = reinterpret_cast<f4_t *>(carve.take(PER > 0 ? kThreads * 16 : 0));
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t row0 = blockIdx.y * M;
  const uint32_t q_heads = a.n[0] / kHead, k_heads = a.n[1] / kHead;
  const uint32_t which = blockIdx.x < q_heads ? 0 : blockIdx.x < q_heads + k_heads ? 1 : 2;
  const uint32_t head = blockIdx.x - (which == 0 ? 0 : which == 1 ? q_heads : q_heads + k_heads);
  const W4Matrix matrix = which == 0 ? a.w[0] : which == 1 ? a.w[1] : a.w[2];

  // every request first: the head's weights and scales (whole rows side by side in memory), what the
  // epilogue needs (rotation row, pool slot), then the stream itself and the norm weights
  FUSED_STAMP(0);
  const uint8_t *head_weights = matrix.weight + (size_t)head * kHead * (a.k >> 1);
  const uint8_t *head_scales = reinterpret_cast<const uint8_t *>(matrix.scale + (size_t)head * kHead * (a.k >> 6));
  copy_to_lds(weights_lds, kHead * (a.k >> 1), [&](uint32_t piece) { return head_weights + (size_t)piece * 16; });
  copy_to_lds(reinterpret_cast<uint8_t *>(scales_lds), kHead * (a.k >> 6) * 2,
              [&](uint32_t piece) { return head_scales + (size_t)piece * 16; });
  const uint32_t epilogue_row = min(row0 + (wave < (uint32_t)M ? wave : 0), a.m - 1);
  const uint16_t cosine_bits = a.cosine[(size_t)epilogue_row * kHead + lane];
  const uint16_t sine_bits = a.sine[(size_t)epilogue_row * kHead + lane];
  const uint32_t slot = a.slots[epilogue_row];
  stage_normalised_rows<M, PER>(a.in, a.norm, a.m, a.k, row0, blockIdx.x == 0 && a.in.x_out != nullptr, x_lds,
                                group_lds, square_lds);
  FUSED_STAMP(3);

  const RowLanes lanes(a.k);
  Held<M> held;
  hold_rows<M>(held, x_lds, a.k, lanes.piece, lanes.present);
  FUSED_STAMP(4);
#pragma unroll 1
  for (uint32_t row = wave * lanes.rows_per_step; row < (uint32_t)kHead; row += kWaves * lanes.rows_per_step) {
    float sums[M];
    rows_dot<M>(lanes, held, weights_lds + row * (a.k >> 1), scales_lds + row * (a.k >> 6), sums);
#pragma unroll
    for (int m = 0; m < M; ++m)
      if (lane < lanes.rows_per_step && row + lane < (uint32_t)kHead) head_lds[m][row + lane] = sums[m];
  }
  FUSED_STAMP(5);
  __syncthreads();
  FUSED_STAMP(6);

  // wave m finishes sequence row0 + m: one column per lane
  if (wave >= (uint32_t)M || row0 + wave >= a.m) return;
  const uint32_t row = row0 + wave;
  const _Float16 value = (_Float16)head_lds[wave][lane];
  const _Float16 partner = (_Float16)head_lds[wave][lane ^ 32];
  const _Float16 turned = rotate_half_value(value, partner, __builtin_bit_cast(_Float16, cosine_bits),
                                            __builtin_bit_cast(_Float16, sine_bits), lane < 32);
  if (which == 0) {
    a.q_out[(size_t)row * a.n[0] + head * kHead + lane] = __builtin_bit_cast(uint16_t, turned);
    return;
  }
  const _Float16 kept = which == 1 ? turned : value;
  uint16_t *out = which == 1 ? a.k_out : a.v_out;
  out[(size_t)row * a.n[which] + head * kHead + lane] = __builtin_bit_cast(uint16_t, kept);
  const uint32_t segment = (which == 1 ? a.key_offset : a.value_offset) + head * kHead;
  uint8_t *token = a.pool + (size_t)slot * a.token_stride;
  uint16_t stored;
  reinterpret_cast<int8_t *>(token)[segment + lane] = q8_quantize((float)kept, &stored);
  if (lane == 0) reinterpret_cast<uint16_t *>(token + a.token_elements)[segment >> 6] = stored;
  FUSED_STAMP(8);
}

// PER: pending partial sums a thread adds to the stream on the way in (0: none), as in fused_qkv_kernel.
// SLICE: columns of the intermediate a workgroup owns, 64 or 32.  Half the columns are half the bytes a CU has
// to pull in before it can start (a CU fills its LDS at about 80 bytes a nanosecond: the 55 KB of a 64-wide
// slice at hidden 576 were not all requested until 1.1 us into the kernel) and half the arithmetic on its four
// SIMDs, for twice the partial sums the next reader adds.
template <int M, int PER, int SLICE>
__global__ __launch_bounds__(kThreads) void fused_ffn_kernel(FusedFfnArgs a) {
  static_assert(SLICE == 32 || SLICE == 64, "whole 16-byte pieces of a down-projection row");
  constexpr int kPieces = SLICE / 32;  // 16-byte pieces of a down-projection row inside the slice
  extern __shared__ __attribute__((aligned(16))) uint8_t fused_lds[];
  __shared__ float square_lds[M][kWaves];
  __shared__ __attribute__((aligned(16))) uint16_t product_lds[M][SLICE];
  Carve carve = {fused_lds};
  const uint32_t row_bytes = a.k >> 1, scale_bytes = SLICE * (a.k >> 6) * 2;
  uint8_t *gate_lds = carve.take(SLICE * row_bytes);
  uint8_t *up_lds = carve.take(SLICE * row_bytes);
  uint16_t *gate_scales_lds = reinterpret_cast<uint16_t *>(carve.take(scale_bytes));
  uint16_t *up_scales_lds = reinterpret_cast<uint16_t *>(carve.take(scale_bytes));
  uint8_t *down_lds = carve.take(a.k * (SLICE / 2));  // SLICE / 2 bytes a row: the slice's columns
  uint16_t *down_scales_lds = reinterpret_cast<uint16_t *>(carve.take(a.k * 2));
  uint16_t *x_lds = reinterpret_cast<uint16_t *>(carve.take(M * a.k * 2));
  f4_t *group_lds = reinterpret_cast<f4_t *>(carve.take(PER > 0 ? kThreads * 16 : 0));
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t row0 = blockIdx.y * M;
  const uint32_t slice = blockIdx.x;  // intermediate columns [SLICE slice, SLICE slice + SLICE)

  FUSED_STAMP(0);
  const uint8_t *gate_weights = a.gate.weight + (size_t)slice * SLICE * row_bytes;
  const uint8_t *up_weights = a.up.weight + (size_t)slice * SLICE * row_bytes;
  const uint8_t *gate_scales = reinterpret_cast<const uint8_t *>(a.gate.scale + (size_t)slice * SLICE * (a.k >> 6));
  const uint8_t *up_scales = reinterpret_cast<const uint8_t *>(a.up.scale + (size_t)slice * SLICE * (a.k >> 6));
  copy_to_lds(gate_lds, SLICE * row_bytes, [&](uint32_t piece) { return gate_weights + (size_t)piece * 16; });
  copy_to_lds(up_lds, SLICE * row_bytes, [&](uint32_t piece) { return up_weights + (size_t)piece * 16; });
  copy_to_lds(reinterpret_cast<uint8_t *>(gate_scales_lds), scale_bytes, [&](uint32_t piece) { return gate_scales + (size_t)piece * 16; });
  copy_to_lds(reinterpret_cast<uint8_t *>(up_scales_lds), scale_bytes, [&](uint32_t piece) { return up_scales + (size_t)piece * 16; });
  // down: row r of the slice is SLICE / 2 bytes, kPieces pieces
  const uint8_t *down_weights = a.down.weight + (size_t)slice * (SLICE / 2);
  copy_to_lds(down_lds, a.k * (SLICE / 2), [&](uint32_t piece) {
    return down_weights + (size_t)(piece / kPieces) * (a.n >> 1) + (piece % kPieces) * 16;
  });
  // (the scales of the slice's down rows pass registers: two bytes a row, 2 n / 64 bytes apart)
  constexpr int kScalePasses = (int)kFusedMaxWidth / kThreads;
  uint16_t down_scales[kScalePasses];
  const uint32_t down_group = (slice * SLICE) >> 6;  // the scale group of the down rows the slice lies in
#pragma unroll
  for (int pass = 0; pass < kScalePasses; ++pass)
    down_scales[pass] = a.down.scale[(size_t)min(threadIdx.x + pass * kThreads, a.k - 1) * (a.n >> 6) + down_group];
  stage_normalised_rows<M, PER>(a.in, a.norm, a.m, a.k, row0, blockIdx.x == 0 && a.in.x_out != nullptr, x_lds, group_lds,
                                square_lds);
#pragma unroll
  for (int pass = 0; pass < kScalePasses; ++pass)
    if (threadIdx.x + pass * kThreads < a.k) down_scales_lds[threadIdx.x + pass * kThreads] = down_scales[pass];
  FUSED_STAMP(3);

  {
    const RowLanes lanes(a.k);
    Held<M> held;
    hold_rows<M>(held, x_lds, a.k, lanes.piece, lanes.present);
    FUSED_STAMP(4);
#pragma unroll 1
    for (uint32_t row = wave * lanes.rows_per_step; row < (uint32_t)SLICE; row += kWaves * lanes.rows_per_step) {
      float gate[M], up[M];
      rows_dot<M>(lanes, held, gate_lds + row * row_bytes, gate_scales_lds + row * (a.k >> 6), gate);
      rows_dot<M>(lanes, held, up_lds + row * row_bytes, up_scales_lds + row * (a.k >> 6), up);
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (lane < lanes.rows_per_step && row + lane < (uint32_t)SLICE)
          product_lds[m][row + lane] = float_to_half_bits(gate[m] / (1.0f + __expf(-gate[m])) * up[m]);
    }
    FUSED_STAMP(5);
  }
  __syncthreads();
  FUSED_STAMP(6);

  // kPieces neighbouring lanes own an output row (+ kThreads / kPieces per pass): each lane 32 of the slice's columns
  const uint32_t piece_select = threadIdx.x % kPieces;
  Held<M> held;
  hold_rows<M>(held, &product_lds[0][0], SLICE, piece_select, true);
#pragma unroll 1
  for (uint32_t column = threadIdx.x / kPieces; column < a.k; column += kThreads / kPieces) {
    const u32x4_t weights = *reinterpret_cast<const u32x4_t *>(down_lds + column * (SLICE / 2) + piece_select * 16);
    float share[M];
    piece_dot<M>(weights, half_bits_to_float(down_scales_lds[column]), held, share);
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float total = share[m];
      if constexpr (kPieces == 2)
        total += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, share[m]), 0xB1, 0xF, 0xF, false));
      if (piece_select == 0 && row0 + m < a.m) a.partials[((size_t)slice * a.m + row0 + m) * a.k + column] = total;
    }
  }
  FUSED_STAMP(8);
}

bool aligned16(const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15) == 0; }

constexpr size_t kLdsBudget = 150 * 1024;
size_t ffn_lds_bytes(uint32_t rows, uint32_t k, bool partials, uint32_t slice = 64);

// Sequences per workgroup: one, until the launch has more workgroups than the device holds at once
// (two share a workgroup's decoded weights; their rows must fit one pass of the staging).
uint32_t rows_per_workgroup(uint32_t m, uint32_t k, uint32_t column_blocks, uint32_t slice = 64) {
  return (uint64_t)m * column_blocks > 2ull * (uint32_t)device_compute_units() && 2 * (k >> 2) <= (uint32_t)kThreads &&
                 ffn_lds_bytes(2, k, true, slice) <= kLdsBudget
             ? 2
             : 1;
}

uint32_t padded(uint32_t bytes) { return (bytes + 15) & ~15u; }

size_t qkv_lds_bytes(uint32_t rows, uint32_t k, bool partials) {
  return padded(kHead * (k >> 1)) + padded(kHead * (k >> 6) * 2) + padded(rows * k * 2) + (partials ? kThreads * 16 : 0);
}

size_t ffn_lds_bytes(uint32_t rows, uint32_t k, bool partials, uint32_t slice) {
  return 2 * padded(slice * (k >> 1)) + 2 * padded(slice * (k >> 6) * 2) + padded(k * (slice / 2)) + padded(k * 2) +
         padded(rows * k * 2) + (partials ? kThreads * 16 : 0);
}

// Partial sums a thread adds on the way in: groups of threads share them (stage_normalised_rows).
uint32_t partials_per_thread(uint32_t rows, uint32_t k, uint32_t partial_count) {
  if (partial_count == 0) return 0;
  const uint32_t units = rows * (k >> 2);
  const uint32_t groups = std::min<uint32_t>(kThreads / units, partial_count);
  return (partial_count + groups - 1) / groups;
}

template <int M, int PER>
hipError_t launch_qkv_instance(const FusedQkvArgs &a, dim3 grid, size_t lds, hipStream_t stream) {
  static bool configured[kMaxDevices] = {};
  if (lds > 64 * 1024)
    if (hipError_t status = allow_dynamic_lds(reinterpret_cast<const void *>(fused_qkv_kernel<M, PER>), 158 * 1024, configured))
      return status;
  hipLaunchKernelGGL((fused_qkv_kernel<M, PER>), grid, dim3(kThreads), lds, stream, a);
  return hipGetLastError();
}

template <int M>
hipError_t launch_qkv_rows(const FusedQkvArgs &a, dim3 grid, hipStream_t stream) {
  const uint32_t per = partials_per_thread(M, a.k, a.in.partial_count);
  const size_t lds = qkv_lds_bytes(M, a.k, per != 0);
  if (per == 0) return launch_qkv_instance<M, 0>(a, grid, lds, stream);
  if (per <= 8) return launch_qkv_instance<M, 8>(a, grid, lds, stream);
  if (per <= 16) return launch_qkv_instance<M, 16>(a, grid, lds, stream);
  return launch_qkv_instance<M, 32>(a, grid, lds, stream);
}

template <int M, int PER, int SLICE>
hipError_t launch_ffn_instance(const FusedFfnArgs &a, dim3 grid, size_t lds, hipStream_t stream) {
  static bool configured[kMaxDevices] = {};
  if (lds > 64 * 1024)
    if (hipError_t status =
            allow_dynamic_lds(reinterpret_cast<const void *>(fused_ffn_kernel<M, PER, SLICE>), 158 * 1024, configured))
      return status;
  hipLaunchKernelGGL((fused_ffn_kernel<M, PER, SLICE>), grid, dim3(kThreads), lds, stream, a);
  return hipGetLastError();
}

template <int M, int SLICE>
hipError_t launch_ffn_rows(const FusedFfnArgs &a, dim3 grid, hipStream_t stream) {
  const uint32_t per = partials_per_thread(M, a.k, a.in.partial_count);
  const size_t lds = ffn_lds_bytes(M, a.k, per != 0, SLICE);
  if (per == 0) return launch_ffn_instance<M, 0, SLICE>(a, grid, lds, stream);
  if (per <= 8) return launch_ffn_instance<M, 8, SLICE>(a, grid, lds, stream);
  if (per <= 16) return launch_ffn_instance<M, 16, SLICE>(a, grid, lds, stream);
  return launch_ffn_instance<M, 32, SLICE>(a, grid, lds, stream);
}

}  // namespace

bool fused_qkv_ok(const FusedQkvArgs &a) {
  if (a.m == 0 || a.k == 0 || a.k % 64 != 0 || a.k > kFusedMaxWidth) return false;
  for (int i = 0; i < 3; ++i)
    if (a.n[i] == 0 || a.n[i] % kHead != 0 || !aligned16(a.w[i].weight) || !aligned16(a.w[i].scale)) return false;
  if (a.in.partial_count > kFusedMaxPartials) return false;
  if (partials_per_thread(1, a.k, a.in.partial_count) > 32) return false;
  if (a.in.partial_count != 0 && (a.in.partials == nullptr || !aligned16(a.in.partials))) return false;
  if (a.token_stride % 2 != 0 || a.token_elements % 2 != 0) return false;
  return aligned16(a.in.x) && aligned16(a.norm.weight) && (a.in.x_out == nullptr || aligned16(a.in.x_out));
}

hipError_t launch_fused_qkv(const FusedQkvArgs &a, hipStream_t stream) {
  if (!fused_qkv_ok(a)) return hipErrorInvalidValue;
  const uint32_t heads = (a.n[0] + a.n[1] + a.n[2]) / kHead;
  uint32_t per = rows_per_workgroup(a.m, a.k, heads);
  if (per == 2 && partials_per_thread(2, a.k, a.in.partial_count) > 32) per = 1;
  const dim3 grid(heads, (a.m + per - 1) / per);
  return per == 1 ? launch_qkv_rows<1>(a, grid, stream) : launch_qkv_rows<2>(a, grid, stream);
}

bool fused_ffn_ok(uint32_t m, uint32_t n, uint32_t k, bool pending, uint32_t slice) {
  return (slice == 32 || slice == 64) && m != 0 && k != 0 && k % 64 == 0 && k <= kFusedMaxWidth &&
         ffn_lds_bytes(1, k, pending, slice) <= kLdsBudget && n != 0 && n % slice == 0 && n / slice <= kFusedMaxPartials;
}

hipError_t launch_fused_ffn(const FusedFfnArgs &a, hipStream_t stream) {
  if (a.in.partial_count > kFusedMaxPartials || partials_per_thread(1, a.k, a.in.partial_count) > 32) return hipErrorInvalidValue;
  if (a.in.partial_count != 0 && (a.in.partials == nullptr || !aligned16(a.in.partials))) return hipErrorInvalidValue;
  if (a.in.x_out != nullptr && (!aligned16(a.in.x_out) || a.in.x_out == a.in.x)) return hipErrorInvalidValue;
  if (!fused_ffn_ok(a.m, a.n, a.k, a.in.partial_count != 0, a.slice) || !aligned16(a.in.x) || !aligned16(a.norm.weight) || !aligned16(a.gate.weight) ||
      !aligned16(a.up.weight) || !aligned16(a.down.weight) || !aligned16(a.partials) || !aligned16(a.gate.scale) ||
      !aligned16(a.up.scale))
    return hipErrorInvalidValue;
  const uint32_t slices = a.n / a.slice;
  uint32_t per = rows_per_workgroup(a.m, a.k, slices, a.slice);
  if (per == 2 && partials_per_thread(2, a.k, a.in.partial_count) > 32) per = 1;
  const dim3 grid(slices, (a.m + per - 1) / per);
  if (a.slice == 32) return per == 1 ? launch_ffn_rows<1, 32>(a, grid, stream) : launch_ffn_rows<2, 32>(a, grid, stream);
  return per == 1 ? launch_ffn_rows<1, 64>(a, grid, stream) : launch_ffn_rows<2, 64>(a, grid, stream);
}

}  // namespace llmopt
