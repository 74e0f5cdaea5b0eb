// W4A16 decode GEMV for one to four activation rows on v_mfma_f32_4x4x4_16B_f16, one workgroup
// per CU, every weight byte requested exactly once and in whole 256-byte row pieces.
//
// Semantics: llmopt_w4a16_linear_f16_g64{,_m4} (lib/metal_w4a16_source.ml:8-194, CPU meaning
// lib/cpu.ml:128-152): y[r, c] = half(sum_k x[r, k] * q[c, k] * s[c, k / 64] (+ addend)).
//
// Geometry.  The instruction multiplies sixteen independent 4x4x4 blocks, one per group of four
// lanes.  Block b of a wave takes the 32-wide K slice b of a 512-wide K range; its four lanes
// j = 0..3 each load 16 bytes (32 nibbles) of weight row 4 * quad + j, so a wave's load
// instruction reads 256 contiguous bytes of each of four weight rows.  The activation is the A
// operand (rows = activation rows, zero rows beyond m), the weights the B operand (columns =
// the four weight rows): lane (b, j) ends with D[i] = sum over its block's 32 K values of
// x[i, k] * w[row j, k], i.e. every lane's four results belong to the weight row whose bytes -
// and whose scale group - that lane loaded: the fp16 group scale is one multiply per lane and
// K range in float32.  A wave owns RQ row quads over the whole of K and keeps their running
// sums in registers; the sixteen blocks' sums meet once, at the end (DPP row rotations and two
// cross-row exchanges), so there is no barrier and no LDS traffic in the reduction.
//
// The activation (all of it: m x K halves) and the workgroup's scales are staged in LDS once,
// the activation in the nibble decoder's pair order together with the decode-bias correction of
// every 32-wide piece (the nibbles are decoded to q + 1032 / q + 72 with one bit operation per
// pair, w4_decode_biased; the MFMA chain of a piece starts from -(1032 * sum x + 72 * sum x)).
// Order of the requests at the start of a workgroup: activation, scales, then only EARLY weight
// loads per wave before the staging waits - a CU's vector memory requests return in issue order
// and a wave stalls at issue once the CU's queue is full, so a long burst of weight loads ahead
// of another wave's activation request would hold the whole workgroup at its barrier - and the
// rest of the ring of DEPTH loads right after.
//
// The K ranges of 512 are a template parameter: strides in LDS, the ring indices and the (unrolled)
// walk over K are compile-time.  K = 4096 and K = 14336 have instantiations of exactly their length;
// at three and four activation rows every other multiple of 128 from 2048 to 8192 runs an
// instantiation whose LDS layout and unrolled walk are cut for the longest such row, with the row's
// real length a launch argument: what lies beyond the row's end is skipped.  (Walking K in a real loop
// was measured twice, with the compiler's waits and with requests in assembly waited for by count:
// 1.3 - 2.6 TB/s against the unrolled walk's 3.9 - 4.4 - a loop's back edge costs the ring its depth.)  Other shapes keep the kernels of w4a16_gemv.hip /
// w4a16_gemv_mfma.hip.  N from 3072 up: beyond one round of workgroups the launch makes several.
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

struct QuadParams {
  const uint16_t *x;
  const uint8_t *w;
  const uint16_t *s;
  uint16_t *y;
  const uint16_t *addend;
  uint32_t has_addend, addend_stride;
  uint32_t m, n, k;
};

__device__ __forceinline__ h4_t pack_h4(uint32_t lo, uint32_t hi) {
  return __builtin_bit_cast(h4_t, make_uint2(lo, hi));
}

__device__ __forceinline__ float dpp_row_rotate4(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_row_rotate8(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true));
}

// Bytes of LDS one workgroup of `waves` working waves needs.
template <int MR, int KL, int RQ>
constexpr size_t quad_lds_bytes(uint32_t waves) {
  return (size_t)MR * (2 * KL * 512 + 16) + (size_t)KL * 16 * 16 + (size_t)waves * RQ * 4 * (KL * 16 + 16);
}

// MR: activation rows staged (m <= MR <= 4); KL: K / 512 (EXACT) or the most K ranges the
// instantiation's LDS layout holds (K = p.k is then any multiple of 512 up to 512 KL, and the walk
// over K stops where the row ends); RQ: row quads per wave; DEPTH: weight loads in flight per wave;
// EARLY: how many of them go out before the staging waits; THREADS: workgroup size (waves beyond
// units_per_wg only help staging).
// Registers: a workgroup is one wave per SIMD, and told only that, the compiler spreads itself over
// the 512 registers a lone wave may have (220 at one row of K = 14336, half of them accumulator
// registers used as spill space) - a CU then holds nothing beside this workgroup, and launches that
// do not depend on each other cannot run side by side on it.  Asked for three waves per SIMD (two at
// four rows, one for the long-row instantiations with two quads per wave, which need the room) the
// same kernels take 58-128 registers with nothing spilled and run a little faster: the serial sweep
// 91.5 -> 90.0 us a step, 85.1 -> 82.9 on two concurrent graph branches (four branches: 70.7-72.0
// either way, within what two runs differ by).
template <int MR, int KL, int RQ>
constexpr int quad_waves_per_simd() {
  return (KL > 8 && RQ == 2) ? 1 : MR <= 2 ? 3 : 2;
}

template <int MR, int KL, int RQ, int DEPTH, int EARLY, int THREADS, bool EXACT = true>
__global__ __launch_bounds__(THREADS)
    __attribute__((amdgpu_waves_per_eu(quad_waves_per_simd<MR, KL, RQ>(), quad_waves_per_simd<MR, KL, RQ>()))) void
    w4a16_gemv_quad_kernel(QuadParams p, uint32_t units_per_wg) {
  static_assert(MR >= 1 && MR <= 4 && EARLY >= 1 && EARLY <= DEPTH && DEPTH <= KL * RQ && THREADS % 64 == 0, "shape");
  constexpr uint32_t KMAX = KL * 512;                  // what the LDS layout is cut for
  const uint32_t K = EXACT ? KMAX : p.k;               // a constant in the exact instantiations
  const uint32_t row_bytes = K / 2, groups = K / 64;
  constexpr uint32_t kRowStride = 2 * KMAX + 16;         // bytes between activation rows in LDS
  constexpr uint32_t kScaleStride = (KMAX / 64) * 2 + 16;  // bytes between scale rows in LDS
  constexpr uint32_t kXUnits = MR * (KMAX / 8);          // 16-byte units of activation to stage
  constexpr int XPER = (kXUnits + THREADS - 1) / THREADS;
  const uint32_t kScaleUnitsPerRow = groups * 2 / 16;
  constexpr int SPER = ((THREADS / 64) * RQ * 4 * ((KMAX / 64) * 2 / 16) + THREADS - 1) / THREADS;
  constexpr int TOTAL_MAX = KL * RQ;
  // K ranges of the row: the last one may be partly there (K a multiple of 128): its missing
  // activations are staged as zeros, its weight requests held inside the row, its scales to the
  // row's last group
  const uint32_t ranges = EXACT ? KL : (K + 511) / 512;
  const int TOTAL = EXACT ? TOTAL_MAX : (int)ranges * RQ;
  const uint32_t scale_pitch = EXACT ? kScaleStride : groups * 2;  // other K: rows side by side, as in memory
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned char *xs = lds_raw;
  float *cin = reinterpret_cast<float *>(lds_raw + MR * kRowStride);  // [piece of 32 K][activation row 0..3]
  unsigned char *ss = lds_raw + MR * kRowStride + KL * 16 * 16;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t b = lane >> 2, j = lane & 3;
  const uint32_t quads = p.n >> 2;
  const uint32_t rows_per_wg = units_per_wg * RQ * 4;
  const uint32_t row0 = blockIdx.x * rows_per_wg;

  // 1. activation and scale requests (clamped, never past the buffers; masked when staged)
  // Unit e of a thread is 16-byte unit `u` of activation row `row`.  When a row is a whole
  // number of passes of the workgroup both are known without a division: the staging runs once
  // per unit, and every vector instruction in it costs four cycles a wave.
  // (Rows are laid out for KMAX values; of a shorter row only the first K / 8 units exist.)
  constexpr bool kWholePasses = (KMAX / 8) % THREADS == 0;
  constexpr uint32_t kPassesPerRow = kWholePasses ? (KMAX / 8) / THREADS : 1;
  auto unit_of = [&](int e, uint32_t &row, uint32_t &u, bool &inside) __attribute__((always_inline)) {
    if constexpr (kWholePasses) {
      row = (uint32_t)e / kPassesPerRow;
      u = threadIdx.x + ((uint32_t)e % kPassesPerRow) * THREADS;
      inside = EXACT || u < ranges * 64;
    } else {
      const uint32_t idx = threadIdx.x + e * THREADS;
      row = min(idx, kXUnits - 1) / (KMAX / 8);
      u = min(idx, kXUnits - 1) % (KMAX / 8);
      inside = idx < kXUnits && (EXACT || u < ranges * 64);
    }
  };
  uint4 xin[XPER];
#pragma unroll
  for (int e = 0; e < XPER; ++e) {
    uint32_t row, u;
    bool inside;
    unit_of(e, row, u, inside);
    xin[e] = reinterpret_cast<const uint4 *>(p.x + (size_t)min(row, p.m - 1) * K)[EXACT ? u : min(u, K / 8 - 1)];
  }
  const uint32_t scale_units = EXACT ? rows_per_wg * kScaleUnitsPerRow : rows_per_wg * groups * 2 / 16;
  const size_t s_first = (size_t)row0 * groups * 2, s_last = (size_t)p.n * groups * 2 - 16;
  // (four named registers, not an array: left as an array the compiler kept it in scratch memory
  // and waited for these loads right here, before the first weight request, to store them there)
  static_assert(SPER <= 4, "scale vectors per thread");
  auto scale_request = [&](int e) __attribute__((always_inline)) {
    return *reinterpret_cast<const uint4 *>(reinterpret_cast<const unsigned char *>(p.s) +
                                            min(s_first + (size_t)(threadIdx.x + e * THREADS) * 16, s_last));
  };
  uint4 scale_in0 = make_uint4(0, 0, 0, 0), scale_in1 = scale_in0, scale_in2 = scale_in0, scale_in3 = scale_in0;
  scale_in0 = scale_request(0);
  if constexpr (SPER > 1) scale_in1 = scale_request(1);
  if constexpr (SPER > 2) scale_in2 = scale_request(2);
  if constexpr (SPER > 3) scale_in3 = scale_request(3);
  // 2. the first weights
  const uint32_t unit = __builtin_amdgcn_readfirstlane(blockIdx.x * units_per_wg + min(wave, units_per_wg - 1));
  u32x4_t wreg[DEPTH];
  const uint32_t w_lane = j * row_bytes + b * 16;
  // the lane's piece of the row's last K range, held inside the row when that range is partly there
  const uint32_t w_lane_last = EXACT ? w_lane : j * row_bytes + min(b * 16, row_bytes - (ranges - 1) * 256 - 16);
  const uint8_t *w_quad[RQ];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) {
    const uint32_t quad = __builtin_amdgcn_readfirstlane(min(unit * RQ + rq, quads - 1));
    w_quad[rq] = p.w + (size_t)quad * 4 * row_bytes;
  }
  auto ring_request = [&](u32x4_t &into, const uint8_t *address) __attribute__((always_inline)) {
    into = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(address));
  };
  uint16_t addend_bits[RQ][MR] = {};
  if (!EXACT && p.has_addend) {
    // (other K: the addend goes out first and lands first; nothing but the ring is then requested in the walk)
#pragma unroll
    for (int q = 0; q < RQ; ++q)
#pragma unroll
      for (int i = 0; i < MR; ++i)
        addend_bits[q][i] = p.addend[(size_t)min((uint32_t)i, p.m - 1) * p.addend_stride + min(unit * RQ + q, quads - 1) * 4 + j];
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int n = 0; n < EARLY; ++n) ring_request(wreg[n], w_quad[n % RQ] + (n / RQ) * 256 + w_lane);
  __builtin_amdgcn_sched_barrier(0);
  if (EARLY < DEPTH) {
    // loads return in issue order: with only the early weights outstanding, the activation and
    // the scales have landed
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(EARLY) : "memory");
#pragma unroll
    for (int n = EARLY; n < DEPTH; ++n) ring_request(wreg[n], w_quad[n % RQ] + (n / RQ) * 256 + w_lane);
    __builtin_amdgcn_sched_barrier(0);
  }
  // 3. stage: pair order, the decode-bias correction of every 32-K piece, the scales
  const h2_t bias_even = {(_Float16)1032.0f, (_Float16)1032.0f}, bias_odd = {(_Float16)72.0f, (_Float16)72.0f};
#pragma unroll
  for (int e = 0; e < XPER; ++e) {
    uint32_t row, u;
    bool inside;
    unit_of(e, row, u, inside);
    uint4 v = pair_order(xin[e]);
    if (row >= p.m || (!EXACT && u >= K / 8)) v = make_uint4(0, 0, 0, 0);
    // 1032 * (x0 + x4 + x2 + x6) + 72 * (x1 + x5 + x3 + x7): exact products, float32 sums
    float corr = __builtin_amdgcn_fdot2(as_h2(v.x), bias_even, 0.0f, false);
    corr = __builtin_amdgcn_fdot2(as_h2(v.z), bias_even, corr, false);
    corr = __builtin_amdgcn_fdot2(as_h2(v.y), bias_odd, corr, false);
    corr = __builtin_amdgcn_fdot2(as_h2(v.w), bias_odd, corr, false);
    // the four 16-byte units of a piece sit in four neighbouring lanes (K / 8 and THREADS are multiples of 4)
    corr += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, corr), 0xB1, 0xF, 0xF, true));
    corr += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, corr), 0x4E, 0xF, 0xF, true));
    if (inside) {
      *reinterpret_cast<uint4 *>(xs + row * kRowStride + u * 16) = v;
      if ((u & 3) == 0) cin[(u >> 2) * 4 + row] = -corr;
    }
  }
  // (corrections of A rows beyond MR are never written: those rows of D are never read)
  auto scale_store = [&](int e, const uint4 &value) __attribute__((always_inline)) {
    const uint32_t idx = threadIdx.x + e * THREADS;
    if (idx < scale_units) {
      if constexpr (EXACT)
        *reinterpret_cast<uint4 *>(ss + (idx / kScaleUnitsPerRow) * kScaleStride + (idx % kScaleUnitsPerRow) * 16) = value;
      else
        *reinterpret_cast<uint4 *>(ss + idx * 16) = value;
    }
  };
  scale_store(0, scale_in0);
  if constexpr (SPER > 1) scale_store(1, scale_in1);
  if constexpr (SPER > 2) scale_store(2, scale_in2);
  if constexpr (SPER > 3) scale_store(3, scale_in3);
  __syncthreads();
  if (wave >= units_per_wg) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }
  // 4. the wave's rows
  f4_t acc[RQ];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) acc[rq] = f4_t{0.f, 0.f, 0.f, 0.f};
  uint4 xa[4];
  f4_t cinit;
  const unsigned char *my_scales = ss + (wave * RQ * 4 + j) * scale_pitch + (EXACT ? (b >> 1) * 2 : 0);
  if constexpr (EXACT) {
  #pragma unroll
    for (int n = 0; n < TOTAL_MAX; ++n) {
      const int kp = n / RQ, rq = n % RQ;
      if (rq == 0) {
  #pragma unroll
        for (int t = 0; t < 4; ++t) {
          xa[t] = make_uint4(0, 0, 0, 0);
          if (j < MR) xa[t] = *reinterpret_cast<const uint4 *>(xs + j * kRowStride + (kp * 64 + 4 * b + t) * 16);
        }
        cinit = *reinterpret_cast<const f4_t *>(cin + (kp * 16 + b) * 4);
      }
      const uint16_t scale_bits = *reinterpret_cast<const uint16_t *>(
          my_scales + rq * 4 * scale_pitch + (uint32_t)kp * 16);
      const u32x4_t words = wreg[n % DEPTH];
      f4_t d = cinit;
  #pragma unroll
      for (int t = 0; t < 4; ++t) {
        const W4Pairs pr = w4_decode_biased(words[t]);
        d = __builtin_amdgcn_mfma_f32_4x4x4f16(pack_h4(xa[t].x, xa[t].y), pack_h4(as_u32(pr.p04), as_u32(pr.p15)), d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_4x4x4f16(pack_h4(xa[t].z, xa[t].w), pack_h4(as_u32(pr.p26), as_u32(pr.p37)), d, 0, 0, 0);
      }
      if (n + DEPTH < TOTAL)
        wreg[n % DEPTH] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4_t *>(w_quad[(n + DEPTH) % RQ] + ((n + DEPTH) / RQ) * 256 + w_lane));
      if (n + DEPTH == TOTAL && p.has_addend) {
        // The addend of this wave's outputs is requested right behind its last weights: it lands
        // with them, and the store path has no load of its own to wait for.  Every lane reads
        // (lanes 0..3 hold row 4 * quad + j; the others repeat them), clamped into the buffer.
  #pragma unroll
        for (int q = 0; q < RQ; ++q)
  #pragma unroll
          for (int i = 0; i < MR; ++i)
            addend_bits[q][i] = p.addend[(size_t)min((uint32_t)i, p.m - 1) * p.addend_stride +
                                         min(unit * RQ + q, quads - 1) * 4 + j];
      }
      const float scale = half_bits_to_float(scale_bits);
  #pragma unroll
      for (int i = 0; i < 4; ++i) acc[rq][i] = fmaf(d[i], scale, acc[rq][i]);
    }
  } else {
    // The unrolled walk of the longest row this instantiation's LDS layout holds; what lies beyond the
    // row's real end is skipped (the same for every wave).
#pragma unroll
    for (int n = 0; n < TOTAL_MAX; ++n) {
      if (n >= TOTAL) continue;
      const int kp = n / RQ, rq = n % RQ;
      if (rq == 0) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          xa[t] = make_uint4(0, 0, 0, 0);
          if (j < MR) xa[t] = *reinterpret_cast<const uint4 *>(xs + j * kRowStride + (kp * 64 + 4 * b + t) * 16);
        }
        cinit = *reinterpret_cast<const f4_t *>(cin + (kp * 16 + b) * 4);
      }
      const uint16_t scale_bits = *reinterpret_cast<const uint16_t *>(
          my_scales + rq * 4 * scale_pitch + min((uint32_t)kp * 8 + (b >> 1), groups - 1) * 2);
      const u32x4_t words = wreg[n % DEPTH];
      f4_t d = cinit;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const W4Pairs pr = w4_decode_biased(words[t]);
        d = __builtin_amdgcn_mfma_f32_4x4x4f16(pack_h4(xa[t].x, xa[t].y), pack_h4(as_u32(pr.p04), as_u32(pr.p15)), d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_4x4x4f16(pack_h4(xa[t].z, xa[t].w), pack_h4(as_u32(pr.p26), as_u32(pr.p37)), d, 0, 0, 0);
      }
      if (n + DEPTH < TOTAL)
        wreg[n % DEPTH] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(
            w_quad[(n + DEPTH) % RQ] + ((n + DEPTH) / RQ) * 256 +
            ((uint32_t)((n + DEPTH) / RQ) == ranges - 1 ? w_lane_last : w_lane)));
      const float scale = half_bits_to_float(scale_bits);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[rq][i] = fmaf(d[i], scale, acc[rq][i]);
    }
  }
  // 5. sum over the sixteen blocks (lanes j + 4 b) and store
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) {
    const uint32_t quad = unit * RQ + rq;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
      float v = acc[rq][i];
      v += dpp_row_rotate4(v);
      v += dpp_row_rotate8(v);
      v += __shfl_xor(v, 16);
      v += __shfl_xor(v, 32);
      if (lane < 4 && (uint32_t)i < p.m && quad < quads)
        p.y[(size_t)i * p.n + quad * 4 + j] =
            float_to_half_bits(p.has_addend ? v + half_bits_to_float(addend_bits[rq][i]) : v);
    }
  }
}

template <int MR, int KL, int RQ, int DEPTH, int EARLY, int THREADS, bool EXACT = true>
hipError_t launch_instance(const QuadParams &p, uint32_t grid, uint32_t units_per_wg, hipStream_t stream) {
  const size_t lds = quad_lds_bytes<MR, KL, RQ>(units_per_wg);
  auto kernel = &w4a16_gemv_quad_kernel<MR, KL, RQ, DEPTH, EARLY, THREADS, EXACT>;
  static bool configured[kMaxDevices] = {};  // once per device: the kernel may use more than the default 64 KB of LDS
  if (hipError_t status = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), 160 * 1024, configured)) return status;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), lds, stream, p, units_per_wg);
  return hipGetLastError();
}

// Row quads per workgroup so that one round of workgroups covers the matrix (0: not served).
struct QuadPlan {
  uint32_t rq, waves, grid;
};

// most: row quads a workgroup takes at most (14 = seven waves of two).
QuadPlan quad_plan(uint32_t n, uint32_t most = 14) {
  const uint32_t quads = n / 4;
  const uint32_t cus = (uint32_t)device_compute_units();
  uint32_t per_wg = (quads + cus - 1) / cus;
  QuadPlan plan = {0, 0, 0};
  if (per_wg < 3) return plan;  // too little work per CU
  if (per_wg > most) {
    // several rounds of workgroups, the same number of quads in each
    const uint32_t rounds = (per_wg + most - 1) / most;
    per_wg = (quads + cus * rounds - 1) / (cus * rounds);
  }
  plan.rq = per_wg <= 7 ? 1 : 2;
  plan.waves = (per_wg + plan.rq - 1) / plan.rq;
  plan.grid = (quads + plan.waves * plan.rq - 1) / (plan.waves * plan.rq);
  return plan;
}

// Any K that is a multiple of 512 within the instantiation's KL ranges: the ring depths of the
// benchmark shapes' instantiations, chosen by the row length (six loads in flight for every long row).
// Long rows other than the benchmark's: one quad per wave (a wave that alternates between two quads of
// 8192 values measured 18.7 us at 8192 x 8192 and four rows against 13.2 with twice the workgroups of one
// quad per wave).
uint32_t any_k_most_quads(uint32_t k) { return k > 4096 ? 7 : 14; }

template <int MR, int KL>
hipError_t launch_rows_any_k(const QuadParams &p, hipStream_t stream) {
  const QuadPlan plan = quad_plan(p.n, any_k_most_quads(p.k));
  const bool wide = plan.waves > 4;
  if (plan.rq == 2) {
    if constexpr (MR == 4 && KL > 16) {
      return hipErrorInvalidValue;
    } else {
      if (wide) return launch_instance<MR, KL, 2, 8, 2, 448, false>(p, plan.grid, plan.waves, stream);
      return launch_instance<MR, KL, 2, 8, 2, 256, false>(p, plan.grid, plan.waves, stream);
    }
  }
  if constexpr (KL <= 16) {
    if (p.k <= 4096) {
      if (wide) return launch_instance<MR, KL, 1, 4, 4, 448, false>(p, plan.grid, plan.waves, stream);
      return launch_instance<MR, KL, 1, 4, 4, 256, false>(p, plan.grid, plan.waves, stream);
    }
  }
  if (wide) return launch_instance<MR, KL, 1, 6, 2, 448, false>(p, plan.grid, plan.waves, stream);
  return launch_instance<MR, KL, 1, 6, 2, 256, false>(p, plan.grid, plan.waves, stream);
}

template <int MR, int KL>
hipError_t launch_rows(const QuadParams &p, hipStream_t stream) {
  const QuadPlan plan = quad_plan(p.n);
  // Ring depths as measured on 4096 x 4096, 4096 x 14336 and 14336 x 4096 (every launch on
  // another HBM copy).  Short rows finish in eight loads per wave: four in flight, all of them
  // ahead of the staging (3.9 - 4.7 us for 1 - 4 rows against 4.4 - 5.0 with eight).  Two quads
  // per wave: eight in flight, two early (7.2 / 7.4 / 8.3 us; sixteen in flight 8.5 - 9.2).
  // Long rows: six in flight for one or two activation rows (8.9 / 9.7 us against 9.4 / 9.7 with
  // eight and 10.0 with twelve), twelve for four rows, whose 115 KB of activation take longer to
  // stage (10.8 us against 11.3 with eight).
  constexpr int kLongDepth = MR <= 2 ? 6 : 12;
  if (plan.rq == 1) {
    if constexpr (KL <= 8) {
      if (plan.waves <= 4) return launch_instance<MR, KL, 1, 4, 4, 256>(p, plan.grid, plan.waves, stream);
      return launch_instance<MR, KL, 1, 4, 4, 448>(p, plan.grid, plan.waves, stream);
    } else {
      if (plan.waves <= 4) return launch_instance<MR, KL, 1, kLongDepth, 2, 256>(p, plan.grid, plan.waves, stream);
      return launch_instance<MR, KL, 1, kLongDepth, 2, 448>(p, plan.grid, plan.waves, stream);
    }
  }
  if (plan.waves <= 4) return launch_instance<MR, KL, 2, 8, 2, 256>(p, plan.grid, plan.waves, stream);
  // (four rows of K = 14336 on more than four waves of two quads spill registers: w4a16_gemv_quad_ok
  // sends that shape - N above 8192 at K = 14336 - to the other kernels)
  if constexpr (MR == 4 && KL > 8)
    return hipErrorInvalidValue;
  else
    return launch_instance<MR, KL, 2, 8, 2, 448>(p, plan.grid, plan.waves, stream);
}

template <int KL>
hipError_t launch_k(const QuadParams &p, hipStream_t stream) {
  if (p.m <= 1) return launch_rows<1, KL>(p, stream);
  if (p.m <= 2) return launch_rows<2, KL>(p, stream);
  return launch_rows<4, KL>(p, stream);
}

template <int KL>
hipError_t launch_any_k(const QuadParams &p, hipStream_t stream) {
  return launch_rows_any_k<4, KL>(p, stream);
}

// Rows of up to 8192 values (four rows of more do not fit the LDS block next to their scales; K = 14336
// has its own instantiation).
constexpr uint32_t kAnyK = 16 * 512;

}  // namespace

bool w4a16_gemv_quad_ok(const W4LinearArgs &a) {
  if (a.m == 0 || a.m > 4 || a.y == nullptr || a.y_f32 != nullptr) return false;
  if (a.n % 4 != 0) return false;
  const QuadPlan plan = quad_plan(a.n);
  if (plan.rq == 0) return false;
  if (a.k == 14336) {
    if (a.m > 2 && plan.rq == 2 && plan.waves > 4) return false;  // no instantiation without spills
  } else if (a.k != 4096) {
    // Other K: three and four activation rows only (at one and two the v_dot2 kernel of
    // w4a16_gemv.hip measured faster on every such shape: 9.9 against 18.7 us at 16384 x 4096, 9.1 against
    // 11.7 at 8192 x 8192; at four rows this one wins, 7.4 against 9.7 us at 5120 x 5120, 13.7 against
    // 15.9 at 5120 x 13824).  K ranges of 512 of which the last may be partly there, at least as many as
    // the ring's first requests reach; four scale rows a whole number of 16-byte units.
    if (a.m < 3 || a.k % 128 != 0 || a.k < 2048 || a.k > kAnyK) return false;
    if (quad_plan(a.n, any_k_most_quads(a.k)).rq == 0) return false;
  }
  // 16-byte loads of activation rows, weight row pieces and scale rows
  if (((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w.weight) |
        reinterpret_cast<uintptr_t>(a.w.scale)) & 15) != 0)
    return false;
  return true;
}

hipError_t launch_w4a16_gemv_quad_linear(const W4LinearArgs &a, hipStream_t stream) {
  if (!w4a16_gemv_quad_ok(a)) return hipErrorInvalidValue;
  QuadParams p = {a.x, a.w.weight, a.w.scale, a.y, a.addend, a.has_addend, a.addend_row_stride, a.m, a.n, a.k};
  if (a.k == 4096) return launch_k<8>(p, stream);
  if (a.k == 14336) return launch_k<28>(p, stream);
  return launch_any_k<16>(p, stream);
}

}  // namespace llmopt
