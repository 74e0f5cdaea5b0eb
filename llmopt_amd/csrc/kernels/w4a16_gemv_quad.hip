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
// K is a template parameter (KL ranges of 512): strides in LDS, the ring indices and the loop
// are compile-time.  Instantiated for K = 4096 and K = 14336; other shapes keep the kernels of
// w4a16_gemv.hip / w4a16_gemv_mfma.hip.
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
  uint32_t m, n;
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

// MR: activation rows staged (m <= MR <= 4); KL: K / 512; RQ: row quads per wave; DEPTH: weight
// loads in flight per wave; EARLY: how many of them go out before the staging waits;
// THREADS: workgroup size (waves beyond units_per_wg only help staging).
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

template <int MR, int KL, int RQ, int DEPTH, int EARLY, int THREADS>
__global__ __launch_bounds__(THREADS)
    __attribute__((amdgpu_waves_per_eu(quad_waves_per_simd<MR, KL, RQ>(), quad_waves_per_simd<MR, KL, RQ>()))) void
    w4a16_gemv_quad_kernel(QuadParams p, uint32_t units_per_wg) {
  static_assert(MR >= 1 && MR <= 4 && EARLY >= 1 && EARLY <= DEPTH && DEPTH <= KL * RQ && THREADS % 64 == 0, "shape");
  constexpr uint32_t K = KL * 512, row_bytes = K / 2, groups = K / 64;
  constexpr uint32_t kRowStride = 2 * K + 16;         // bytes between activation rows in LDS
  constexpr uint32_t kScaleStride = groups * 2 + 16;  // bytes between scale rows in LDS
  constexpr uint32_t kXUnits = MR * (K / 8);          // 16-byte units of activation to stage
  constexpr int XPER = (kXUnits + THREADS - 1) / THREADS;
  constexpr uint32_t kScaleUnitsPerRow = groups * 2 / 16;
  constexpr int SPER = ((THREADS / 64) * RQ * 4 * kScaleUnitsPerRow + THREADS - 1) / THREADS;
  constexpr int TOTAL = KL * RQ;
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
  constexpr bool kWholePasses = (K / 8) % THREADS == 0;
  constexpr uint32_t kPassesPerRow = kWholePasses ? (K / 8) / THREADS : 1;
  auto unit_of = [&](int e, uint32_t &row, uint32_t &u, bool &inside) __attribute__((always_inline)) {
    if constexpr (kWholePasses) {
      row = (uint32_t)e / kPassesPerRow;
      u = threadIdx.x + ((uint32_t)e % kPassesPerRow) * THREADS;
      inside = true;
    } else {
      const uint32_t idx = threadIdx.x + e * THREADS;
      inside = idx < kXUnits;
      row = min(idx, kXUnits - 1) / (K / 8);
      u = min(idx, kXUnits - 1) % (K / 8);
    }
  };
  uint4 xin[XPER];
#pragma unroll
  for (int e = 0; e < XPER; ++e) {
    uint32_t row, u;
    bool inside;
    unit_of(e, row, u, inside);
    xin[e] = reinterpret_cast<const uint4 *>(p.x + (size_t)min(row, p.m - 1) * K)[u];
  }
  const uint32_t scale_units = rows_per_wg * kScaleUnitsPerRow;
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
  const uint8_t *w_quad[RQ];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) {
    const uint32_t quad = __builtin_amdgcn_readfirstlane(min(unit * RQ + rq, quads - 1));
    w_quad[rq] = p.w + (size_t)quad * 4 * row_bytes;
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int n = 0; n < EARLY; ++n)
    wreg[n] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(w_quad[n % RQ] + (n / RQ) * 256 + w_lane));
  __builtin_amdgcn_sched_barrier(0);
  if (EARLY < DEPTH) {
    // loads return in issue order: with only the early weights outstanding, the activation and
    // the scales have landed
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(EARLY) : "memory");
#pragma unroll
    for (int n = EARLY; n < DEPTH; ++n)
      wreg[n] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(w_quad[n % RQ] + (n / RQ) * 256 + w_lane));
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
    if (row >= p.m) v = make_uint4(0, 0, 0, 0);
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
    if (idx < scale_units)
      *reinterpret_cast<uint4 *>(ss + (idx / kScaleUnitsPerRow) * kScaleStride + (idx % kScaleUnitsPerRow) * 16) = value;
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
  uint16_t addend_bits[RQ][MR] = {};
  const unsigned char *my_scales = ss + (wave * RQ * 4 + j) * kScaleStride + (b >> 1) * 2;
#pragma unroll
  for (int n = 0; n < TOTAL; ++n) {
    const int kp = n / RQ, rq = n % RQ;
    if (rq == 0) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        xa[t] = make_uint4(0, 0, 0, 0);
        if (j < MR) xa[t] = *reinterpret_cast<const uint4 *>(xs + j * kRowStride + (kp * 64 + 4 * b + t) * 16);
      }
      cinit = *reinterpret_cast<const f4_t *>(cin + (kp * 16 + b) * 4);
    }
    const uint16_t scale_bits = *reinterpret_cast<const uint16_t *>(my_scales + rq * 4 * kScaleStride + kp * 16);
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

template <int MR, int KL, int RQ, int DEPTH, int EARLY, int THREADS>
hipError_t launch_instance(const QuadParams &p, uint32_t grid, uint32_t units_per_wg, hipStream_t stream) {
  const size_t lds = quad_lds_bytes<MR, KL, RQ>(units_per_wg);
  auto kernel = &w4a16_gemv_quad_kernel<MR, KL, RQ, DEPTH, EARLY, THREADS>;
  static bool configured = false;  // once per process: the kernel may use more than the default 64 KB of LDS
  if (!configured) {
    const hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (status != hipSuccess) return status;
    configured = true;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), lds, stream, p, units_per_wg);
  return hipGetLastError();
}

// Row quads per workgroup so that one round of workgroups covers the matrix (0: not served).
struct QuadPlan {
  uint32_t rq, waves, grid;
};

QuadPlan quad_plan(uint32_t n) {
  const uint32_t quads = n / 4;
  const uint32_t cus = (uint32_t)device_compute_units();
  const uint32_t per_wg = (quads + cus - 1) / cus;
  QuadPlan plan = {0, 0, 0};
  if (per_wg < 3 || per_wg > 14) return plan;  // too little work per CU, or more than seven waves of two quads
  plan.rq = per_wg <= 7 ? 1 : 2;
  plan.waves = (per_wg + plan.rq - 1) / plan.rq;
  plan.grid = (quads + plan.waves * plan.rq - 1) / (plan.waves * plan.rq);
  return plan;
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

}  // namespace

bool w4a16_gemv_quad_ok(const W4LinearArgs &a) {
  if (a.m == 0 || a.m > 4 || a.y == nullptr || a.y_f32 != nullptr) return false;
  if (a.k != 4096 && a.k != 14336) return false;
  if (a.n % 4 != 0) return false;
  const QuadPlan plan = quad_plan(a.n);
  if (plan.rq == 0) return false;
  if (a.k == 14336 && a.m > 2 && plan.rq == 2 && plan.waves > 4) return false;  // no instantiation without spills
  // 16-byte loads of activation rows, weight row pieces and scale rows
  if (((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w.weight) |
        reinterpret_cast<uintptr_t>(a.w.scale)) & 15) != 0)
    return false;
  return true;
}

hipError_t launch_w4a16_gemv_quad_linear(const W4LinearArgs &a, hipStream_t stream) {
  if (!w4a16_gemv_quad_ok(a)) return hipErrorInvalidValue;
  QuadParams p = {a.x, a.w.weight, a.w.scale, a.y, a.addend, a.has_addend, a.addend_row_stride, a.m, a.n};
  if (a.k == 4096) return launch_k<8>(p, stream);
  return launch_k<28>(p, stream);
}

}  // namespace llmopt
