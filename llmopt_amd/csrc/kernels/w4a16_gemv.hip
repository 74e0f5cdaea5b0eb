// W4A16 decode GEMV for gfx950: y[M<=8, N] = x[M, K] . W4[N, K]^T.
//
// HBM-bound: the int4 weight stream (N*K/2 bytes) is read exactly once with
// 128-bit loads, one wave owning R complete weight rows so that each lane's
// 16-byte segment (32 K values, inside a single 64-wide scale group) is part
// of a fully coalesced 1 KiB wave access.  Nibbles are decoded to exact fp16
// integers in registers, multiplied with v_dot2_f32_f16 into fp32 partials,
// scaled per group in fp32 and reduced across the wave with DPP.
//
// Replaces the one-SIMD-group-per-output kernels
// llmopt_w4a16_linear_f16_g64{,_m4,_m8}, llmopt_w4a16_qkv_linear_f16_g64* and
// llmopt_w4a16_dual_swiglu_f16_g64* / llmopt_w4a16_down_add_f16_g64*
// (lib/metal_w4a16_source.ml:8-966) for m <= 8.
#include <algorithm>
#include <cstdlib>
#include <utility>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

template <typename F, int... I>
__device__ __forceinline__ void static_for_each(F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<0>) ... f(integral_constant<N-1>): a loop whose index is a constant in every pass
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_each(f, std::make_integer_sequence<int, (N > 0 ? N : 0)>{});
}

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

struct GemvSegment {
  const uint8_t *w;
  const uint16_t *s;
  uint16_t *y;
  uint32_t n;
};

struct GemvParams {
  const uint16_t *x;
  uint32_t m, k;
  // blockIdx.y selects the matrix (QKV: three of them; DUAL: seg0 = gate, seg1 = up)
  GemvSegment seg0, seg1, seg2;
  const uint16_t *addend;
  uint32_t has_addend;
  uint32_t addend_stride;
  float *y_f32;  // optional float32 copy of seg0's output (same indexing), may be null
  W4Norm norm;   // XREG variants only
};

// M: activation rows held per lane, R: weight rows per wave and tile, U: K
// chunks (2048 K values each) per work item, XLDS: activation staged once per
// workgroup in LDS (pair order), DUAL: rows [0,R/2) are gate rows and [R/2,R)
// the matching up rows; the output is silu(gate)*up.
//
// The grid is persistent: every wave walks row tiles gw, gw + W, gw + 2W, ...
// (gw = global wave index) and, inside a tile, items of U chunks.  The weight
// segments and scales of the next item are loaded into registers before the
// current item is decoded, so HBM latency overlaps the VALU work.
//
// D > 0 (with XLDS): a ring of D items in flight per wave instead of one.  The
// loads are then issued as assembly and waited for by count (vector loads
// return in issue order, so "at most n younger loads outstanding" names the
// ones that have landed); left to the compiler, the wait at the loop head is
// for everything in flight and the ring degenerates to one item.  ADD (ring
// only): the residual addend of a tile travels with its items, so that the
// store path has no load of its own to wait for.
// XREG (ring only, K <= 2048 U): an item covers a whole row, so a lane meets the same U x 32 K
// values in every item and keeps its pieces of the activation in registers - no LDS copy, no
// workgroup barrier before the first row.
template <int M, int R, int U, bool XLDS, bool DUAL, int D = 0, bool ADD = false, bool XREG = false>
__global__ __launch_bounds__(kThreads) void w4a16_gemv_kernel(GemvParams p) {
  static_assert(D == 0 || XLDS, "the ring of loads needs the activation in LDS");
  static_assert(!XREG || D > 0, "the register activation belongs to the ring");
  static_assert(!ADD || (D > 0 && !DUAL), "the addend travels with the ring only");
  extern __shared__ uint4 x_lds[];
  const int lane = threadIdx.x & 63;
  // wave-uniform values are forced into scalar registers: tile indices, row
  // pointers and the matrix selection then cost no vector work
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const GemvSegment sg = blockIdx.y == 0 ? p.seg0 : blockIdx.y == 1 ? p.seg1 : p.seg2;
  const uint32_t tiles = (sg.n + (DUAL ? R / 2 : R) - 1) / (DUAL ? R / 2 : R);
  const uint32_t K = p.k;
  const uint32_t segs = K >> 5;              // 16-byte weight segments per row
  const uint32_t chunks = (segs + 63) >> 6;  // wave-wide steps over K
  const uint32_t items_per_tile = (chunks + U - 1) / U;
  constexpr int C = DUAL ? R / 2 : R;  // output columns per tile

  const uint32_t wave_count = gridDim.x * kWaves;
  const uint32_t first_tile = blockIdx.x * kWaves + wave;

  // Raw loaded registers only: nothing here may be touched before the item is
  // consumed, or the compiler has to wait for the loads right after issuing them.
  struct Item {
    u32x4_t w[R][U];
    uint32_t s[R][U];  // fp16 bits in the low half
    uint32_t addend[ADD ? C : 1][ADD ? M : 1];
  };

  auto tile_rows = [&](uint32_t tile, const u32x4_t *(&wrow)[R], const uint16_t *(&srow)[R]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t col = min(tile * C + (uint32_t)(DUAL ? r % C : r), sg.n - 1);
      const uint8_t *w = DUAL && r >= C ? p.seg1.w : sg.w;
      const uint16_t *sc = DUAL && r >= C ? p.seg1.s : sg.s;
      wrow[r] = reinterpret_cast<const u32x4_t *>(w + (size_t)col * (K >> 1));
      srow[r] = sc + (size_t)col * (K >> 6);
    }
  };

  // `real` = false is the prefetch past the last item: still issued (see the
  // main loop) but every lane reads segment 0 of the rows, one line per row.
  auto load_item = [&](uint32_t tile, uint32_t item, bool real, Item &out) {
    const u32x4_t *wrow[R];
    const uint16_t *srow[R];
    tile_rows(tile, wrow, srow);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t seg = (item * U + u) * 64 + lane;
      const uint32_t safe = (real && seg < segs) ? seg : 0;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        out.w[r][u] = __builtin_nontemporal_load(wrow[r] + safe);
        out.s[r][u] = srow[r][safe >> 1];
      }
    }
  };

  // The same loads for the ring: assembly, so that nothing waits for them but wait_item.
  // Between an issue and its wait_item the set must not be copied (its registers are
  // written when the data lands, not when the statement ends).
  constexpr int LOADS = 2 * R * U + (ADD ? C * M : 0);  // vector loads of one issue_item
  auto issue_item = [&](uint32_t tile, uint32_t item, bool real, Item &out) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
    const u32x4_t *wrow[R];
    const uint16_t *srow[R];
    tile_rows(tile, wrow, srow);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t seg = (item * U + u) * 64 + lane;
      const uint32_t safe = (real && seg < segs) ? seg : 0;
      const uint32_t w_offset = safe * 16, s_offset = (safe >> 1) * 2;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(out.w[r][u]) : "v"(w_offset), "s"(wrow[r]) : "memory");
        asm volatile("global_load_ushort %0, %1, %2" : "=&v"(out.s[r][u]) : "v"(s_offset), "s"(srow[r]) : "memory");
      }
    }
    if (ADD) {
      const uint32_t zero = 0;
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const uint32_t col = min(tile * C + (uint32_t)c, sg.n - 1);
#pragma unroll
        for (int m = 0; m < M; ++m) {
          const uint16_t *src = p.addend + (size_t)((uint32_t)m < p.m ? m : 0) * p.addend_stride + col;
          asm volatile("global_load_ushort %0, %1, %2" : "=&v"(out.addend[ADD ? c : 0][ADD ? m : 0]) : "v"(zero), "s"(src) : "memory");
        }
      }
    }
#endif
  };
  auto wait_item = [&](Item &f, auto younger) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int n = decltype(younger)::value;
    static_assert(n < 64, "vmcnt is a six-bit counter");
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < U; ++u)
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(f.w[r][u]), "+v"(f.s[r][u]) : "n"(n) : "memory");
    if (ADD) {
#pragma unroll
      for (int c = 0; c < C; ++c)
#pragma unroll
        for (int m = 0; m < M; ++m)
          asm volatile("" : "+v"(f.addend[ADD ? c : 0][ADD ? m : 0]));
    }
#endif
  };

  // first weights are in flight while the activation is staged
  Item item_a, item_b;
  Item ring[D > 0 ? D : 1];
  uint32_t ring_tile[D > 0 ? D : 1], ring_item[D > 0 ? D : 1];
  const bool has_work = first_tile < tiles;
  uint32_t ahead_tile = first_tile, ahead_item = 0;  // the next item to request
  auto request = [&](int d) __attribute__((always_inline)) {
    ring_tile[d] = ahead_tile;
    ring_item[d] = ahead_item;
    const bool real = ahead_tile < tiles;
    issue_item(real ? ahead_tile : first_tile, ahead_item, real, ring[d]);
    if (++ahead_item == items_per_tile) {
      ahead_item = 0;
      ahead_tile += wave_count;
    }
  };
  // Ring: the activation is requested first (loads return in order, so it lands before the
  // ring and the staging below does not wait for weights), up to kXAhead vectors per thread.
  constexpr int kXAhead = 8;
  static_assert(kXAhead == 8, "the wait below names eight registers");
  const uint32_t vectors_per_row = chunks * 256;  // includes zero padding
  const uint32_t x_vectors = (uint32_t)M * vectors_per_row;  // a multiple of kThreads
  // The staging below walks x_vectors in steps of kThreads and stores without a bound of its own:
  // only a block size that divides the 256 vectors of a chunk keeps every index inside the LDS
  // block (a 1024-thread block overruns it whenever rows x chunks is not a multiple of four;
  // tests/test_gemv_index_bounds.py enumerates both).
  static_assert(256 % kThreads == 0, "the activation staging needs a block size that divides 256");
  static_assert(kXAhead * kThreads >= 256, "the vectors requested ahead cover at least one chunk of one row");
  constexpr int XA = D > 0 ? kXAhead : 1;
  u32x4_t x_ahead[XA];
  auto x_source = [&](uint32_t i, bool &valid) {
    const uint32_t m = i / vectors_per_row;
    const uint32_t kk = i - m * vectors_per_row;  // index of an 8-K block
    valid = m < p.m && kk < (K >> 3);
    return reinterpret_cast<const uint4 *>(p.x + (size_t)(valid ? m : 0) * K) + (valid ? kk : 0);
  };
  auto x_store = [&](uint32_t i, uint4 value) {
    const uint32_t m = i / vectors_per_row;
    const uint32_t kk = i - m * vectors_per_row;
    const uint32_t seg = kk >> 2, j = kk & 3;
    x_lds[((m * chunks + (seg >> 6)) * 4 + j) * 64 + (seg & 63)] = value;
  };
  // XREG: the lane's own four vectors per chunk of every row; pair order and bias correction as in LDS
  u32x4_t x_own[XREG ? M : 1][XREG ? U : 1][4];
  u32x4_t gain_own[XREG ? U : 1][4];  // the RMS norm weights of the same K values, if any
  uint4 x_held[XREG ? M : 1][XREG ? U : 1][4];
  float correction_held[XREG ? M : 1][XREG ? U : 1];
  if constexpr (XREG) {
    const bool normalise = p.norm.weight != nullptr;  // the same for every wave
#if defined(__HIP_DEVICE_COMPILE__)
    if (normalise) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint16_t *gain = p.norm.weight + min((uint32_t)(u * 64 + lane), segs - 1) * 32;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(gain_own[u][j]) : "v"(gain + j * 8) : "memory");
      }
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t own_segment = min((uint32_t)(u * 64 + lane), segs - 1);
        const uint16_t *row = p.x + (size_t)min((uint32_t)m, p.m - 1) * K + own_segment * 32;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(x_own[m][u][j]) : "v"(row + j * 8) : "memory");
      }
#endif
    static_for<D>([&](auto index) __attribute__((always_inline)) { request(decltype(index)::value); });
#if defined(__HIP_DEVICE_COMPILE__)
    // only the ring's requests may still be outstanding
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(x_own[0][0][0]) : "n"(D * LOADS) : "memory");
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(x_own[m][u][j]));
    if (normalise) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(gain_own[u][j]));
    }
#endif
    if (normalise) {
      // The wave holds whole rows: mean square by a wave reduction, then the half values the
      // separate normalisation kernel would have stored (float32 products in its order).
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float square_sum = 0.0f;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const bool present = (uint32_t)(u * 64 + lane) < segs;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const h8_t x = __builtin_bit_cast(h8_t, x_own[m][u][j]);
#pragma unroll
            for (int e = 0; e < 8; ++e) square_sum += present ? (float)x[e] * (float)x[e] : 0.0f;
          }
        }
        square_sum = wave_sum(square_sum);
        const float inverse = rsqrtf(square_sum / (float)K + p.norm.epsilon);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const h8_t x = __builtin_bit_cast(h8_t, x_own[m][u][j]);
            const h8_t g = __builtin_bit_cast(h8_t, gain_own[u][j]);
            h8_t y;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float value = (float)x[e], gain = (float)g[e];
              y[e] = (_Float16)(p.norm.weight_first ? value * gain * inverse : value * inverse * gain);
            }
            x_own[m][u][j] = __builtin_bit_cast(u32x4_t, y);
          }
      }
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool present = (uint32_t)(u * 64 + lane) < segs && (uint32_t)m < p.m;
        float sum_a = 0.0f, sum_b = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint4 v = pair_order(__builtin_bit_cast(uint4, x_own[m][u][j]));
          x_held[m][u][j] = present ? v : make_uint4(0, 0, 0, 0);
          const h2_t a0 = as_h2(x_held[m][u][j].x), b0 = as_h2(x_held[m][u][j].y);
          const h2_t a1 = as_h2(x_held[m][u][j].z), b1 = as_h2(x_held[m][u][j].w);
          sum_a += ((float)a0[0] + (float)a0[1]) + ((float)a1[0] + (float)a1[1]);
          sum_b += ((float)b0[0] + (float)b0[1]) + ((float)b1[0] + (float)b1[1]);
        }
        correction_held[m][u] = 1032.0f * sum_a + 72.0f * sum_b;
      }
  } else if constexpr (D > 0) {
#if defined(__HIP_DEVICE_COMPILE__)
    static_for<kXAhead>([&](auto index) __attribute__((always_inline)) {
      constexpr int n = decltype(index)::value;
      x_ahead[n] = u32x4_t{0, 0, 0, 0};
      if ((uint32_t)n * kThreads < x_vectors) {  // the same for every thread
        bool valid;
        const uint4 *src = x_source(threadIdx.x + n * kThreads, valid);
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(x_ahead[n]) : "v"(src) : "memory");
      }
    });
#endif
    // also by a wave without work (its requests read a clamped row): the wait below counts on them
    static_for<D>([&](auto index) __attribute__((always_inline)) { request(decltype(index)::value); });
  } else if (has_work) {
    load_item(first_tile, 0, true, item_a);
  }

  // Bias correction of w4_decode_biased per (m, chunk, lane), after the vectors.
  float *corr_lds = reinterpret_cast<float *>(x_lds + (size_t)M * chunks * 256);
  if (XLDS && !XREG) {
    // LDS layout [m][chunk][j][lane] of uint4: the j-th 8-K block of every
    // lane's segment is contiguous across lanes (conflict-free b128 reads).
    uint32_t first_vector = threadIdx.x;
    if constexpr (D > 0) {
#if defined(__HIP_DEVICE_COMPILE__)
      // only the ring's requests may still be outstanding
      asm volatile("s_waitcnt vmcnt(%8)"
                   : "+v"(x_ahead[0]), "+v"(x_ahead[1 % XA]), "+v"(x_ahead[2 % XA]), "+v"(x_ahead[3 % XA]),
                     "+v"(x_ahead[4 % XA]), "+v"(x_ahead[5 % XA]), "+v"(x_ahead[6 % XA]), "+v"(x_ahead[7 % XA])
                   : "n"(D * LOADS)
                   : "memory");
#endif
      static_for<kXAhead>([&](auto index) __attribute__((always_inline)) {
        constexpr int n = decltype(index)::value;
        if ((uint32_t)n * kThreads < x_vectors) {
          bool valid;
          const uint32_t i = threadIdx.x + n * kThreads;
          (void)x_source(i, valid);
          const uint4 loaded = pair_order(__builtin_bit_cast(uint4, x_ahead[n]));
          x_store(i, valid ? loaded : make_uint4(0, 0, 0, 0));
        }
      });
      first_vector += kXAhead * kThreads;  // anything beyond waits for the ring as well
    }
    for (uint32_t i = first_vector; i < x_vectors; i += kThreads) {
      bool valid;
      const uint4 *src = x_source(i, valid);
      x_store(i, valid ? pair_order(*src) : make_uint4(0, 0, 0, 0));
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < (uint32_t)M * chunks * 64; i += kThreads) {
      const uint32_t mc = i >> 6, ln = i & 63;  // mc = m * chunks + chunk
      float sum_a = 0.0f, sum_b = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4 v = x_lds[(mc * 4 + j) * 64 + ln];
        const h2_t a0 = as_h2(v.x), b0 = as_h2(v.y), a1 = as_h2(v.z), b1 = as_h2(v.w);
        sum_a += ((float)a0[0] + (float)a0[1]) + ((float)a1[0] + (float)a1[1]);
        sum_b += ((float)b0[0] + (float)b0[1]) + ((float)b1[0] + (float)b1[1]);
      }
      corr_lds[i] = 1032.0f * sum_a + 72.0f * sum_b;
    }
    __syncthreads();
  }
  if (!has_work) return;

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

  // Decodes one item into acc; when it is the last item of its tile, reduces
  // across the wave and stores.
  auto consume = [&](uint32_t tile, uint32_t item, const Item &cur) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t c = item * U + u;
      const uint32_t seg = c * 64 + lane;
      const bool ok = seg < segs;  // a segment past the row end contributes scale 0
      const uint32_t safe = ok ? seg : 0;
      const uint32_t c_safe = c < chunks ? c : 0;
      float part[R][M];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) part[r][m] = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4 xp[M];
#pragma unroll
        for (int m = 0; m < M; ++m) {
          if (XREG) {
            xp[m] = x_held[XREG ? m : 0][XREG ? u : 0][j];
          } else if (XLDS) {
            xp[m] = x_lds[((m * chunks + c_safe) * 4 + j) * 64 + lane];
          } else {
            const uint32_t row = (uint32_t)m < p.m ? m : 0;
            xp[m] = pair_order(
                reinterpret_cast<const uint4 *>(p.x + (size_t)row * K)[safe * 4 + j]);
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const W4Pairs q = XLDS ? w4_decode_biased(cur.w[r][u][j]) : w4_decode_pairs(cur.w[r][u][j]);
#pragma unroll
          for (int m = 0; m < M; ++m) {
            float a = part[r][m];
            a = __builtin_amdgcn_fdot2(q.p04, as_h2(xp[m].x), a, false);
            a = __builtin_amdgcn_fdot2(q.p15, as_h2(xp[m].y), a, false);
            a = __builtin_amdgcn_fdot2(q.p26, as_h2(xp[m].z), a, false);
            a = __builtin_amdgcn_fdot2(q.p37, as_h2(xp[m].w), a, false);
            part[r][m] = a;
          }
        }
      }
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float correction = XREG   ? correction_held[XREG ? m : 0][XREG ? u : 0]
                                 : XLDS ? corr_lds[(m * chunks + c_safe) * 64 + lane]
                                        : 0.0f;
#pragma unroll
        for (int r = 0; r < R; ++r)
          acc[r][m] = fmaf(part[r][m] - correction, ok ? half_bits_to_float((uint16_t)cur.s[r][u]) : 0.0f,
                           acc[r][m]);
      }
    }

    if (item + 1 == items_per_tile) {
      const uint32_t n = sg.n;
      const uint32_t col0 = tile * C;
      float total[R][M];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) {
          total[r][m] = wave_sum(acc[r][m]);
          acc[r][m] = 0.0f;
        }
      if (lane == 0) {
#pragma unroll
        for (int cidx = 0; cidx < C; ++cidx) {
          const uint32_t col = col0 + cidx;
          if (col >= n) break;
#pragma unroll
          for (int m = 0; m < M; ++m) {
            if ((uint32_t)m >= p.m) break;
            float value;
            if (DUAL) {
              const float gate = total[cidx][m];
              const float up = total[cidx + C][m];
              value = gate / (1.0f + __expf(-gate)) * up;
            } else {
              value = total[cidx][m];
              if (ADD)
                value += half_bits_to_float((uint16_t)cur.addend[ADD ? cidx : 0][ADD ? m : 0]);
              else if (D == 0 && p.has_addend)
                value += half_bits_to_float(p.addend[(size_t)m * p.addend_stride + col]);
            }
            if (sg.y != nullptr) sg.y[(size_t)m * n + col] = float_to_half_bits(value);
            if (!DUAL && p.y_f32 != nullptr) p.y_f32[(size_t)m * n + col] = value;
          }
        }
      }
    }
  };

  auto advance = [&](uint32_t &tile, uint32_t &item) {
    if (++item == items_per_tile) {
      item = 0;
      tile += wave_count;
    }
  };

  // Ping-pong between two register sets: the next item's loads are issued
  // before the current item is decoded.  The prefetch is unconditional (past
  // the end it reads one line per row) so that no branch skips the loads:
  // with a skipped path the compiler must assume the shorter load queue and
  // waits for the fresh loads before decoding the old ones.
  if (D > 0) {
    // ring[d] is consumed while the D - 1 younger requests are in flight, then requested again
    // D items ahead; requests past the last tile are still issued (one line per row, unused)
    // so that the number of loads in flight stays what wait_item assumes.
    bool done = false;
    while (!done) {
      static_for<D>([&](auto index) __attribute__((always_inline)) {
        constexpr int d = decltype(index)::value;
        if (done) return;
        if (ring_tile[d] >= tiles) {
          done = true;
          return;
        }
        wait_item(ring[d], std::integral_constant<int, (D - 1) * LOADS>{});
        consume(ring_tile[d], ring_item[d], ring[d]);
        request(d);
      });
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // requests in flight still target live registers
    return;
  }
  uint32_t tile = first_tile, item = 0;
  while (true) {
    uint32_t next_tile = tile, next_item = item;
    advance(next_tile, next_item);
    bool more = next_tile < tiles;
    load_item(more ? next_tile : tile, next_item, more, item_b);
    consume(tile, item, item_a);
    if (!more) break;
    tile = next_tile;
    item = next_item;
    advance(next_tile, next_item);
    more = next_tile < tiles;
    load_item(more ? next_tile : tile, next_item, more, item_a);
    consume(tile, item, item_b);
    if (!more) break;
    tile = next_tile;
    item = next_item;
  }
}

}  // namespace

int device_compute_units() {
  static int cached = 0;
  if (cached == 0) {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        count <= 0)
      count = 256;
    cached = count;
  }
  return cached;
}

// The register-activation variants (one or two rows, K of at most one 2048-wide chunk) hold
// whole rows per wave and can normalise them.
bool w4a16_gemv_norm_ok(uint32_t m, uint32_t k) { return m <= (uint32_t)kGemvDotRows && k <= 2048 && k % 64 == 0; }

namespace {

template <int M, int R, int U, bool DUAL, int D = 0>
hipError_t launch_variant(const GemvParams &p, uint32_t matrices, uint32_t max_n, hipStream_t stream) {
  // a tile is R weight rows (DUAL: R/2 gate rows + the matching R/2 up rows)
  constexpr int C = DUAL ? R / 2 : R;
  const uint32_t tiles = (max_n + C - 1) / C;  // of the largest matrix

  const uint32_t segs = p.k >> 5;
  const uint32_t chunks = (segs + 63) >> 6;
  // activation vectors (pair order) + one float of bias correction per (m, chunk, lane)
  const size_t lds_bytes = (size_t)M * chunks * 256 * sizeof(uint4) + (size_t)M * chunks * 64 * sizeof(float);
  const bool use_lds = lds_bytes <= 64 * 1024;
  const int cus = device_compute_units();
  // workgroups per CU: 12 waves with two items in flight each for the ring (measured against 8
  // and 16), 8 waves otherwise; fewer when the activation fills the LDS
  int per_cu = D > 0 && use_lds ? 3 : 2;
  while (per_cu > 1 && lds_bytes * per_cu > 150 * 1024) --per_cu;
  const uint32_t wanted = (tiles + kWaves - 1) / kWaves;
  const uint32_t blocks = std::max<uint32_t>(1, std::min<uint32_t>(wanted, (uint32_t)(cus * per_cu)));
  if constexpr (D > 0) {
    if (chunks == (uint32_t)U) {  // an item covers the row: the activation stays in registers, no LDS
      if constexpr (!DUAL) {
        if (p.has_addend) {
          hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, U, true, DUAL, D, true, true>), dim3(blocks, matrices),
                             dim3(kThreads), 0, stream, p);
          return hipGetLastError();
        }
      }
      hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, U, true, DUAL, D, false, true>), dim3(blocks, matrices),
                         dim3(kThreads), 0, stream, p);
      return hipGetLastError();
    }
  }
  if (use_lds && D > 0) {
    if constexpr (!DUAL && D > 0) {
      if (p.has_addend) {
        hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, U, true, DUAL, D, true>), dim3(blocks, matrices),
                           dim3(kThreads), lds_bytes, stream, p);
        return hipGetLastError();
      }
    }
    if constexpr (D > 0)
      hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, U, true, DUAL, D, false>), dim3(blocks, matrices),
                         dim3(kThreads), lds_bytes, stream, p);
  } else if (use_lds) {
    hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, U, true, DUAL>), dim3(blocks, matrices), dim3(kThreads),
                       lds_bytes, stream, p);
  } else {
    hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, U, false, DUAL>), dim3(blocks, matrices), dim3(kThreads), 0,
                       stream, p);
  }
  return hipGetLastError();
}

template <bool DUAL>
hipError_t launch_by_rows(const GemvParams &p, uint32_t matrices, uint32_t max_n, hipStream_t stream) {
  // small work items (2 rows x one 2048-wide K chunk) measured fastest: finer
  // interleaving of waves over the row tiles and a shorter drain at the end
  // one and two rows: two items in flight per wave (deeper rings measured slower)
  // long rows at one activation row: single-row items, three in flight (8.8 against 9.1 us at 14336 x 4096)
  if constexpr (!DUAL) {
    if (p.m <= 1 && p.k >= 8192) return launch_variant<1, 1, 1, DUAL, 3>(p, matrices, max_n, stream);
  }
  if (p.m <= 1) return launch_variant<1, 2, 1, DUAL, 2>(p, matrices, max_n, stream);
  if (p.m <= 2) return launch_variant<2, 2, 1, DUAL, 2>(p, matrices, max_n, stream);
  if (p.m <= 4) return launch_variant<4, 2, 1, DUAL>(p, matrices, max_n, stream);
  return launch_variant<8, 2, 1, DUAL>(p, matrices, max_n, stream);
}

}  // namespace

hipError_t launch_w4a16_gemv_linear(const W4LinearArgs &a, hipStream_t stream) {
  GemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.seg0 = {a.w.weight, a.w.scale, a.y, a.n};
  p.addend = a.addend;
  p.has_addend = a.has_addend;
  p.addend_stride = a.addend_row_stride;
  p.y_f32 = a.y_f32;
  return launch_by_rows<false>(p, 1, a.n, stream);
}

hipError_t launch_w4a16_gemv_qkv(const W4QkvArgs &a, hipStream_t stream) {
  GemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.seg0 = {a.w[0].weight, a.w[0].scale, a.y[0], a.n[0]};
  p.seg1 = {a.w[1].weight, a.w[1].scale, a.y[1], a.n[1]};
  p.seg2 = {a.w[2].weight, a.w[2].scale, a.y[2], a.n[2]};
  p.norm = a.norm;
  if (p.norm.weight != nullptr && !w4a16_gemv_norm_ok(a.m, a.k)) return hipErrorInvalidValue;
  return launch_by_rows<false>(p, 3, std::max(a.n[0], std::max(a.n[1], a.n[2])), stream);
}

hipError_t launch_w4a16_gemv_dual_swiglu(const W4DualSwigluArgs &a, hipStream_t stream) {
  GemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.seg0 = {a.gate.weight, a.gate.scale, a.product, a.n};
  p.seg1 = {a.up.weight, a.up.scale, a.product, a.n};
  p.norm = a.norm;
  if (p.norm.weight != nullptr && !w4a16_gemv_norm_ok(a.m, a.k)) return hipErrorInvalidValue;
  return launch_by_rows<true>(p, 1, a.n, stream);
}

}  // namespace llmopt
