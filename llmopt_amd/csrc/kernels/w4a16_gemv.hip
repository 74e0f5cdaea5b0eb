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

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

struct GemvSegment {
  const uint8_t *w;
  const uint16_t *s;
  uint16_t *y;
  uint32_t n;
  uint32_t tile_begin;  // first tile index of this matrix
};

struct GemvParams {
  const uint16_t *x;
  uint32_t m, k;
  GemvSegment seg[3];
  uint32_t nseg;
  uint32_t tiles;
  const uint16_t *addend;
  uint32_t has_addend;
  uint32_t addend_stride;
};

// M: activation rows held per lane, R: weight rows per wave, XLDS: activation
// staged once per workgroup in LDS (pair order), DUAL: rows [0,R/2) are gate
// rows and [R/2,R) the matching up rows; the output is silu(gate)*up.
template <int M, int R, bool XLDS, bool DUAL>
__global__ __launch_bounds__(kThreads) void w4a16_gemv_kernel(GemvParams p) {
  extern __shared__ uint4 x_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const uint32_t K = p.k;
  const uint32_t segs = K >> 5;             // 16-byte weight segments per row
  const uint32_t chunks = (segs + 63) >> 6;  // wave-wide steps over K
  constexpr int C = DUAL ? R / 2 : R;        // output columns per wave

  if (XLDS) {
    // LDS layout [m][chunk][j][lane] of uint4: the j-th 8-K block of every
    // lane's segment is contiguous across lanes (conflict-free b128 reads).
    const uint32_t vectors_per_row = chunks * 256;  // includes zero padding
    for (uint32_t i = threadIdx.x; i < (uint32_t)M * vectors_per_row; i += kThreads) {
      const uint32_t m = i / vectors_per_row;
      const uint32_t kk = i - m * vectors_per_row;  // index of an 8-K block
      uint4 value = make_uint4(0, 0, 0, 0);
      if (m < p.m && kk < (K >> 3))
        value = pair_order(reinterpret_cast<const uint4 *>(p.x + (size_t)m * K)[kk]);
      const uint32_t seg = kk >> 2, j = kk & 3;
      x_lds[((m * chunks + (seg >> 6)) * 4 + j) * 64 + (seg & 63)] = value;
    }
    __syncthreads();
  }

  for (uint32_t tile = blockIdx.x; tile < p.tiles; tile += gridDim.x) {
    uint32_t which = 0;
    if (!DUAL) {
      if (p.nseg > 1 && tile >= p.seg[1].tile_begin) which = 1;
      if (p.nseg > 2 && tile >= p.seg[2].tile_begin) which = 2;
    }
    const GemvSegment &sg = p.seg[which];
    const uint32_t n = sg.n;
    const uint32_t col0 = (tile - sg.tile_begin) * (kWaves * C) + wave * C;
    if (col0 >= n) continue;  // whole wave idle (wave-uniform)

    const u32x4_t *wrow[R];
    const uint16_t *srow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t col = min(col0 + (uint32_t)(DUAL ? r % C : r), n - 1);
      const GemvSegment &src = DUAL ? p.seg[r / C] : sg;
      wrow[r] = reinterpret_cast<const u32x4_t *>(src.w + (size_t)col * (K >> 1));
      srow[r] = src.s + (size_t)col * (K >> 6);
    }

    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

    u32x4_t w_cur[R];
    float s_cur[R];
    auto load_chunk = [&](uint32_t c, u32x4_t(&wv)[R], float(&sv)[R]) {
      const uint32_t seg = c * 64 + lane;
      const bool ok = seg < segs;
      const uint32_t safe = ok ? seg : 0;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        wv[r] = __builtin_nontemporal_load(wrow[r] + safe);
        sv[r] = half_bits_to_float(srow[r][safe >> 1]);
        if (!ok) {
          wv[r] = u32x4_t{0, 0, 0, 0};  // q = 0
          sv[r] = 0.0f;
        }
      }
    };
    load_chunk(0, w_cur, s_cur);

    for (uint32_t c = 0; c < chunks; ++c) {
      u32x4_t w_next[R];
      float s_next[R];
      if (c + 1 < chunks) load_chunk(c + 1, w_next, s_next);

      const uint32_t seg = c * 64 + lane;
      const uint32_t safe = seg < segs ? seg : 0;
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
          if (XLDS) {
            xp[m] = x_lds[((m * chunks + c) * 4 + j) * 64 + lane];
          } else {
            const uint32_t row = (uint32_t)m < p.m ? m : 0;
            xp[m] = pair_order(
                reinterpret_cast<const uint4 *>(p.x + (size_t)row * K)[safe * 4 + j]);
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint32_t word = w_cur[r][j];
          const W4Pairs q = w4_decode_pairs(word);
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
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = fmaf(part[r][m], s_cur[r], acc[r][m]);

      if (c + 1 < chunks) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          w_cur[r] = w_next[r];
          s_cur[r] = s_next[r];
        }
      }
    }

    // wave reduction; the result is uniform, lane 0 stores
    float total[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) total[r][m] = wave_sum(acc[r][m]);

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
            if (p.has_addend)
              value += half_bits_to_float(p.addend[(size_t)m * p.addend_stride + col]);
          }
          sg.y[(size_t)m * n + col] = float_to_half_bits(value);
        }
      }
    }
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

namespace {

template <int M, int R, bool DUAL>
hipError_t launch_variant(const GemvParams &p, hipStream_t stream) {
  const uint32_t segs = p.k >> 5;
  const uint32_t chunks = (segs + 63) >> 6;
  const size_t lds_bytes = (size_t)M * chunks * 256 * sizeof(uint4);
  const bool use_lds = lds_bytes <= 64 * 1024;
  const int cus = device_compute_units();
  int per_cu = 4;
  if (use_lds && lds_bytes > 0)
    per_cu = (int)std::min<size_t>(4, std::max<size_t>(1, (size_t)(160 * 1024) / lds_bytes));
  const uint32_t blocks = std::min<uint32_t>(p.tiles, (uint32_t)(cus * per_cu));
  if (use_lds) {
    hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, true, DUAL>), dim3(blocks), dim3(kThreads),
                       lds_bytes, stream, p);
  } else {
    hipLaunchKernelGGL((w4a16_gemv_kernel<M, R, false, DUAL>), dim3(blocks), dim3(kThreads), 0,
                       stream, p);
  }
  return hipGetLastError();
}

template <bool DUAL>
hipError_t launch_by_rows(GemvParams &p, hipStream_t stream) {
  // tiles depend on the columns a workgroup covers: kWaves * C
  auto finish = [&](int columns_per_wave) {
    uint32_t tiles = 0;
    const uint32_t per_tile = kWaves * columns_per_wave;
    const uint32_t count = DUAL ? 1 : p.nseg;
    for (uint32_t i = 0; i < count; ++i) {
      p.seg[i].tile_begin = tiles;
      tiles += (p.seg[i].n + per_tile - 1) / per_tile;
    }
    if (DUAL) p.seg[1].tile_begin = 0;
    p.tiles = tiles;
  };
  if (p.m <= 1) {
    finish(DUAL ? 2 : 4);
    return launch_variant<1, 4, DUAL>(p, stream);
  }
  if (p.m <= 2) {
    finish(DUAL ? 2 : 4);
    return launch_variant<2, 4, DUAL>(p, stream);
  }
  if (p.m <= 4) {
    finish(DUAL ? 1 : 2);
    return launch_variant<4, 2, DUAL>(p, stream);
  }
  finish(DUAL ? 1 : 2);
  return launch_variant<8, 2, DUAL>(p, stream);
}

__global__ void w4_dequant_f32_kernel(const uint8_t *weight, const uint16_t *scale, float *out,
                                      uint32_t n, uint32_t k) {
  // one thread per packed byte
  const size_t index = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t bytes_per_row = k >> 1;
  if (index >= (size_t)n * bytes_per_row) return;
  const size_t row = index / bytes_per_row;
  const size_t byte_in_row = index - row * bytes_per_row;
  const uint32_t byte = weight[index];
  const int low = (int)(byte & 15u) - ((byte & 8u) ? 16 : 0);
  const int high = (int)(byte >> 4) - ((byte & 128u) ? 16 : 0);
  const float s = half_bits_to_float(scale[row * (k >> 6) + (byte_in_row >> 5)]);
  out[row * k + 2 * byte_in_row] = (float)low * s;
  out[row * k + 2 * byte_in_row + 1] = (float)high * s;
}

}  // namespace

hipError_t launch_w4a16_gemv_linear(const W4LinearArgs &a, hipStream_t stream) {
  GemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.seg[0] = {a.w.weight, a.w.scale, a.y, a.n, 0};
  p.nseg = 1;
  p.addend = a.addend;
  p.has_addend = a.has_addend;
  p.addend_stride = a.addend_row_stride;
  return launch_by_rows<false>(p, stream);
}

hipError_t launch_w4a16_gemv_qkv(const W4QkvArgs &a, hipStream_t stream) {
  GemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  for (int i = 0; i < 3; ++i) p.seg[i] = {a.w[i].weight, a.w[i].scale, a.y[i], a.n[i], 0};
  p.nseg = 3;
  return launch_by_rows<false>(p, stream);
}

hipError_t launch_w4a16_gemv_dual_swiglu(const W4DualSwigluArgs &a, hipStream_t stream) {
  GemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.seg[0] = {a.gate.weight, a.gate.scale, a.product, a.n, 0};
  p.seg[1] = {a.up.weight, a.up.scale, a.product, a.n, 0};
  p.nseg = 2;
  return launch_by_rows<true>(p, stream);
}

hipError_t launch_w4_dequant_f32(const W4Matrix &w, float *out, uint32_t n, uint32_t k,
                                 hipStream_t stream) {
  const size_t total = (size_t)n * (k >> 1);
  const uint32_t blocks = (uint32_t)((total + 255) / 256);
  hipLaunchKernelGGL(w4_dequant_f32_kernel, dim3(blocks), dim3(256), 0, stream, w.weight, w.scale,
                     out, n, k);
  return hipGetLastError();
}

}  // namespace llmopt
