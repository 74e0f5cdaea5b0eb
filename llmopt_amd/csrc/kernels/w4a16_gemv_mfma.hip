// W4A16 decode GEMV for 5 <= M <= 8 activation rows on gfx950, using the matrix
// cores for the contraction.
//
// With more than four activation rows the v_dot2 path of w4a16_gemv.hip becomes VALU
// bound (4 dot instructions per row per weight dword).  Here one
// v_mfma_f32_32x32x16_f16 contracts four independent 8(m) x 8(n) x 16(k)
// blocks at once: matrix columns 8q..8q+7 are 8 weight rows in scale group
// g0 + q (q = 0..3) and the activation occupies A rows 8q..8q+7 with the K
// values of that same group; the off-diagonal blocks are not used.  Every lane
// therefore loads one 16-byte weight segment that lies inside a single 64-wide
// scale group (so the fp16 group scale is one scalar per lane, applied in fp32
// to the accumulator), and each wave-wide load covers 8 rows x 128 contiguous
// bytes; a wave takes two adjacent steps, i.e. 256 contiguous bytes per row.
//
// A workgroup of 4 waves owns one 8-row tile; the waves split the K steps
// (256 K values each) and are reduced through LDS at the end.  The activation
// is staged through LDS in chunks of 2048 K values in the operand order of the
// nibble decode.
//
// Same arithmetic contract as llmopt_w4a16_linear_f16_g64_m4 / _m8,
// llmopt_w4a16_qkv_linear_f16_g64_m4, llmopt_w4a16_dual_swiglu_f16_g64_m4 and
// llmopt_w4a16_down_add_f16_g64_m4 (lib/metal_w4a16_source.ml:42-966).
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int MP = 8;                 // activation rows held (padded)
constexpr int TN = 8;                 // weight rows per workgroup tile
constexpr int KC = 2048;              // K values staged per chunk
constexpr int kStepsPerChunk = KC / 256;
constexpr int kStepsPerWave = kStepsPerChunk / kWaves;  // 2: one per ping-pong buffer
static_assert(kStepsPerWave == 2, "the ping-pong below assumes two steps per wave and chunk");

struct MfmaMatrix {
  const uint8_t *w;
  const uint16_t *s;
  uint16_t *y;
  uint32_t n;
};

struct MfmaGemvParams {
  const uint16_t *x;
  uint32_t m, k;
  MfmaMatrix mat0, mat1, mat2;  // blockIdx.y selects (DUAL: mat0 = gate, mat1 = up)
  const uint16_t *addend;
  uint32_t has_addend;
  uint32_t addend_stride;
};

template <bool DUAL>
__global__ __launch_bounds__(kThreads) void w4a16_gemv_mfma_kernel(MfmaGemvParams p) {
  constexpr int NW = DUAL ? 2 : 1;
  extern __shared__ uint4 lds[];
  uint4 *x_lds = lds;                                                    // KC * MP / 8 vectors
  float *red_lds = reinterpret_cast<float *>(lds + (size_t)KC * MP / 8);  // [NW][waves][MP][TN]

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t c = lane & 31;   // matrix column: weight row r of group quarter q
  const uint32_t kq = lane >> 5;  // which 8-wide K block of an MFMA this lane holds
  const uint32_t q = c >> 3;      // scale group within the step
  const uint32_t r = c & 7;       // weight row within the tile / activation row
  const MfmaMatrix mat = DUAL ? p.mat0 : (blockIdx.y == 0 ? p.mat0 : blockIdx.y == 1 ? p.mat1 : p.mat2);
  const uint32_t K = p.k;
  const uint32_t groups = K >> 6;
  const uint32_t steps = (groups + 3) >> 2;
  const uint32_t chunks = (K + KC - 1) / KC;
  const uint32_t n0 = blockIdx.x * TN;
  if (n0 >= mat.n) return;  // a shorter matrix of a QKV launch (whole workgroup)
  const uint32_t row = min(n0 + r, mat.n - 1);

  const uint8_t *wrow[NW];
  const uint16_t *srow[NW];
  wrow[0] = mat.w + (size_t)row * (K >> 1);
  srow[0] = mat.s + (size_t)row * groups;
  if (DUAL) {
    wrow[NW - 1] = p.mat1.w + (size_t)row * (K >> 1);
    srow[NW - 1] = p.mat1.s + (size_t)row * groups;
  }

  struct Item {  // raw loaded registers only (see w4a16_gemv.hip)
    u32x4_t w[NW];
    uint16_t s[NW];
  };
  auto load_step = [&](uint32_t step, Item &out) __attribute__((always_inline)) {
    const uint32_t g = min(step * 4 + q, groups - 1);
#pragma unroll
    for (int v = 0; v < NW; ++v) {
      out.w[v] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4_t *>(wrow[v] + (size_t)g * 32 + kq * 16));
      out.s[v] = srow[v][g];
    }
  };

  // The useful block of a lane's tile is registers 4q..4q+3 (rows 8q + kq*4 + i);
  // all 16 are accumulated and the block is picked at the end.
  f16x_t acc[NW];
#pragma unroll
  for (int v = 0; v < NW; ++v)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[v][i] = 0.0f;

  auto consume = [&](uint32_t step, uint32_t chunk, const Item &cur) __attribute__((always_inline)) {
    const uint32_t g = step * 4 + q;
    const bool ok = g < groups;
    const uint32_t g_local = min(g, groups - 1) - chunk * (KC / 64);
    h8_t a_frag[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      a_frag[j] = __builtin_bit_cast(h8_t, x_lds[((g_local * 4 + j) * 2 + kq) * MP + r]);
#pragma unroll
    for (int v = 0; v < NW; ++v) {
      f16x_t tile;
#pragma unroll
      for (int i = 0; i < 16; ++i) tile[i] = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const W4Pairs w = w4_decode_pairs(cur.w[v][j]);
        uint4 packed;
        packed.x = as_u32(w.p04);
        packed.y = as_u32(w.p15);
        packed.z = as_u32(w.p26);
        packed.w = as_u32(w.p37);
        tile = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_frag[j], __builtin_bit_cast(h8_t, packed), tile, 0, 0, 0);
      }
      const float scale = ok ? half_bits_to_float(cur.s[v]) : 0.0f;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[v][i] = fmaf(tile[i], scale, acc[v][i]);
    }
  };

  // this wave's steps in chunk ch are ch*8 + 2*wave and the next one
  Item item_a, item_b;
  load_step(min(2 * wave, steps - 1), item_a);
  for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
    // stage x[:, chunk*KC .. +KC) in operand order: vector index
    // ((g_local*4 + j)*2 + kq)*MP + m holds K block g*64 + kq*32 + j*8 of row m
    for (uint32_t i = threadIdx.x; i < (uint32_t)MP * (KC / 8); i += kThreads) {
      const uint32_t m = i / (KC / 8);
      const uint32_t kk = i - m * (KC / 8);
      const uint32_t k0 = chunk * KC + kk * 8;
      uint4 value = make_uint4(0, 0, 0, 0);
      if (m < p.m && k0 < K)
        value = pair_order(*reinterpret_cast<const uint4 *>(p.x + (size_t)m * K + k0));
      x_lds[(((kk >> 3) * 4 + (kk & 3)) * 2 + ((kk >> 2) & 1)) * MP + m] = value;
    }
    __syncthreads();
    const uint32_t step_a = chunk * kStepsPerChunk + 2 * wave;
    const uint32_t step_b = step_a + 1;
    const uint32_t step_c = step_a + kStepsPerChunk;  // first step of the next chunk
    load_step(min(step_b, steps - 1), item_b);
    if (step_a < steps) consume(step_a, chunk, item_a);
    load_step(min(step_c, steps - 1), item_a);
    if (step_b < steps) consume(step_b, chunk, item_b);
    __syncthreads();  // every wave is done with this chunk of x
  }

  // pick the lane's block, add the four group quarters of each weight row
  // (8, 16 and 24 lanes apart), then reduce the waves through LDS
#pragma unroll
  for (int v = 0; v < NW; ++v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mine = q == 0 ? acc[v][i] : q == 1 ? acc[v][4 + i] : q == 2 ? acc[v][8 + i] : acc[v][12 + i];
      mine += __builtin_bit_cast(
          float, __builtin_amdgcn_ds_bpermute((int)((lane ^ 8) << 2), __builtin_bit_cast(int, mine)));
      mine += __builtin_bit_cast(
          float, __builtin_amdgcn_ds_bpermute((int)((lane ^ 16) << 2), __builtin_bit_cast(int, mine)));
      if (q == 0) red_lds[((v * kWaves + wave) * MP + kq * 4 + i) * TN + r] = mine;
    }
  }
  __syncthreads();
  if (threadIdx.x < MP * TN) {
    const uint32_t m = threadIdx.x / TN, col_in_tile = threadIdx.x % TN;
    const uint32_t col = n0 + col_in_tile;
    if (m < p.m && col < mat.n) {
      float total[NW];
#pragma unroll
      for (int v = 0; v < NW; ++v) {
        total[v] = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total[v] += red_lds[((v * kWaves + w) * MP + m) * TN + col_in_tile];
      }
      float value;
      if (DUAL) {
        value = total[0] / (1.0f + __expf(-total[0])) * total[NW - 1];
      } else {
        value = total[0];
        if (p.has_addend) value += half_bits_to_float(p.addend[(size_t)m * p.addend_stride + col]);
      }
      mat.y[(size_t)m * mat.n + col] = float_to_half_bits(value);
    }
  }
}

template <bool DUAL>
hipError_t launch(const MfmaGemvParams &p, uint32_t matrices, uint32_t max_n, hipStream_t stream) {
  constexpr int NW = DUAL ? 2 : 1;
  const size_t lds_bytes = (size_t)KC * MP * 2 + (size_t)NW * kWaves * MP * TN * sizeof(float);
  const dim3 grid((max_n + TN - 1) / TN, matrices);
  hipLaunchKernelGGL((w4a16_gemv_mfma_kernel<DUAL>), grid, dim3(kThreads), lds_bytes, stream, p);
  return hipGetLastError();
}

}  // namespace

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
  return launch<false>(p, 1, a.n, stream);
}

hipError_t launch_w4a16_gemv_mfma_qkv(const W4QkvArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.w[0].weight, a.w[0].scale, a.y[0], a.n[0]};
  p.mat1 = {a.w[1].weight, a.w[1].scale, a.y[1], a.n[1]};
  p.mat2 = {a.w[2].weight, a.w[2].scale, a.y[2], a.n[2]};
  return launch<false>(p, 3, std::max(a.n[0], std::max(a.n[1], a.n[2])), stream);
}

hipError_t launch_w4a16_gemv_mfma_dual_swiglu(const W4DualSwigluArgs &a, hipStream_t stream) {
  MfmaGemvParams p = {};
  p.x = a.x;
  p.m = a.m;
  p.k = a.k;
  p.mat0 = {a.gate.weight, a.gate.scale, a.product, a.n};
  p.mat1 = {a.up.weight, a.up.scale, a.product, a.n};
  p.mat2 = p.mat0;
  return launch<true>(p, 1, a.n, stream);
}

}  // namespace llmopt
