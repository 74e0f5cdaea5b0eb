// W4A16 prefill GEMM for gfx950: y[M, N] = x[M, K] . W4[N, K]^T with fp16 MFMA
// and fp32 accumulation.
//
// The reference has no matrix-core W4A16 kernel: it runs the GEMV kernel
// llmopt_w4a16_linear_f16_g64_m4 for every m >= 2
// (lib/metal_dispatch_linear.ml:975-982).  Same arithmetic contract here
// (lib/metal_w4a16_source.ml:42-122), different machine mapping:
//
//  * int4 nibbles are decoded to *exact* fp16 integers and staged in LDS; the
//    fp16 group scale is never folded into the fp16 operand.  Each 64-wide K
//    group is contracted by v_mfma_f32_32x32x16_f16 into a temporary fp32 tile
//    which is then scaled by float(scale[n, g]) and added to the running fp32
//    tile, so q*s is applied in fp32 exactly as `float(q) * s` in the reference.
//  * The activation tile is the MFMA A operand (rows = m) and the weight tile
//    the B operand (columns = n), so every lane's 16 accumulator values belong
//    to one output column and the group scale is one scalar per lane.
//  * K order inside an aligned block of 8 is permuted identically for both
//    operands (see w4_decode_pairs / pair_order), which costs nothing in a dot
//    product and keeps the nibble decode at 9 VALU ops per 8 weights.
#include <algorithm>

#include "kernels.h"
#include "kernels_internal.h"
#include "w4_common.h"

namespace llmopt {
namespace {

constexpr int BK = 64;              // one scale group per K step
constexpr int LDS_STRIDE = BK + 8;  // halfs; 144-byte rows keep b128 reads conflict-free
constexpr int kWaves = 8;           // 4 (m) x 2 (n) waves, two per SIMD
constexpr int kThreads = kWaves * 64;

struct GemmParams {
  const uint16_t *x;
  const uint8_t *w[2];  // [1] = up matrix for the dual (SwiGLU) variant
  const uint16_t *s[2];
  const uint16_t *addend;
  uint32_t has_addend;
  uint32_t addend_stride;
  uint16_t *y;
  uint32_t m, n, k;
  uint32_t tiles_m, tiles_n;
};

__device__ __forceinline__ f16x_t zero_tile() {
  f16x_t z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.0f;
  return z;
}

// Each wave owns WM x WN MFMA tiles of 32 x 32 outputs; the workgroup tile is
// (4 * WM * 32) x (2 * WN * 32).  DUAL computes gate and up tiles of the same
// outputs and stores silu(gate) * up.
template <int WM, int WN, bool DUAL>
__global__ __launch_bounds__(kThreads) void w4a16_gemm_kernel(GemmParams p) {
  constexpr int NW = DUAL ? 2 : 1;  // weight matrices per tile
  constexpr int BM = 4 * WM * 32;
  constexpr int BN = 2 * WN * 32;
  constexpr int X_VECTORS = BM * BK / 8 / kThreads;    // 16-byte activation vectors per thread
  constexpr int W_VECTORS = (BN * BK / 32 + kThreads - 1) / kThreads;  // 32-nibble vectors per thread
  static_assert(BM * BK / 8 % kThreads == 0, "activation tile must divide over the threads");
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  _Float16 *x_lds = reinterpret_cast<_Float16 *>(gemm_lds);
  _Float16 *w_lds = x_lds + BM * LDS_STRIDE;            // [NW][BN * LDS_STRIDE]
  float *s_lds = reinterpret_cast<float *>(w_lds + NW * BN * LDS_STRIDE);  // [NW][BN]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1;
  const int wave_n = wave & 1;

  // XCD-aware tile order: workgroups are handed to the 8 XCDs round-robin, so
  // give each XCD a contiguous run of tiles (m fastest: neighbours share the
  // weight strip in that XCD's L2).
  const uint32_t total = p.tiles_m * p.tiles_n;
  uint32_t logical = blockIdx.x;
  if (total % 8 == 0) logical = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
  const uint32_t tile_m = logical % p.tiles_m;
  const uint32_t tile_n = logical / p.tiles_m;
  const uint32_t m0 = tile_m * BM;
  const uint32_t n0 = tile_n * BN;
  const uint32_t K = p.k;

  // global -> register staging: x rows (tid/8) + 64*i, vector tid%8;
  // w row (tid/2) + 256*i, half tid%2
  const uint32_t x_vec = tid & 7;
  const uint32_t x_row = tid >> 3;
  const uint32_t w_row = tid >> 1;
  const uint32_t w_half = tid & 1;

  uint4 x_reg[X_VECTORS];
  u32x4_t w_reg[NW][W_VECTORS];
  uint16_t s_reg[NW][W_VECTORS];

  auto load_global = [&](uint32_t k0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < X_VECTORS; ++i) {
      const uint32_t row = min(m0 + x_row + 64 * i, p.m - 1);  // rows past m are never stored
      x_reg[i] = reinterpret_cast<const uint4 *>(p.x + (size_t)row * K + k0)[x_vec];
    }
#pragma unroll
    for (int i = 0; i < W_VECTORS; ++i) {
      const uint32_t local = w_row + 256 * i;
      const uint32_t col = min(n0 + local, p.n - 1);  // columns past n are never stored
#pragma unroll
      for (int v = 0; v < NW; ++v) {
        w_reg[v][i] = reinterpret_cast<const u32x4_t *>(p.w[v] + (size_t)col * (K >> 1) + (k0 >> 1))[w_half];
        s_reg[v][i] = p.s[v][(size_t)col * (K >> 6) + (k0 >> 6)];
      }
    }
  };

  auto store_lds = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < X_VECTORS; ++i)
      *reinterpret_cast<uint4 *>(&x_lds[(x_row + 64 * i) * LDS_STRIDE + x_vec * 8]) = pair_order(x_reg[i]);
#pragma unroll
    for (int i = 0; i < W_VECTORS; ++i) {
      const uint32_t local = w_row + 256 * i;
      if (BN % 256 != 0 && local >= (uint32_t)BN) continue;
#pragma unroll
      for (int v = 0; v < NW; ++v) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const W4Pairs q = w4_decode_pairs(w_reg[v][i][j]);
          uint4 packed;
          packed.x = as_u32(q.p04);
          packed.y = as_u32(q.p15);
          packed.z = as_u32(q.p26);
          packed.w = as_u32(q.p37);
          *reinterpret_cast<uint4 *>(&w_lds[(v * BN + local) * LDS_STRIDE + w_half * 32 + j * 8]) = packed;
        }
        if (w_half == 0) s_lds[v * BN + local] = half_bits_to_float(s_reg[v][i]);
      }
    }
  };

  f16x_t acc[NW][WM][WN];
#pragma unroll
  for (int v = 0; v < NW; ++v)
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
      for (int b = 0; b < WN; ++b) acc[v][a][b] = zero_tile();

  const int frag_row = lane & 31;  // operand row (A) / column (B) inside a 32-wide tile
  const int frag_k = (lane >> 5) * 8;
  const int row_base = wave_m * WM * 32;
  const int col_base = wave_n * WN * 32;

  load_global(0);
  for (uint32_t k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();  // previous step's LDS reads are done
    store_lds();
    __syncthreads();
    if (k0 + BK < K) load_global(k0 + BK);

    h8_t a_frag[WM][BK / 16];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks)
        a_frag[a][ks] = *reinterpret_cast<const h8_t *>(
            &x_lds[(row_base + a * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
#pragma unroll
    for (int v = 0; v < NW; ++v) {
#pragma unroll
      for (int b = 0; b < WN; ++b) {
        h8_t b_frag[BK / 16];
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks)
          b_frag[ks] = *reinterpret_cast<const h8_t *>(
              &w_lds[(v * BN + col_base + b * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
        const float scale = s_lds[v * BN + col_base + b * 32 + frag_row];
#pragma unroll
        for (int a = 0; a < WM; ++a) {
          // one 64-wide scale group: four chained MFMAs into a temporary tile,
          // then acc += temporary * float(scale) in fp32
          f16x_t part = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_frag[a][0], b_frag[0], zero_tile(), 0, 0, 0);
#pragma unroll
          for (int ks = 1; ks < BK / 16; ++ks)
            part = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_frag[a][ks], b_frag[ks], part, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[v][a][b][i] = fmaf(part[i], scale, acc[v][a][b][i]);
        }
      }
    }
  }

  // epilogue: lane owns column col, rows (i/4)*8 + (lane/32)*4 + i%4 of each tile
#pragma unroll
  for (int b = 0; b < WN; ++b) {
    const uint32_t col = n0 + col_base + b * 32 + frag_row;
    if (col >= p.n) continue;
#pragma unroll
    for (int a = 0; a < WM; ++a) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t row = m0 + row_base + a * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
        if (row >= p.m) continue;
        float value;
        if (DUAL) {
          const float gate = acc[0][a][b][i];
          const float up = acc[NW - 1][a][b][i];
          value = gate / (1.0f + __expf(-gate)) * up;
        } else {
          value = acc[0][a][b][i];
          if (p.has_addend)
            value += half_bits_to_float(p.addend[(size_t)row * p.addend_stride + col]);
        }
        p.y[(size_t)row * p.n + col] = float_to_half_bits(value);
      }
    }
  }
}

template <int WM, int WN, bool DUAL>
hipError_t launch_tile(GemmParams &p, hipStream_t stream) {
  constexpr int NW = DUAL ? 2 : 1;
  constexpr int BM = 4 * WM * 32;
  constexpr int BN = 2 * WN * 32;
  constexpr size_t lds_bytes =
      (size_t)(BM + NW * BN) * LDS_STRIDE * sizeof(_Float16) + (size_t)NW * BN * sizeof(float);
  static bool configured = false;
  if (!configured) {
    hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(&w4a16_gemm_kernel<WM, WN, DUAL>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (status != hipSuccess) return status;
    configured = true;
  }
  p.tiles_m = (p.m + BM - 1) / BM;
  p.tiles_n = (p.n + BN - 1) / BN;
  const uint32_t blocks = p.tiles_m * p.tiles_n;
  hipLaunchKernelGGL((w4a16_gemm_kernel<WM, WN, DUAL>), dim3(blocks), dim3(kThreads), lds_bytes, stream, p);
  return hipGetLastError();
}

template <bool DUAL>
hipError_t launch_gemm(GemmParams &p, hipStream_t stream) {
  if (DUAL) return launch_tile<2, 2, true>(p, stream);  // 256 x 128, two accumulator sets
  // 256 x 256 when that still gives every CU a tile, otherwise 128 x 256 / 128 x 128
  const int cus = device_compute_units();
  const uint64_t big = (uint64_t)((p.m + 255) / 256) * ((p.n + 255) / 256);
  if (big >= (uint64_t)cus) return launch_tile<2, 4, false>(p, stream);
  const uint64_t mid = (uint64_t)((p.m + 127) / 128) * ((p.n + 255) / 256);
  if (mid >= (uint64_t)cus) return launch_tile<1, 4, false>(p, stream);
  return launch_tile<1, 2, false>(p, stream);
}

}  // namespace

hipError_t launch_w4a16_gemm_linear(const W4LinearArgs &a, hipStream_t stream) {
  GemmParams p = {};
  p.x = a.x;
  p.w[0] = a.w.weight;
  p.s[0] = a.w.scale;
  p.w[1] = a.w.weight;
  p.s[1] = a.w.scale;
  p.addend = a.addend;
  p.has_addend = a.has_addend;
  p.addend_stride = a.addend_row_stride;
  p.y = a.y;
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  return launch_gemm<false>(p, stream);
}

hipError_t launch_w4a16_gemm_dual_swiglu(const W4DualSwigluArgs &a, hipStream_t stream) {
  GemmParams p = {};
  p.x = a.x;
  p.w[0] = a.gate.weight;
  p.s[0] = a.gate.scale;
  p.w[1] = a.up.weight;
  p.s[1] = a.up.scale;
  p.y = a.product;
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  return launch_gemm<true>(p, stream);
}

// ---- m-based choice between the streaming GEMV and the MFMA GEMM ------------

hipError_t launch_w4a16_linear(const W4LinearArgs &args, hipStream_t stream) {
  if (args.m <= kGemvDotRows) return launch_w4a16_gemv_linear(args, stream);
  if (args.m <= kGemvMaxRows && (!w4a16_gemv_mfma_needs_split(args.k) || args.workspace != nullptr))
    return launch_w4a16_gemv_mfma_linear(args, stream);
  return launch_w4a16_gemm_linear(args, stream);
}

hipError_t launch_w4a16_dual_swiglu(const W4DualSwigluArgs &args, hipStream_t stream) {
  if (args.m <= kGemvDotRows) return launch_w4a16_gemv_dual_swiglu(args, stream);
  if (args.m <= kGemvMaxRows && !w4a16_gemv_mfma_needs_split(args.k))
    return launch_w4a16_gemv_mfma_dual_swiglu(args, stream);
  return launch_w4a16_gemm_dual_swiglu(args, stream);
}

hipError_t launch_w4a16_qkv(const W4QkvArgs &args, hipStream_t stream) {
  if (args.m <= kGemvDotRows) return launch_w4a16_gemv_qkv(args, stream);
  if (args.m <= kGemvMaxRows && !w4a16_gemv_mfma_needs_split(args.k))
    return launch_w4a16_gemv_mfma_qkv(args, stream);
  // prefill: three GEMMs sharing the activation through L2
  for (int i = 0; i < 3; ++i) {
    W4LinearArgs one = {};
    one.x = args.x;
    one.w = args.w[i];
    one.y = args.y[i];
    one.m = args.m;
    one.n = args.n[i];
    one.k = args.k;
    hipError_t status = launch_w4a16_gemm_linear(one, stream);
    if (status != hipSuccess) return status;
  }
  return hipSuccess;
}

}  // namespace llmopt
