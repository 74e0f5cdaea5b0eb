// W4A16 prefill GEMM for gfx950: y[M, N] = x[M, K] . W4[N, K]^T with fp16 MFMA
// and fp32 accumulation.
//
// The reference has no matrix-core W4A16 kernel: it runs the GEMV kernel
// llmopt_w4a16_linear_f16_g64_m4 for every m >= 2
// (lib/metal_dispatch_linear.ml:975-982).  Same arithmetic contract here
// (lib/metal_w4a16_source.ml:42-122), different machine mapping:
//
//  * int4 nibbles are decoded to exact fp16 integers, multiplied by the fp16
//    group scale in fp16 (one rounding, at most 2^-11 relative per weight; the
//    product overflows fp16 only for scales above 8188) and staged in LDS as
//    the MFMA B operand in natural K order; accumulation is fp32.
//  * Activation tiles are copied global -> LDS without passing registers,
//    weight nibbles pass registers for the decode.  LDS holds two stages and a
//    K step has one barrier; the decode of the next stage is issued between
//    groups of MFMAs of the current one.
//  * The activation tile is the MFMA A operand (rows = m) and the weight tile
//    the B operand (columns = n), so every lane's 16 accumulator values belong
//    to one output column.
#include <algorithm>
#include <type_traits>

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
  // K split over blockIdx.y (SPLITK instantiations): every workgroup covers k_len of K, leaves
  // its tile's float32 sums in partials[split][tile], and the last one to arrive at a tile (one
  // counter per tile, zero between launches) adds the splits in order and stores the output.
  uint32_t k_len;
  float *partials;
  uint32_t *counters;
  // segments > 1: several matrices multiply the same activation in one launch (the QKV projection).
  // Their column tiles follow each other (seg_tiles each); a workgroup's tile lies in one segment
  // and takes its weights, scales, output and width from there.  No addend, no K split.
  uint32_t segments;
  const uint8_t *seg_w[3];
  const uint16_t *seg_s[3];
  uint16_t *seg_y[3];
  uint32_t seg_n[3];
  uint32_t seg_tiles[3];
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
// XS: LDS stages of the activation tile = steps a K loop iteration is unrolled by = weight
// register sets.  2 for the large tiles, whose steps are long enough to cover a load; 4 for the
// small ones, whose steps are shorter than the trip to memory: the activation copy then runs
// three steps ahead of its use and the weights four (K is rounded up to whole passes of four
// steps, the surplus steps run on zero weights).
template <int WM, int WN, bool DUAL, int XS, bool SPLITK = false>
__global__ __launch_bounds__(kThreads) void w4a16_gemm_kernel(GemmParams p) {
  static_assert(XS == 2 || XS == 4, "the weight stage alternates with the step: an even unroll");
  static_assert(!SPLITK || !DUAL, "silu(gate) * up is not linear in the K ranges");
  constexpr int WS = XS;            // weight register sets
  constexpr int NW = DUAL ? 2 : 1;  // weight matrices per tile
  constexpr int BM = 4 * WM * 32;
  constexpr int BN = 2 * WN * 32;
  constexpr int W_VECTORS = (BN * BK / 32 + kThreads - 1) / kThreads;  // 32-nibble vectors per thread
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  // x[BM] rows of BK halfs, vector index swizzled, in XS stages; w[NW][BN] rows of LDS_STRIDE
  // halfs in two.  XS = 2: {x, w} {x, w}; XS = 4: the four x stages, then the two of w.
  constexpr int X_HALFS = BM * BK;
  constexpr int W_HALFS = NW * BN * LDS_STRIDE;
  constexpr int X_STAGE_HALFS = XS == 2 ? X_HALFS + W_HALFS : X_HALFS;  // from one x stage to the next
  constexpr int W_STAGE_HALFS = XS == 2 ? X_HALFS + W_HALFS : W_HALFS;
  constexpr int W_BASE_HALFS = XS == 2 ? X_HALFS : XS * X_HALFS;
  constexpr int X_CHUNKS = BM / 8 / (kThreads / 64);  // 8-row direct loads per wave and K step
  static_assert(BM / 8 % (kThreads / 64) == 0, "activation tile must divide over the waves");
  _Float16 *stage_lds = reinterpret_cast<_Float16 *>(gemm_lds);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  const uint8_t *weight0 = p.w[0];
  const uint16_t *scale0 = p.s[0];
  uint16_t *output0 = p.y;
  uint32_t width = p.n, tile_column = tile_n;
  if constexpr (!DUAL && !SPLITK) {
    if (p.segments > 1) {
      uint32_t segment = 0;
      while (segment + 1 < p.segments && tile_column >= p.seg_tiles[segment]) tile_column -= p.seg_tiles[segment++];
      weight0 = p.seg_w[segment];
      scale0 = p.seg_s[segment];
      output0 = p.seg_y[segment];
      width = p.seg_n[segment];
    }
  }
  const uint32_t m0 = tile_m * BM;
  const uint32_t n0 = tile_column * BN;
  const uint32_t K = p.k;                                   // row stride of x and of the weights
  const uint32_t KS = SPLITK ? p.k_len : p.k;               // this workgroup's extent of K ...
  const uint32_t k_base = SPLITK ? blockIdx.y * p.k_len : 0;  // ... and where it begins

  // Activations go global -> LDS directly, 8 rows (1 KiB) per wave-wide load:
  // lane l fills physical vector l % 8 of row l / 8, i.e. fetches the logical
  // vector which the swizzle maps there.
  const uint16_t *x_src[X_CHUNKS];
#pragma unroll
  for (int c = 0; c < X_CHUNKS; ++c) {
    const uint32_t tile_row = (wave * X_CHUNKS + c) * 8 + (lane >> 3);
    const uint32_t vec = (lane & 7) ^ ((tile_row >> 1) & 7u);
    const uint32_t row = min(m0 + tile_row, p.m - 1);  // rows past m are never stored
    x_src[c] = p.x + (size_t)row * K + k_base + vec * 8;
  }
  // Every vector memory load of the K loop is issued as assembly and waited for
  // by hand: loads return in order, so "at most n outstanding" names exactly
  // which of them have landed, and no wait is stricter than the data flow needs
  // (the compiler's own bookkeeping waits for the activation copy before the
  // next LDS write, and for the youngest weight loads on every other step).
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)gemm_lds;
  auto fetch_x = [&](uint32_t k0, int stage) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < X_CHUNKS; ++c) {
      const uint32_t lds_address =
          lds_base + (uint32_t)((stage * X_STAGE_HALFS + (wave * X_CHUNKS + c) * 8 * BK) * sizeof(_Float16));
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                   :
                   : "v"(x_src[c] + k0), "s"(lds_address)
                   : "memory");
    }
  };

  // Weights go global -> registers (a row of 32 bytes per K step, shared by two or four threads) -> decode -> LDS.
  // WS register sets: set s % WS holds the weights of step s; it is decoded during step
  // s - 1 and requested again right after, for step s - 1 + WS.
  static_assert(W_VECTORS == 1, "one 32-nibble vector per thread and matrix");
  // Every thread takes an equal share of the decode.  Two matrices of 128 columns are 256 weight
  // rows, one per thread pair: a thread fetches and decodes one matrix (rows 0..127 gate, 128..255
  // up).  One matrix of 128 columns: four threads share a row, eight bytes each.  (Before, half
  // the threads did all of it in both cases.)
  constexpr bool kThreadPerMatrix = DUAL && NW * BN == kThreads / 2;
  constexpr int NWF = kThreadPerMatrix ? 1 : NW;                                   // matrices a thread fetches
  constexpr int ROW_THREADS = (!DUAL && BN * 4 == kThreads) ? 4 : 2;             // threads sharing a row's 32 bytes
  constexpr int DW = 8 / ROW_THREADS;                                              // dwords (of 8 nibbles) per thread
  static_assert(DUAL || BN * ROW_THREADS == kThreads, "every thread has a row piece");
  const uint32_t w_row = tid / ROW_THREADS;
  const uint32_t w_half = tid % ROW_THREADS;
  typedef uint32_t words_t __attribute__((ext_vector_type(DW)));
  struct Fetched {
    words_t w[NWF];
    uint32_t s[NWF];  // fp16 bits in the low half
  };
  Fetched fetched[WS];
  constexpr int W_LOADS = 2 * NWF;  // vector memory loads of one fetch_w
  const uint32_t fetch_matrix = kThreadPerMatrix ? w_row / BN : 0;
  const uint32_t fetch_row = kThreadPerMatrix ? w_row % BN : w_row;
  const uint32_t w_col = min(n0 + fetch_row, width - 1);  // columns past n are never stored
  const uint8_t *w_base[NWF];
  const uint16_t *s_base[NWF];
#pragma unroll
  for (int v = 0; v < NWF; ++v) {
    w_base[v] = kThreadPerMatrix ? (fetch_matrix ? p.w[NW - 1] : p.w[0]) : (v == 0 ? weight0 : p.w[v]);
    s_base[v] = kThreadPerMatrix ? (fetch_matrix ? p.s[NW - 1] : p.s[0]) : (v == 0 ? scale0 : p.s[v]);
  }

  // The compiler takes the destination of these loads as written when the statement ends, while
  // the data lands later: between a fetch_w and the wait_w of the same set, control flow must
  // give it no reason to copy the set (a second loop with its own register allocation did, and
  // read registers whose loads were still in flight).
  auto fetch_w = [&](Fetched &f, uint32_t k0) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < NWF; ++v) {
      const void *w_src = w_base[v] + (size_t)w_col * (K >> 1) + ((k_base + k0) >> 1) + w_half * (DW * 4);
      const void *s_src = s_base[v] + (size_t)w_col * (K >> 6) + ((k_base + k0) >> 6);
      if constexpr (DW == 4)
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(f.w[v]) : "v"(w_src) : "memory");
      else
        asm volatile("global_load_dwordx2 %0, %1, off" : "=&v"(f.w[v]) : "v"(w_src) : "memory");
      asm volatile("global_load_ushort %0, %1, off" : "=&v"(f.s[v]) : "v"(s_src) : "memory");
    }
  };
  // at most `younger` loads issued after those of f are still outstanding
  auto wait_w = [&](Fetched &f, auto younger) __attribute__((always_inline)) {
    constexpr int n = decltype(younger)::value;
    if constexpr (NWF == 1)
      asm volatile("s_waitcnt vmcnt(%2)" : "+v"(f.w[0]), "+v"(f.s[0]) : "n"(n) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(%4)"
                   : "+v"(f.w[0]), "+v"(f.s[0]), "+v"(f.w[1]), "+v"(f.s[1])
                   : "n"(n)
                   : "memory");
  };
  auto wait_all = [&](auto younger) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(decltype(younger)::value) : "memory");
  };

  // The decode of one fetched set into an LDS stage, cut into items of one
  // weight dword (8 nibbles): q * s as fp16 (one rounding, 2^-11 relative at
  // most), in natural K order.
  constexpr int ITEMS = NWF * DW;
  // live = false: the set belongs to a step past the end of K (XS = 4 rounds the steps up to whole
  // loop passes; the requests of such a step are clamped to the last K block): it is stored as
  // zeros, so the step's MFMAs add nothing.
  auto store_item = [&](const Fetched &f, int stage, int item, bool live) __attribute__((always_inline)) {
    _Float16 *w_lds = stage_lds + W_BASE_HALFS + stage * W_STAGE_HALFS;
    const int v = item / DW;
    const int j = item % DW;
    if (DUAL && !kThreadPerMatrix && w_row >= (uint32_t)BN) return;
    const _Float16 scale = live ? __builtin_bit_cast(_Float16, (uint16_t)f.s[v]) : (_Float16)0.0f;
    const uint4 packed = w4_scaled_natural(f.w[v][j], scale);
    // (one matrix per thread: w_row runs over the rows of both matrices, as v * BN + row does)
    *reinterpret_cast<uint4 *>(&w_lds[(v * BN + w_row) * LDS_STRIDE + w_half * (DW * 8) + j * 8]) = packed;
  };

  f16x_t acc[NW][WM][WN];
#pragma unroll
  for (int v = 0; v < NW; ++v)
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
      for (int b = 0; b < WN; ++b) acc[v][a][b] = zero_tile();

  const int frag_row = lane & 31;  // operand row (A) / column (B) inside a 32-wide tile
  const int frag_kq = lane >> 5;
  const int frag_k = frag_kq * 8;
  const int row_base = wave_m * WM * 32;
  const int col_base = wave_n * WN * 32;

  // One barrier per K step.  Step i runs its MFMAs from weight stage i % 2 and activation
  // stage i % XS while the set fetched for step i + 1 is decoded into the other weight stage;
  // that set is then requested again for step i + 1 + WS, and the activation copy of step
  // i + XS - 1 goes into the stage step i - 1 read (requests past the end fetch the last K
  // block again, which nothing reads).  Loads return in order, so the two waits count the
  // loads issued after the one they need: every step issues X_CHUNKS copies, then W_LOADS
  // weight loads.  The issue order is fixed by hand: groups of
  // four chained MFMAs alternate with one or two decode items, and the weight
  // operands of the next column block are read while the current one computes,
  // so the matrix pipe does not wait for the vector work, LDS or HBM.
  constexpr int BLOCKS = NW * WN;      // column blocks of a step
  constexpr int GROUPS = BLOCKS * WM;  // MFMA groups of a step
  constexpr int ITEMS_PER_GROUP = (ITEMS + GROUPS - 1) / GROUPS;
  constexpr int STEP_LOADS = X_CHUNKS + W_LOADS;
  auto step = [&](uint32_t k0, auto index) __attribute__((always_inline)) {
    constexpr int j = decltype(index)::value;  // step number modulo XS
    constexpr int stage = j & 1;
    constexpr int next_set = (j + 1) % WS;
    __syncthreads();  // this stage is written; the other stage's readers are done
    const _Float16 *x_lds = stage_lds + j * X_STAGE_HALFS;
    const _Float16 *w_lds = stage_lds + W_BASE_HALFS + stage * W_STAGE_HALFS;
    h8_t a_frag[WM][BK / 16];
    h8_t b_frag[2][BK / 16];
    auto read_block = [&](int block) __attribute__((always_inline)) {
      const int v = block / WN;
      const int b = block % WN;
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks)
        b_frag[block & 1][ks] = *reinterpret_cast<const h8_t *>(
            &w_lds[(v * BN + col_base + b * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
    };
    read_block(0);
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks)
        a_frag[a][ks] = *reinterpret_cast<const h8_t *>(
            &x_lds[(row_base + a * 32 + frag_row) * BK +
                   (((ks * 2 + frag_kq) ^ (((row_base + a * 32 + frag_row) >> 1) & 7)) << 3)]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int block = 0; block < BLOCKS; ++block) {
      const int v = block / WN;
      const int b = block % WN;
#pragma unroll
      for (int a = 0; a < WM; ++a) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks)
          acc[v][a][b] =
              __builtin_amdgcn_mfma_f32_32x32x16_f16(a_frag[a][ks], b_frag[block & 1][ks], acc[v][a][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (a == 0 && block + 1 < BLOCKS) read_block(block + 1);
        const int group = block * WM + a;
        // the set was requested at the end of step i - WS: WS - 1 steps of loads are younger
        // (XS = 2: the wait that ended the last step left one set of weight loads)
        if (group == 0)
          wait_w(fetched[next_set], std::integral_constant<int, XS == 2 ? W_LOADS : (WS - 1) * STEP_LOADS>{});
#pragma unroll
        for (int n = 0; n < ITEMS_PER_GROUP; ++n)
          if (group * ITEMS_PER_GROUP + n < ITEMS)
            store_item(fetched[next_set], stage ^ 1, group * ITEMS_PER_GROUP + n, XS == 2 || k0 + BK < KS);
        if (group == 0) fetch_x(min(k0 + (XS - 1) * BK, KS - BK), (j + XS - 1) % XS);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    fetch_w(fetched[next_set], min(k0 + (1 + WS) * BK, KS - BK));
    __builtin_amdgcn_sched_barrier(0);
    // the activation copy of step i + 1 has landed: it went out in step i + 2 - XS, before
    // that step's weight loads and the XS - 2 steps of loads since
    wait_all(std::integral_constant<int, (XS - 2) * STEP_LOADS + W_LOADS>{});
  };

#pragma unroll
  for (int s = 0; s < XS - 1; ++s) fetch_x(min((uint32_t)s * BK, KS - BK), s);
#pragma unroll
  for (int s = 0; s < WS; ++s) fetch_w(fetched[s], min((uint32_t)s * BK, KS - BK));
  wait_w(fetched[0], std::integral_constant<int, (WS - 1) * W_LOADS>{});
#pragma unroll
  for (int item = 0; item < ITEMS; ++item) store_item(fetched[0], 0, item, true);
  fetch_w(fetched[0], min((uint32_t)WS * BK, KS - BK));
  if constexpr (XS == 2) {
    for (uint32_t k0 = 0; k0 < KS; k0 += 2 * BK) {
      step(k0, std::integral_constant<int, 0>{});
      if (k0 + BK < KS) step(k0 + BK, std::integral_constant<int, 1>{});
    }
  } else {  // whole passes of XS steps (the surplus ones multiply by zeros): no branch between a request and its wait
    wait_all(std::integral_constant<int, W_LOADS>{});  // every activation copy and every other set has landed
    for (uint32_t k0 = 0; k0 < KS; k0 += XS * BK) {
      step(k0, std::integral_constant<int, 0>{});
      step(k0 + BK, std::integral_constant<int, 1>{});
      step(k0 + 2 * BK, std::integral_constant<int, 2>{});
      step(k0 + 3 * BK, std::integral_constant<int, 3>{});
    }
  }
  wait_all(std::integral_constant<int, 0>{});  // the surplus requests still target live registers

  if constexpr (SPLITK) {
    // Hand-over between the workgroups of a tile through memory every CU sees: device-scope
    // 16-byte stores and loads (no cache write-back, no per-element atomics).  A partial tile is
    // kept in the accumulators' own layout - [wave][a][b][i / 4][lane] float4 - so a lane reads
    // back exactly the registers its counterpart wrote, one coalesced KiB per wave instruction.
    // One arrival per workgroup; the last to arrive adds the splits in split order, its own sums
    // taking their place in that order: the same result whichever arrives last.
    __shared__ uint32_t arrival_lds;
    constexpr uint32_t kTileFloats = (uint32_t)BM * BN;
    constexpr int QUADS = WM * WN * 4;  // float4 groups per lane
    const size_t tile_count = (size_t)p.tiles_m * p.tiles_n;
    auto quad_address = [&](uint32_t split, int quad) __attribute__((always_inline)) {
      return p.partials + ((split * tile_count + logical) * kTileFloats) + ((size_t)(wave * QUADS + quad) * 64 + lane) * 4;
    };
#pragma unroll
    for (int b = 0; b < WN; ++b)
#pragma unroll
      for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f4_t value = {acc[0][a][b][g * 4], acc[0][a][b][g * 4 + 1], acc[0][a][b][g * 4 + 2], acc[0][a][b][g * 4 + 3]};
          asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(quad_address(blockIdx.y, (b * WM + a) * 4 + g)), "v"(value) : "memory");
        }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // every wave's stores have been acknowledged
    if (tid == 0) {
      const uint32_t arrived = __hip_atomic_fetch_add(p.counters + logical, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = arrived == gridDim.y - 1;
      if (last) __hip_atomic_store(p.counters + logical, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      arrival_lds = last ? 1u : 0u;
    }
    __syncthreads();
    if (arrival_lds == 0) return;
    f4_t sum[QUADS];
#pragma unroll
    for (int q = 0; q < QUADS; ++q) sum[q] = f4_t{0.f, 0.f, 0.f, 0.f};
    for (uint32_t split = 0; split < gridDim.y; ++split) {
      if (split == blockIdx.y) {
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
          for (int a = 0; a < WM; ++a)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
              for (int e = 0; e < 4; ++e) sum[(b * WM + a) * 4 + g][e] += acc[0][a][b][g * 4 + e];
      } else {
        f4_t other[QUADS];
#pragma unroll
        for (int q = 0; q < QUADS; ++q)
          asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(other[q]) : "v"(quad_address(split, q)) : "memory");
#pragma unroll
        for (int q = 0; q < QUADS; ++q) asm volatile("s_waitcnt vmcnt(0)" : "+v"(other[q]) : : "memory");
#pragma unroll
        for (int q = 0; q < QUADS; ++q) sum[q] += other[q];
      }
    }
#pragma unroll
    for (int b = 0; b < WN; ++b)
#pragma unroll
      for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[0][a][b][i] = sum[(b * WM + a) * 4 + i / 4][i % 4];
  }
  // epilogue: lane owns column col, rows (i/4)*8 + (lane/32)*4 + i%4 of each tile
#pragma unroll
  for (int b = 0; b < WN; ++b) {
    const uint32_t col = n0 + col_base + b * 32 + frag_row;
    if (col >= width) continue;
#pragma unroll
    for (int a = 0; a < WM; ++a) {
      // The sixteen addends of a 32 x 32 block are requested together, for rows past m at the last
      // row's address: a load under a per-element test is waited for where it stands, and the
      // epilogue of a tile with a residual was sixteen trips to memory per block, one after the other.
      uint16_t addend_bits[16] = {};
      if (!DUAL && p.has_addend) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t row = m0 + row_base + a * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
          addend_bits[i] = p.addend[(size_t)min(row, p.m - 1) * p.addend_stride + col];
        }
      }
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
          if (p.has_addend) value += half_bits_to_float(addend_bits[i]);
        }
        output0[(size_t)row * width + col] = float_to_half_bits(value);
      }
    }
  }
}

template <int WM, int WN, bool DUAL, int XS = 2, bool SPLITK = false>
hipError_t launch_tile(GemmParams &p, hipStream_t stream, uint32_t splits = 1) {
  constexpr int NW = DUAL ? 2 : 1;
  constexpr int BM = 4 * WM * 32;
  constexpr int BN = 2 * WN * 32;
  constexpr size_t lds_bytes = ((size_t)XS * BM * BK + 2 * (size_t)NW * BN * LDS_STRIDE) * sizeof(_Float16);
  static_assert(lds_bytes <= 160 * 1024, "a workgroup's stages must fit the CU's LDS");
  static bool configured[kMaxDevices] = {};
  if (hipError_t status = allow_dynamic_lds(reinterpret_cast<const void *>(&w4a16_gemm_kernel<WM, WN, DUAL, XS, SPLITK>),
                                            (int)lds_bytes, configured))
    return status;
  p.tiles_m = (p.m + BM - 1) / BM;
  p.tiles_n = (p.n + BN - 1) / BN;
  if (p.segments > 1) {
    if (DUAL || SPLITK || p.has_addend) return hipErrorInvalidValue;
    p.tiles_n = 0;
    for (uint32_t i = 0; i < p.segments; ++i) p.tiles_n += p.seg_tiles[i] = (p.seg_n[i] + BN - 1) / BN;
  }
  const uint32_t blocks = p.tiles_m * p.tiles_n;
  p.k_len = p.k / splits;
  hipLaunchKernelGGL((w4a16_gemm_kernel<WM, WN, DUAL, XS, SPLITK>), dim3(blocks, splits), dim3(kThreads), lds_bytes,
                     stream, p);
  return hipGetLastError();
}

// K ranges per tile when 128 x 128 tiles leave at least half the CUs without one (1: no split):
// as many as fill the device, each a whole number of four-step loop passes.
uint32_t gemm_k_splits(uint32_t m, uint32_t n, uint32_t k) {
  const uint64_t tiles = (uint64_t)((m + 127) / 128) * ((n + 127) / 128);
  const uint64_t cus = (uint64_t)device_compute_units();
  if (tiles == 0 || tiles * 2 > cus) return 1;
  uint32_t splits = (uint32_t)std::min<uint64_t>(4, cus / tiles);
  while (splits > 1 && (k % splits != 0 || (k / splits) % (4 * BK) != 0)) --splits;
  return splits;
}

template <bool DUAL>
hipError_t launch_gemm(GemmParams &p, hipStream_t stream) {
  const int cus = device_compute_units();
  if (DUAL) {
    // 256 x 128, two accumulator sets; 128 x 128 with four activation stages when even those tiles
    // leave CUs without one (the decode model's 576 -> 1536 pair at 2048 rows: 96 tiles of 256 x 128,
    // whose nine two-stage steps each wait out a trip to memory)
    const uint64_t small_pair = (uint64_t)((p.m + 127) / 128) * ((p.n + 127) / 128);
    if (small_pair <= (uint64_t)cus) return launch_tile<1, 2, true, 4>(p, stream);
    return launch_tile<2, 2, true>(p, stream);
  }
  // 256 x 256 when that still gives every CU a tile, otherwise 256 x 128 / 128 x 256 / 128 x 128
  const uint64_t big = (uint64_t)((p.m + 255) / 256) * ((p.n + 255) / 256);
  if (big >= (uint64_t)cus) return launch_tile<2, 4, false>(p, stream);
  // Half that size, tall (256 x 128) or wide (128 x 256), whichever pads less; the tall one when
  // they tie (its waves read 16 operand vectors from LDS per 16 MFMAs, the wide one's 20: 76.5
  // against 80 us at 512 x 14336, 81.7 against 86.3 at 2048 x 4096).  Also when a few CUs stay
  // without a tile: 224 such tiles beat 448 of 128 x 128, two on most CUs.
  const uint64_t tall = (uint64_t)((p.m + 255) / 256) * ((p.n + 127) / 128);
  const uint64_t wide = (uint64_t)((p.m + 127) / 128) * ((p.n + 255) / 256);
  if (std::min(tall, wide) * 8 >= (uint64_t)cus * 7)
    return tall <= wide ? launch_tile<2, 2, false>(p, stream) : launch_tile<1, 4, false>(p, stream);
  // 128 x 128 tiles have steps shorter than a trip to memory.  With two stages they fit a CU
  // twice, which covers the loads; when there is at most one tile per CU anyway, four
  // activation stages do (measured 58 -> 49 us at 512 x 4096 x 4096, and nothing for the 128 x 256
  // tiles, which stay with two).
  const uint64_t small = (uint64_t)((p.m + 127) / 128) * ((p.n + 127) / 128);
  // Fewer tiles than half the CUs: K is split over workgroups as well, so that every CU holds a
  // tile (128 tiles at 512 x 4096 x 4096 left half the device idle).
  const uint32_t splits = gemm_k_splits(p.m, p.n, p.k);
  if (splits > 1 && p.partials != nullptr && p.counters != nullptr)
    return launch_tile<1, 2, false, 4, true>(p, stream, splits);
  if (small <= (uint64_t)cus) return launch_tile<1, 2, false, 4>(p, stream);
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
  const uint64_t tiles = (uint64_t)((a.m + 127) / 128) * ((a.n + 127) / 128);
  if (a.workspace != nullptr && a.counters != nullptr && tiles <= a.counter_count &&
      a.workspace_bytes >= w4a16_gemm_workspace_bytes(a.m, a.n, a.k)) {
    p.partials = static_cast<float *>(a.workspace);
    p.counters = a.counters;
  }
  return launch_gemm<false>(p, stream);
}

size_t w4a16_gemm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
  const uint32_t splits = gemm_k_splits(m, n, k);
  const size_t tiles = (size_t)((m + 127) / 128) * ((n + 127) / 128);  // whole 128 x 128 tiles of float32
  return splits > 1 ? (size_t)splits * tiles * 128 * 128 * sizeof(float) : 0;
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
  if (w4a16_gemv_quad_ok(args)) return launch_w4a16_gemv_quad_linear(args, stream);
  // Many short rows (the LM head of a model with a small hidden size): the dot-product kernel takes
  // rows of a few hundred bytes one wave at a time, the matrix-core kernel's 16-row tiles stream
  // them faster (49152 x 576 at two rows: 9.8 against 15.6 us; at one row 9.8 against 11.6).
  const bool many_short_rows = args.n >= 16384 && args.k <= 1024 && !w4a16_gemv_mfma_needs_split(args.k);
  if (args.m <= kGemvDotRows && !many_short_rows) return launch_w4a16_gemv_linear(args, stream);
  if (args.m <= kGemvMaxRows && (!w4a16_gemv_mfma_needs_split(args.k) || args.workspace != nullptr))
    return launch_w4a16_gemv_mfma_linear(args, stream);
  if (w4a16_gemv_mfma_row_groups_ok(args.m, args.n, args.k) && args.y_f32 == nullptr)
    return launch_w4a16_gemv_mfma_linear(args, stream);
  return launch_w4a16_gemm_linear(args, stream);
}

bool w4a16_norm_in_kernel(uint32_t m, uint64_t columns, uint32_t k) {
  if (m <= kGemvDotRows) return w4a16_gemv_norm_ok(m, k);
  // the matrix-core GEMV with K inside one workgroup (same conditions as the launchers below), up to
  // 32 rows: every workgroup normalises its eight rows again, which at 128 rows costs more than
  // the separate launch (decode step 2.83 against 2.74 ms; 1.35 against 1.39 ms at 32 rows)
  return m <= 32 && k % 64 == 0 && k >= 8 &&
         ((m <= kGemvMaxRows && !w4a16_gemv_mfma_needs_split(k)) || w4a16_gemv_mfma_row_groups_ok(m, columns, k));
}

hipError_t launch_w4a16_dual_swiglu(const W4DualSwigluArgs &args, hipStream_t stream) {
  if (args.norm.weight != nullptr && !w4a16_norm_in_kernel(args.m, 2ull * args.n, args.k)) return hipErrorInvalidValue;
  if (args.m <= kGemvDotRows) return launch_w4a16_gemv_dual_swiglu(args, stream);
  if ((args.m <= kGemvMaxRows && !w4a16_gemv_mfma_needs_split(args.k)) ||
      w4a16_gemv_mfma_row_groups_ok(args.m, 2ull * args.n, args.k))
    return launch_w4a16_gemv_mfma_dual_swiglu(args, stream);
  return launch_w4a16_gemm_dual_swiglu(args, stream);
}

hipError_t launch_w4a16_qkv(const W4QkvArgs &args, hipStream_t stream) {
  if (args.norm.weight != nullptr &&
      !w4a16_norm_in_kernel(args.m, (uint64_t)args.n[0] + args.n[1] + args.n[2], args.k))
    return hipErrorInvalidValue;
  if (args.m <= kGemvDotRows) return launch_w4a16_gemv_qkv(args, stream);
  if ((args.m <= kGemvMaxRows && !w4a16_gemv_mfma_needs_split(args.k)) ||
      w4a16_gemv_mfma_row_groups_ok(args.m, (uint64_t)args.n[0] + args.n[1] + args.n[2], args.k))
    return launch_w4a16_gemv_mfma_qkv(args, stream);
  // prefill.  Small projections (at most two 128 x 128 tiles per CU over the three matrices): one
  // launch whose column tiles run over the three matrices - each of them alone leaves most CUs
  // without a tile and costs a launch (the 576 / 192 / 192-wide projections of the small model:
  // 11 us each, three times a layer).
  const uint64_t row_tiles = (args.m + 127) / 128;
  const uint64_t tiles = row_tiles * ((args.n[0] + 127) / 128 + (args.n[1] + 127) / 128 + (args.n[2] + 127) / 128);
  if (tiles <= 2 * (uint64_t)device_compute_units() && args.n[0] > 0 && args.n[1] > 0 && args.n[2] > 0) {
    GemmParams p = {};
    p.x = args.x;
    p.m = args.m;
    p.k = args.k;
    p.segments = 3;
    for (int i = 0; i < 3; ++i) {
      p.seg_w[i] = args.w[i].weight;
      p.seg_s[i] = args.w[i].scale;
      p.seg_y[i] = args.y[i];
      p.seg_n[i] = args.n[i];
    }
    p.w[0] = p.w[1] = p.seg_w[0];
    p.s[0] = p.s[1] = p.seg_s[0];
    p.y = p.seg_y[0];
    p.n = p.seg_n[0];
    if (tiles <= (uint64_t)device_compute_units()) return launch_tile<1, 2, false, 4>(p, stream);
    return launch_tile<1, 2, false>(p, stream);
  }
  // large ones: three GEMMs sharing the activation through L2
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
