// Launchers shared between kernel translation units (not part of the host
// interface): the m-based choice between the streaming GEMV and the MFMA GEMM
// is made in w4a16_linear.hip.
#pragma once

#include "kernels.h"

namespace llmopt {

int device_compute_units();

// hipFuncSetAttribute applies to one device: launchers that raise a kernel's dynamic LDS limit keep
// one "done" flag per device (a process may hold a context on each).
constexpr int kMaxDevices = 64;
inline int current_device() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return -1;
  return device;
}
// Raises `kernel`'s dynamic LDS limit to `bytes` on the current device, once per device (`done`: the
// launcher's own flags).
inline hipError_t allow_dynamic_lds(const void *kernel, int bytes, bool (&done)[kMaxDevices]) {
  const int device = current_device();
  if (device < 0) return hipErrorInvalidDevice;
  if (done[device]) return hipSuccess;
  const hipError_t status = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (status == hipSuccess) done[device] = true;
  return status;
}

hipError_t launch_w4a16_gemv_linear(const W4LinearArgs &args, hipStream_t stream);
hipError_t launch_w4a16_gemv_qkv(const W4QkvArgs &args, hipStream_t stream);
hipError_t launch_w4a16_gemv_dual_swiglu(const W4DualSwigluArgs &args, hipStream_t stream);

// kGemvDotRows < m <= kGemvMaxRows: matrix-core GEMV
// true when K does not fit one workgroup (more than 16 ranges of 256): only the plain
// linear can then run (it splits K over workgroups and needs scratch)
bool w4a16_gemv_norm_ok(uint32_t m, uint32_t k);
bool w4a16_gemv_mfma_needs_split(uint32_t k);
// kGemvMaxRows < m <= 128 with small weights and a K one workgroup covers: the
// same kernel once per group of 8 rows (the weights are re-read from L2), which
// beats a handful of 128-wide GEMM tiles on 256 CUs.  `columns` = all outputs
// of the launch (three matrices of a QKV launch, two of a SwiGLU pair).
bool w4a16_gemv_mfma_row_groups_ok(uint32_t m, uint64_t columns, uint32_t k);
hipError_t launch_w4a16_gemv_mfma_linear(const W4LinearArgs &args, hipStream_t stream);
hipError_t launch_w4a16_gemv_mfma_qkv(const W4QkvArgs &args, hipStream_t stream);
hipError_t launch_w4a16_gemv_mfma_dual_swiglu(const W4DualSwigluArgs &args, hipStream_t stream);

// One to four rows at the K values w4a16_gemv_quad.hip is instantiated for: whole-row-piece loads
// on the 4x4x4 matrix-core blocks, one workgroup per CU.
bool w4a16_gemv_quad_ok(const W4LinearArgs &args);
hipError_t launch_w4a16_gemv_quad_linear(const W4LinearArgs &args, hipStream_t stream);

hipError_t launch_w4a16_gemm_linear(const W4LinearArgs &args, hipStream_t stream);
hipError_t launch_w4a16_gemm_dual_swiglu(const W4DualSwigluArgs &args, hipStream_t stream);

}  // namespace llmopt
