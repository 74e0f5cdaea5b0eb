// Internal runtime objects behind include/llmopt_hip.h: context, buffers,
// kernel registry, recorded dispatches.  Host C++ only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>

#include <atomic>
#include <string>
#include <vector>

#include "../../include/llmopt_hip.h"

namespace llmopt {

// ---- errors ---------------------------------------------------------------
// Sets the calling thread's last-error message and returns `code`.
int fail(int code, const char *format, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t error, const char *what);
const char *last_error();
void clear_error();

#define LLMOPT_HIP_TRY(expr, what)                                   \
  do {                                                               \
    hipError_t llmopt_status_ = (expr);                              \
    if (llmopt_status_ != hipSuccess) return fail_hip(llmopt_status_, what); \
  } while (0)

// ---- objects --------------------------------------------------------------
struct RefCounted {
  std::atomic<int> refs{1};
};

}  // namespace llmopt

struct llmopt_hip_context : llmopt::RefCounted {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  std::string name;
  int compute_units = 256;
  // Scratch for kernels that need device memory beyond inputs and outputs
  // (split-context attention partials).  Grown on demand, reused across calls
  // on the context's single stream.
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  // Counts replacements of the workspace block: a captured graph holds the block's address and
  // is captured again when this has moved on.
  uint64_t workspace_generation = 0;
  // While a retained plan captures its records the workspace cannot be replaced (nothing may be
  // allocated, and nodes already captured hold the old address): requests beyond the block are
  // only recorded here, the capture is thrown away, the block grown, the capture repeated.
  bool sizing_capture = false;
  size_t sizing_wanted = 0;
  // Set whenever a launch asks for the workspace or the counters (a profiled commit keeps such
  // launches off its concurrent branches: they share the memory).
  bool scratch_touched = false;
  // Arrival counters of kernels that split one output tile over several
  // workgroups; zeroed once, every kernel leaves them zero.
  uint32_t *counters = nullptr;
  uint32_t counter_count = 0;
};

struct llmopt_hip_buffer : llmopt::RefCounted {
  llmopt_hip_context *context = nullptr;
  llmopt_hip_buffer *parent = nullptr;  // retained when this is a view
  uint8_t *device = nullptr;            // address of byte 0 of this buffer
  size_t length = 0;
  bool owns_memory = false;
};

struct llmopt_hip_library : llmopt::RefCounted {
  llmopt_hip_context *context = nullptr;
  std::string path;
};

namespace llmopt {

struct BoundBuffer {
  uint8_t *device;
  size_t length;
};

// A validated-at-launch dispatch: everything a kernel handler needs.
struct DispatchRecord {
  std::string name;
  std::vector<BoundBuffer> buffers;
  std::vector<llmopt_hip_buffer *> retained;  // keeps the handles alive
  std::vector<uint8_t> parameters;
  int64_t grid[3];
  int64_t group[3];
  bool barrier_before = false;
  // Set by a retained plan on llmopt_attention_q8_paged_* records: the context length is read
  // from this device word (one per sequence, all equal) instead of parameter byte 12, and the
  // launch is sized for `device_past_capacity` tokens, so that one captured launch serves every
  // step of a sequence.
  const uint32_t *device_past_lengths = nullptr;
  uint32_t device_past_capacity = 0;
  // Set by a retained plan on its llmopt_cache_pack_checkpoint_q8_simd launches: the checkpoint slot of
  // the step lives in device memory (the reference rewrites byte 0 of the parameter block per step,
  // native/ocaml_metal_stubs.m:2186-2188).
  const uint32_t *device_checkpoint = nullptr;
};

// A kernel handler checks buffer count, parameter length and buffer sizes
// against the parameter block, then launches asynchronously on the context's
// stream.  Returns LLMOPT_OK or a failure status (message set).
typedef int (*KernelHandler)(llmopt_hip_context *context, const DispatchRecord &record);

struct KernelEntryPoint {
  const char *name;
  const char *operation;  // Kernel_abi.Operation.to_string (lib/kernel_abi.ml:37-70)
  KernelHandler handler;
};

// All implemented entry points (ops_*.cpp add theirs).
const std::vector<KernelEntryPoint> &kernel_table();
const KernelEntryPoint *find_kernel(const char *name);

// ---- helpers for handlers --------------------------------------------------
// "Metal %s buffer is too small" check of native/ocaml_metal_stubs.m:972-985.
int require_buffer_size(const BoundBuffer &buffer, uint64_t required, const char *name);
int require_buffer_count(const DispatchRecord &record, size_t expected);
int require_parameter_bytes(const DispatchRecord &record, size_t expected);
uint32_t param_u32(const DispatchRecord &record, size_t byte_offset);
float param_f32(const DispatchRecord &record, size_t byte_offset);
// Returns device scratch of at least `bytes` (256-byte aligned) or nullptr
// with the error set.
void *context_workspace(llmopt_hip_context *context, size_t bytes);
// Returns the context's zero-initialised arrival counters (allocated on first
// use) or nullptr with the error set.
uint32_t *context_counters(llmopt_hip_context *context, uint32_t *count);
struct RotaryQkArgs;
// RotaryQKParams (the first 28 parameter bytes) and the six rotary buffers (the first six of
// the record), checked as llmopt_rotary_qk_f16_simd_h64 checks them.
int parse_rotary_qk(const DispatchRecord &record, RotaryQkArgs *out);

// Resolves, for the current device, the address of the static scratch array behind
// llmopt_hip_attention_q8_paged_no_alloc (once per device).
int no_alloc_prepare_current_device();

void retain(RefCounted *object);
// Returns true when the caller dropped the last reference.
bool release(RefCounted *object);

int build_record(llmopt_hip_library *library, const llmopt_hip_dispatch_item *item,
                 DispatchRecord *out);
int launch_record(llmopt_hip_context *context, const DispatchRecord &record);
void drop_record(DispatchRecord *record);
// Makes the context's device the calling thread's current one.
int use_device(llmopt_hip_context *context);

}  // namespace llmopt
