// The one entry point of this library that allocates nothing, for callers that cannot: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// llmopt_hip_attention_q8_paged_no_alloc is llmopt_attention_q8_paged_simd_* (one slot table,
// no mask) with plain device pointers instead of buffer handles.  The split-context kernels
// keep their partial results - per (KV head, chunk): running maximum, denominator and the
// unnormalised weighted sum of the head group - in scratch memory; the dispatch entry takes it
// from the context's growable workspace, this one from a fixed array in the code object.
//
// Every call on a GPU shares that GPU's array, and the array keeps the last call's contents.
// Nothing in it has to start at zero: the merge kernel reads exactly the partial results the
// split kernel of the same call wrote (both derive the chunk layout from the same arguments).
// Two calls that overlap in time on one GPU (different streams, or different threads) race on
// the array; calls on one stream are ordered and safe.
#include "../../include/llmopt_hip.h"
#include "kernels/kernels.h"
#include "runtime.h"

#include <string.h>

static __device__ __align__(256) unsigned char scratch[LLMOPT_NO_ALLOC_SCRATCH_BYTES];

namespace llmopt {
namespace {

constexpr int kMaxDevices = 64;
// Address of `scratch` on each device: the array's name is only a host-side handle, and every
// GPU holds its own copy at its own address.
void *g_scratch_address[kMaxDevices] = {};

int scratch_of_current_device(void **out) {
  int device = 0;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return fail_hip(status, "HIP could not name the current device");
  if (device < 0 || device >= kMaxDevices)
    return fail(LLMOPT_ERR_FAILURE, "HIP device index %d is beyond the %d this entry point serves", device,
                kMaxDevices);
  void *address = __atomic_load_n(&g_scratch_address[device], __ATOMIC_ACQUIRE);
  if (address == nullptr) {
    status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (status != hipSuccess || address == nullptr)
      return fail_hip(status, "HIP could not resolve the static attention scratch");
    __atomic_store_n(&g_scratch_address[device], address, __ATOMIC_RELEASE);
  }
  *out = address;
  return LLMOPT_OK;
}

uint32_t word(const uint8_t *parameters, size_t byte_offset) {
  uint32_t value = 0;
  memcpy(&value, parameters + byte_offset, 4);
  return value;
}

}  // namespace

int no_alloc_prepare_current_device() {
  void *address = nullptr;
  return scratch_of_current_device(&address);
}

}  // namespace llmopt

using namespace llmopt;

extern "C" int llmopt_hip_attention_q8_paged_no_alloc(void *hip_stream, const void *parameters,
                                                      const void *query, const void *current_key,
                                                      const void *current_value, const void *pool,
                                                      size_t pool_bytes, const uint32_t *slots,
                                                      size_t slot_count, void *output) {
  static const char name[] = "llmopt_hip_attention_q8_paged_no_alloc";
  if (parameters == nullptr || query == nullptr || current_key == nullptr || current_value == nullptr ||
      output == nullptr)
    return fail(LLMOPT_ERR_INVALID, "%s received a null pointer", name);
  const uint8_t *p = static_cast<const uint8_t *>(parameters);
  Q8AttentionArgs args = {};
  args.batches = word(p, 0);
  args.query_heads = word(p, 4);
  args.kv_heads = word(p, 8);
  args.past_length = word(p, 12);
  args.head_dim = word(p, 16);
  args.mask_batches = word(p, 20);
  args.mask_heads = word(p, 24);
  args.token_elements = word(p, 28);
  args.key_offset = word(p, 32);
  args.value_offset = word(p, 36);
  const uint32_t group_size = word(p, 40);
  args.token_stride = word(p, 44);
  memcpy(&args.scale, p + 48, 4);
  args.query_length = word(p, 52);
  args.mask_dtype = word(p, 56);
  args.window = word(p, 60);
  args.max_past_length = args.past_length;
  if (group_size != 64) return fail(LLMOPT_ERR_INVALID, "%s supports the Q8 group size 64 only, got %u", name, group_size);
  if (args.head_dim == 0 || args.head_dim % 64 != 0 || args.head_dim > 512)
    return fail(LLMOPT_ERR_INVALID, "%s requires head_dim to be a multiple of 64 up to 512", name);
  if (args.token_elements % 64 != 0 ||
      args.token_stride < args.token_elements + 2 * (args.token_elements / 64))
    return fail(LLMOPT_ERR_INVALID, "%s received an inconsistent Q8 token layout", name);
  if (args.batches == 0 || args.kv_heads == 0 || args.query_heads == 0 || args.query_heads % args.kv_heads != 0)
    return fail(LLMOPT_ERR_INVALID, "%s requires query heads to be a multiple of kv heads", name);
  const uint64_t segment = (uint64_t)args.kv_heads * args.head_dim;
  if (args.key_offset % 64 != 0 || args.value_offset % 64 != 0 ||
      args.key_offset + segment > args.token_elements || args.value_offset + segment > args.token_elements)
    return fail(LLMOPT_ERR_INVALID, "%s K/V segments lie outside the token", name);
  if (args.mask_batches != 0 && args.mask_dtype != 0) return fail(LLMOPT_ERR_INVALID, "%s does not take a mask", name);
  if (args.past_length > 0) {
    if (pool == nullptr || slots == nullptr) return fail(LLMOPT_ERR_INVALID, "%s received a null pointer", name);
    if (pool_bytes < args.token_stride)
      return fail(LLMOPT_ERR_INVALID, "HIP pool buffer is too small: required=%llu actual=%llu",
                  (unsigned long long)args.token_stride, (unsigned long long)pool_bytes);
    if (slot_count < args.past_length)
      return fail(LLMOPT_ERR_INVALID, "HIP slots buffer is too small: required=%llu actual=%llu",
                  (unsigned long long)args.past_length * 4, (unsigned long long)slot_count * 4);
  }
  args.query = static_cast<const uint16_t *>(query);
  args.current_key = static_cast<const uint16_t *>(current_key);
  args.current_value = static_cast<const uint16_t *>(current_value);
  args.pool = static_cast<const uint8_t *>(pool);
  args.pool_bytes = pool_bytes;
  args.slots = slots;
  args.output = static_cast<uint16_t *>(output);
  const size_t wanted = q8_attention_workspace_bytes(args);
  if (wanted > (size_t)LLMOPT_NO_ALLOC_SCRATCH_BYTES)
    return fail(LLMOPT_ERR_INVALID,
                "%s: %zu bytes of partial results exceed the static scratch of %u bytes "
                "(fewer sequences, KV heads or context tokens per call)",
                name, wanted, (unsigned)LLMOPT_NO_ALLOC_SCRATCH_BYTES);
  if (wanted > 0) {
    void *address = nullptr;
    if (int status = scratch_of_current_device(&address)) return status;
    args.workspace = address;
    args.workspace_bytes = wanted;
  }
  const hipError_t status = launch_q8_attention(args, static_cast<hipStream_t>(hip_stream));
  if (status != hipSuccess) return fail(LLMOPT_ERR_FAILURE, "%s launch failed: %s", name, hipGetErrorString(status));
  return LLMOPT_OK;
}
