// Retained decode plans and the ring queue that feeds one from a worker thread: the HIP
// counterparts of caml_llmopt_prebaked_create / _execute (native/ocaml_metal_stubs.m:1879-2560)
// and caml_llmopt_ring_* (:1465-1877).
//
// The reference freezes a dispatch array once and replays it per token on one serial encoder,
// patching the context length into byte 12 of every llmopt_attention_q8_paged_* parameter block.
// Here the frozen array becomes ONE HIP graph, instantiated at create: the per-step values live
// in device memory that the captured kernels read - the token in the caller's token buffer, the
// context length in a word of the plan that the paged attention launches take instead of
// parameter byte 12 - and a step is one small state launch, one graph launch and a 4-byte
// read-back.  The attention launches are sized for the capacity of their slot table, so the same
// graph serves every step of a sequence.  Buffers the caller updates between steps with
// llmopt_hip_buffer_write / set_int64 / set_u32_array (rotary rows, the new token's slot, the
// per-sequence lengths of the batched extension) are read by the kernels from device memory
// anyway.
#include "kernels/kernels.h"
#include "runtime.h"

#include <pthread.h>
#include <sched.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <memory>
#include <string>

using namespace llmopt;

struct llmopt_hip_prebaked : llmopt::RefCounted {
  llmopt_hip_library *library = nullptr;
  std::vector<DispatchRecord> records;
  std::vector<bool> is_paged_attention;
  // llmopt_cache_pack_checkpoint_q8_simd: byte 0 of its parameter block is the step's checkpoint slot
  // (native/ocaml_metal_stubs.m:1965, 2186-2199)
  std::vector<bool> is_checkpoint_pack;
  uint32_t *device_checkpoint = nullptr;  // the word behind device_past's, when the plan packs a checkpoint
  uint32_t checkpoint = 0;                // of the step being enqueued
  // the highest checkpoint slot every checkpoint pack of the plan has room for in its pool (a retained
  // plan reads the step's slot from device memory, where the launch can only clamp it: the host
  // refuses a step beyond this before anything is queued)
  uint32_t checkpoint_limit = 0xffffffffu;
  llmopt_hip_buffer *token_buffer = nullptr;
  llmopt_hip_buffer *output_buffer = nullptr;
  // context length of the step, one word per sequence of the widest attention record
  uint32_t *device_past = nullptr;
  uint32_t past_count = 0;
  uint32_t past_capacity = 0xffffffffu;  // longest context the captured launches are sized for
  // false: a record cannot be frozen (a masked attention: the mask's row length follows the
  // context) and every step launches the records from the host, as the reference does
  bool single_submission = true;
  hipGraph_t graph = nullptr;
  hipGraphExec_t executable = nullptr;
  uint64_t workspace_generation = 0;
  uint32_t *debug_flag = nullptr;  // device word of the NaN-check replay
};

namespace {

void destroy_graph(llmopt_hip_prebaked *plan) {
  if (plan->executable) (void)hipGraphExecDestroy(plan->executable);
  if (plan->graph) (void)hipGraphDestroy(plan->graph);
  plan->executable = nullptr;
  plan->graph = nullptr;
}

int launch_records(llmopt_hip_prebaked *plan) {
  llmopt_hip_context *context = plan->library->context;
  for (const DispatchRecord &record : plan->records)
    if (int status = launch_record(context, record)) return status;
  return LLMOPT_OK;
}

// Captures the records into plan->graph / plan->executable.  Nothing runs on the GPU.
int capture_plan(llmopt_hip_prebaked *plan) {
  llmopt_hip_context *context = plan->library->context;
  destroy_graph(plan);
  // allocated and cleared outside the capture (kernels that split a tile over workgroups)
  uint32_t counter_count = 0;
  if (context_counters(context, &counter_count) == nullptr) return LLMOPT_ERR_FAILURE;
  for (int attempt = 0; attempt < 2; ++attempt) {
    context->sizing_capture = true;
    context->sizing_wanted = 0;
    if (hipStreamBeginCapture(context->stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
      context->sizing_capture = false;
      return fail(LLMOPT_ERR_FAILURE, "HIP stream capture could not begin");
    }
    int status = launch_records(plan);
    hipGraph_t graph = nullptr;
    const hipError_t ended = hipStreamEndCapture(context->stream, &graph);
    context->sizing_capture = false;
    if (ended != hipSuccess && status == LLMOPT_OK) status = fail(LLMOPT_ERR_FAILURE, "HIP stream capture failed");
    if (status != LLMOPT_OK) {
      if (graph) (void)hipGraphDestroy(graph);
      (void)hipGetLastError();
      return status;
    }
    if (context->sizing_wanted > context->workspace_bytes) {
      // some launch wanted more scratch than the context holds: this capture is void
      (void)hipGraphDestroy(graph);
      if (context_workspace(context, context->sizing_wanted) == nullptr) return LLMOPT_ERR_FAILURE;
      continue;
    }
    plan->graph = graph;
    if (hipGraphInstantiate(&plan->executable, graph, nullptr, nullptr, 0) != hipSuccess) {
      destroy_graph(plan);
      return fail(LLMOPT_ERR_FAILURE, "HIP graph instantiation failed");
    }
    plan->workspace_generation = context->workspace_generation;
    return LLMOPT_OK;
  }
  return fail(LLMOPT_ERR_FAILURE, "prebaked HIP plan could not settle its kernel workspace");
}

// Queues one step on the context's stream: state, records, and the copy of the first int32 of
// the output buffer to `host_token` (pinned memory, or pageable when the caller waits right
// after).  chain: the input token is the output token the previous step left in the output
// buffer (the reference's llmopt_chain_token_id launch).
int enqueue_step(llmopt_hip_prebaked *plan, int64_t token, bool chain, int64_t past_tokens, int32_t *host_token) {
  const uint32_t checkpoint = plan->checkpoint;
  llmopt_hip_context *context = plan->library->context;
  if (int status = use_device(context)) return status;
  if (past_tokens < 0 || (uint64_t)past_tokens > plan->past_capacity)
    return fail(LLMOPT_ERR_INVALID, "prebaked HIP plan holds %u context tokens, step asks for %lld",
                plan->past_capacity, (long long)past_tokens);
  int64_t *token_slot = nullptr;
  if (plan->token_buffer) {
    if (plan->token_buffer->length < 8) return fail(LLMOPT_ERR_INVALID, "buffer offset out of bounds");
    token_slot = reinterpret_cast<int64_t *>(plan->token_buffer->device);
  }
  const int32_t *chain_from = nullptr;
  if (chain) {
    if (plan->output_buffer == nullptr || plan->output_buffer->length < 4 || token_slot == nullptr)
      return fail(LLMOPT_ERR_INVALID, "chained decode step needs a token buffer and an output buffer");
    chain_from = reinterpret_cast<const int32_t *>(plan->output_buffer->device);
  }
  if (plan->single_submission) {
    if (plan->executable == nullptr || plan->workspace_generation != context->workspace_generation)
      if (int status = capture_plan(plan)) return status;
    LLMOPT_HIP_TRY(launch_plan_state(token_slot, token, chain_from, plan->device_past, (uint32_t)past_tokens,
                                     plan->past_count, plan->device_checkpoint, checkpoint, context->stream),
                   "HIP could not write the decode step's state");
    LLMOPT_HIP_TRY(hipGraphLaunch(plan->executable, context->stream), "HIP graph launch failed");
  } else {
    LLMOPT_HIP_TRY(launch_plan_state(token_slot, token, chain_from, nullptr, 0, 0, nullptr, 0, context->stream),
                   "HIP could not write the decode token");
    for (size_t i = 0; i < plan->records.size(); ++i) {
      DispatchRecord &record = plan->records[i];
      if (plan->is_checkpoint_pack[i] && record.parameters.size() >= 4) memcpy(record.parameters.data(), &checkpoint, 4);
      if (plan->is_paged_attention[i] && record.parameters.size() >= 16) {
        const uint32_t past = (uint32_t)past_tokens;
        memcpy(record.parameters.data() + 12, &past, 4);
      }
      if (int status = launch_record(context, record)) {
        (void)hipStreamSynchronize(context->stream);
        return status;
      }
    }
  }
  if (host_token != nullptr) {
    *host_token = 0;
    if (plan->output_buffer && plan->output_buffer->length >= 4)
      LLMOPT_HIP_TRY(hipMemcpyAsync(host_token, plan->output_buffer->device, 4, hipMemcpyDeviceToHost, context->stream),
                     "HIP could not read the decode output");
  }
  return LLMOPT_OK;
}

// ---- debug replays (native/ocaml_metal_stubs.m:2136-2347) ----------------------------------
// LLMOPT_DEBUG_NAN_CHECK (for steps with past_tokens > 0, or every step under
// LLMOPT_CHECK_PREFILL): the records run one at a time, and the first record that leaves a NaN
// in one of its buffers that held none before is reported on stderr.  The reference ends the
// process there; this library returns an error that names the record instead.
// LLMOPT_PROFILE_BREAKDOWN: the records run one at a time between two HIP events each; GPU time
// by kernel name goes to stderr as the reference's table.

bool nan_check_applies(const std::string &name) {
  // integer buffers and packed cache bytes are not floating point (same exclusions as the reference)
  return name.find("_i64") == std::string::npos && name.find("cache_pack") == std::string::npos;
}

int range_has_nan(llmopt_hip_prebaked *plan, const std::string &name, const BoundBuffer &buffer, bool *bad) {
  *bad = false;
  if (buffer.device == nullptr || buffer.length == 0 || !nan_check_applies(name)) return LLMOPT_OK;
  llmopt_hip_context *context = plan->library->context;
  if (plan->debug_flag == nullptr)
    LLMOPT_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&plan->debug_flag), 4), "HIP could not allocate the NaN-check flag");
  const bool f32 = name == "llmopt_matmul" || name.find("_f32") != std::string::npos;
  uint32_t found = 0;
  LLMOPT_HIP_TRY(hipMemsetAsync(plan->debug_flag, 0, 4, context->stream), "HIP could not clear the NaN-check flag");
  LLMOPT_HIP_TRY(launch_nan_scan(buffer.device, buffer.length, f32, plan->debug_flag, context->stream),
                 "HIP could not scan a buffer");
  LLMOPT_HIP_TRY(hipMemcpyAsync(&found, plan->debug_flag, 4, hipMemcpyDeviceToHost, context->stream),
                 "HIP could not read the NaN-check flag");
  LLMOPT_HIP_TRY(hipStreamSynchronize(context->stream), "NaN-check scan failed");
  *bad = found != 0;
  return LLMOPT_OK;
}

int debug_step(llmopt_hip_prebaked *plan, int64_t token, int64_t past_tokens, bool nan_check, int32_t *host_token) {
  llmopt_hip_context *context = plan->library->context;
  if (int status = use_device(context)) return status;
  if (past_tokens < 0 || (uint64_t)past_tokens > plan->past_capacity)
    return fail(LLMOPT_ERR_INVALID, "prebaked HIP plan holds %u context tokens, step asks for %lld",
                plan->past_capacity, (long long)past_tokens);
  int64_t *token_slot = nullptr;
  if (plan->token_buffer) {
    if (plan->token_buffer->length < 8) return fail(LLMOPT_ERR_INVALID, "buffer offset out of bounds");
    token_slot = reinterpret_cast<int64_t *>(plan->token_buffer->device);
  }
  // frozen records read the context length from the plan's device words, the others from byte 12
  LLMOPT_HIP_TRY(launch_plan_state(token_slot, token, nullptr, plan->single_submission ? plan->device_past : nullptr,
                                   (uint32_t)past_tokens, plan->single_submission ? plan->past_count : 0,
                                   plan->single_submission ? plan->device_checkpoint : nullptr, plan->checkpoint,
                                   context->stream),
                 "HIP could not write the decode step's state");
  hipEvent_t before = nullptr, after = nullptr;
  if (!nan_check) {
    LLMOPT_HIP_TRY(hipEventCreate(&before), "HIP event creation failed");
    LLMOPT_HIP_TRY(hipEventCreate(&after), "HIP event creation failed");
  }
  struct Stat { double total_ms = 0.0; size_t count = 0; };
  std::map<std::string, Stat> stats;
  double overall_ms = 0.0;
  int status = LLMOPT_OK;
  if (nan_check)
    fprintf(stderr, "[DEBUG_NAN_CHECK] Starting check across %zu records (past_tokens=%lld)...\n", plan->records.size(),
            (long long)past_tokens);
  for (size_t i = 0; i < plan->records.size() && status == LLMOPT_OK; ++i) {
    DispatchRecord &record = plan->records[i];
    if (!plan->single_submission && plan->is_paged_attention[i] && record.parameters.size() >= 16) {
      const uint32_t past = (uint32_t)past_tokens;
      memcpy(record.parameters.data() + 12, &past, 4);
    }
    if (!plan->single_submission && plan->is_checkpoint_pack[i] && record.parameters.size() >= 4)
      memcpy(record.parameters.data(), &plan->checkpoint, 4);
    std::vector<bool> bad_before(record.buffers.size(), false);
    if (nan_check)
      for (size_t b = 0; b < record.buffers.size() && status == LLMOPT_OK; ++b) {
        bool bad = false;
        status = range_has_nan(plan, record.name, record.buffers[b], &bad);
        bad_before[b] = bad;
      }
    if (status != LLMOPT_OK) break;
    if (!nan_check && hipEventRecord(before, context->stream) != hipSuccess) status = fail(LLMOPT_ERR_FAILURE, "HIP event record failed");
    if (status == LLMOPT_OK) status = launch_record(context, record);
    if (status == LLMOPT_OK && !nan_check && hipEventRecord(after, context->stream) != hipSuccess)
      status = fail(LLMOPT_ERR_FAILURE, "HIP event record failed");
    if (hipStreamSynchronize(context->stream) != hipSuccess && status == LLMOPT_OK)
      status = fail(LLMOPT_ERR_FAILURE, "dispatch %zu '%s' failed on the GPU", i, record.name.c_str());
    if (status != LLMOPT_OK) break;
    if (!nan_check) {
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, before, after) != hipSuccess) ms = 0.0f;
      overall_ms += ms;
      Stat &stat = stats[record.name];
      stat.total_ms += ms;
      stat.count += 1;
      continue;
    }
    for (size_t b = 0; b < record.buffers.size(); ++b) {
      bool bad = false;
      status = range_has_nan(plan, record.name, record.buffers[b], &bad);
      if (status != LLMOPT_OK) break;
      if (!bad || bad_before[b]) continue;
      uint16_t words[16] = {};
      const size_t shown = std::min<size_t>(16, record.buffers[b].length / 2);
      (void)hipMemcpy(words, record.buffers[b].device, shown * 2, hipMemcpyDeviceToHost);
      fprintf(stderr, "\n==================================================\n");
      fprintf(stderr, "[DEBUG_NAN_CHECK] FIRST NaN PRODUCED AT RECORD %zu:\n  kernel: '%s'\n", i, record.name.c_str());
      fprintf(stderr, "  buffer: %zu (length=%zu)\n", b, record.buffers[b].length);
      fprintf(stderr, "  grid: (%lld, %lld, %lld), group: (%lld, %lld, %lld)\n", (long long)record.grid[0],
              (long long)record.grid[1], (long long)record.grid[2], (long long)record.group[0],
              (long long)record.group[1], (long long)record.group[2]);
      if (!record.parameters.empty()) {
        fprintf(stderr, "  parameters (%zu bytes, u32):", record.parameters.size());
        for (size_t p = 0; p + 4 <= record.parameters.size() && p < 48; p += 4) {
          uint32_t word = 0;
          memcpy(&word, record.parameters.data() + p, 4);
          fprintf(stderr, " %u", word);
        }
        fprintf(stderr, "\n");
      }
      fprintf(stderr, "  first 16 half words (hex):");
      for (size_t k = 0; k < shown; ++k) fprintf(stderr, " 0x%04x", words[k]);
      fprintf(stderr, "\n");
      for (size_t other = 0; other < record.buffers.size(); ++other)
        fprintf(stderr, "  buffer[%zu]: len=%zu\n", other, record.buffers[other].length);
      fprintf(stderr, "==================================================\n\n");
      fflush(stderr);
      status = fail(LLMOPT_ERR_FAILURE, "NaN check: record %zu '%s' produced the first NaN, in buffer %zu", i,
                    record.name.c_str(), b);
      break;
    }
  }
  if (before) (void)hipEventDestroy(before);
  if (after) (void)hipEventDestroy(after);
  if (status != LLMOPT_OK) return status;
  if (!nan_check) {
    std::vector<std::pair<std::string, Stat>> order(stats.begin(), stats.end());
    std::stable_sort(order.begin(), order.end(),
                     [](const auto &a, const auto &b) { return a.second.total_ms > b.second.total_ms; });
    fprintf(stderr, "\n========== DECODE KERNEL BREAKDOWN (past_tokens=%lld) ==========\n", (long long)past_tokens);
    fprintf(stderr, "%-48s | %5s | %10s | %10s | %6s\n", "Kernel Name", "Calls", "Total (ms)", "Avg (us)", "Pct");
    fprintf(stderr, "-------------------------------------------------+-------+------------+------------+-------\n");
    for (const auto &entry : order)
      fprintf(stderr, "%-48s | %5zu | %10.3f | %10.2f | %5.1f%%\n", entry.first.c_str(), entry.second.count,
              entry.second.total_ms, entry.second.total_ms / entry.second.count * 1000.0,
              overall_ms > 0 ? entry.second.total_ms / overall_ms * 100.0 : 0.0);
    fprintf(stderr, "-------------------------------------------------+-------+------------+------------+-------\n");
    fprintf(stderr, "%-48s | %5zu | %10.3f |            | 100.0%%\n", "TOTAL DISPATCHES", plan->records.size(), overall_ms);
    fprintf(stderr, "===============================================================\n\n");
    fflush(stderr);
  }
  *host_token = 0;
  if (plan->output_buffer && plan->output_buffer->length >= 4)
    LLMOPT_HIP_TRY(hipMemcpy(host_token, plan->output_buffer->device, 4, hipMemcpyDeviceToHost),
                   "HIP could not read the decode output");
  return LLMOPT_OK;
}

bool is_reference_paged_attention(const char *name) {
  static const char prefix[] = "llmopt_attention_q8_paged_";
  // the batched extension keeps its lengths in a caller-owned device buffer: nothing to patch
  return strncmp(name, prefix, sizeof prefix - 1) == 0 && strcmp(name, "llmopt_attention_q8_paged_batched") != 0;
}

}  // namespace

extern "C" {

int llmopt_hip_prebaked_create(llmopt_hip_library *library, const llmopt_hip_dispatch_item *items, size_t count,
                               llmopt_hip_buffer *token_buffer, llmopt_hip_buffer *output_buffer,
                               llmopt_hip_prebaked **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "plan output pointer is null");
  *out = nullptr;
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  if (count == 0 || items == nullptr)
    return fail(LLMOPT_ERR_INVALID, "prebaked HIP plan requires at least one dispatch");
  for (size_t i = 0; i < count; ++i) {
    if (items[i].buffer_count > 16) return fail(LLMOPT_ERR_INVALID, "prebaked HIP dispatch exceeds 16 buffers");
    if (items[i].parameter_bytes > 256)
      return fail(LLMOPT_ERR_INVALID, "prebaked HIP dispatch parameters exceed 256 bytes");
  }
  llmopt_hip_context *context = library->context;
  if (int status = use_device(context)) return status;
  llmopt_hip_prebaked *plan = new llmopt_hip_prebaked();
  plan->library = library;
  retain(library);
  if (token_buffer) {
    plan->token_buffer = token_buffer;
    retain(token_buffer);
  }
  if (output_buffer) {
    plan->output_buffer = output_buffer;
    retain(output_buffer);
  }
  plan->records.resize(count);
  int status = LLMOPT_OK;
  for (size_t i = 0; i < count && status == LLMOPT_OK; ++i) {
    status = build_record(library, &items[i], &plan->records[i]);
    if (status != LLMOPT_OK) break;
    const bool paged = is_reference_paged_attention(items[i].name);
    plan->is_paged_attention.push_back(paged);
    plan->is_checkpoint_pack.push_back(strcmp(items[i].name, "llmopt_cache_pack_checkpoint_q8_simd") == 0);
    const DispatchRecord &record = plan->records[i];
    if (plan->is_checkpoint_pack[i] && record.parameters.size() >= 28 && record.buffers.size() >= 2) {
      // CheckpointCacheParams: checkpoint_stride at byte 24; buffers: source, pool
      const uint32_t stride = param_u32(record, 24);
      const uint64_t slots = stride != 0 ? record.buffers[1].length / stride : 0;
      plan->checkpoint_limit = (uint32_t)std::min<uint64_t>(plan->checkpoint_limit, slots != 0 ? slots - 1 : 0);
    }
    if (!paged || record.parameters.size() < 64 || record.buffers.size() < 7) continue;
    plan->past_count = std::max(plan->past_count, param_u32(record, 0));
    if (param_u32(record, 20) != 0 && param_u32(record, 56) != 0) plan->single_submission = false;  // masked
    // the launch is sized for what the slot table can hold, up to the split kernels' limit
    const uint64_t slots = record.buffers[4].length / 4;
    plan->past_capacity = (uint32_t)std::min<uint64_t>(plan->past_capacity, std::min<uint64_t>(slots, kQ8AttentionSplitTokens));
  }
  plan->is_paged_attention.resize(count, false);
  plan->is_checkpoint_pack.resize(count, false);
  if (status == LLMOPT_OK && plan->single_submission) {
    const uint32_t past_words = std::max<uint32_t>(plan->past_count, 1);
    const uint32_t words = past_words + 1;  // the step's checkpoint slot behind the context lengths
    void *block = nullptr;
    if (hipMalloc(&block, (size_t)words * 4) != hipSuccess || hipMemset(block, 0, (size_t)words * 4) != hipSuccess) {
      if (block) (void)hipFree(block);
      status = fail(LLMOPT_ERR_FAILURE, "HIP could not allocate the plan's step state");
    } else {
      plan->device_past = static_cast<uint32_t *>(block);
      for (size_t i = 0; i < count; ++i) {
        if (plan->is_paged_attention[i]) {
          plan->records[i].device_past_lengths = plan->device_past;
          plan->records[i].device_past_capacity = plan->past_capacity;
        }
        if (plan->is_checkpoint_pack[i]) {
          plan->device_checkpoint = plan->device_past + past_words;
          plan->records[i].device_checkpoint = plan->device_checkpoint;
        }
      }
      status = capture_plan(plan);
    }
  }
  if (status != LLMOPT_OK) {
    llmopt_hip_release_prebaked(plan);
    return status;
  }
  *out = plan;
  return LLMOPT_OK;
}

void llmopt_hip_release_prebaked(llmopt_hip_prebaked *plan) {
  if (!release(plan)) return;
  llmopt_hip_context *context = plan->library->context;
  (void)hipSetDevice(context->device);
  (void)hipStreamSynchronize(context->stream);
  destroy_graph(plan);
  if (plan->device_past) (void)hipFree(plan->device_past);
  if (plan->debug_flag) (void)hipFree(plan->debug_flag);
  for (DispatchRecord &record : plan->records) drop_record(&record);
  if (plan->token_buffer) llmopt_hip_release_buffer(plan->token_buffer);
  if (plan->output_buffer) llmopt_hip_release_buffer(plan->output_buffer);
  llmopt_hip_release_library(plan->library);
  delete plan;
}

int llmopt_hip_prebaked_execute(llmopt_hip_prebaked *plan, int64_t token, int64_t past_tokens, int64_t checkpoint,
                                int64_t *out_token) {
  if (plan == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP prebaked plan has been finalized");
  // the slot llmopt_cache_pack_checkpoint_q8_simd launches of the plan write this step (as the reference:
  // the low 32 bits of the argument; the ring queue has no such argument and keeps the last one)
  if (plan->checkpoint_limit != 0xffffffffu && (uint32_t)(int32_t)checkpoint > plan->checkpoint_limit)
    return fail(LLMOPT_ERR_INVALID, "HIP checkpoint pool buffer is too small: the plan's pools hold checkpoints 0..%u, step asks for %u",
                plan->checkpoint_limit, (uint32_t)(int32_t)checkpoint);
  plan->checkpoint = (uint32_t)(int32_t)checkpoint;
  int32_t next_token = 0;
  const bool nan_check =
      getenv("LLMOPT_DEBUG_NAN_CHECK") != nullptr && (past_tokens > 0 || getenv("LLMOPT_CHECK_PREFILL") != nullptr);
  if (nan_check || getenv("LLMOPT_PROFILE_BREAKDOWN") != nullptr) {
    if (int status = debug_step(plan, token, past_tokens, nan_check, &next_token)) return status;
    if (out_token) *out_token = (int64_t)next_token;
    return LLMOPT_OK;
  }
  if (int status = enqueue_step(plan, token, false, past_tokens, &next_token)) return status;
  if (hipStreamSynchronize(plan->library->context->stream) != hipSuccess)
    return fail(LLMOPT_ERR_FAILURE, "Prebaked HIP batch failed");
  if (out_token) *out_token = (int64_t)next_token;
  return LLMOPT_OK;
}

int llmopt_hip_prebaked_is_single_submission(llmopt_hip_prebaked *plan) {
  if (plan == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP prebaked plan has been finalized");
  return plan->single_submission && plan->executable != nullptr ? 1 : 0;
}

}  // extern "C"

// ---- ring queue -----------------------------------------------------------------------------
// A submission queue and a completion queue of 256 entries each between one submitting thread
// and one worker thread (single producer, single consumer on both, as in the reference).  The
// worker runs one decode step per submission: through a retained plan (start_worker), or
// through a host function (start_worker_with: other executors, and the queue's own tests).

namespace {
constexpr uint32_t kRingCapacity = 256;  // LLMOPT_RING_CAPACITY

struct Submission {
  uint32_t request_id;
  int32_t token;
  int32_t past_tokens;
  uint32_t flags;
};
struct Completion {
  uint32_t request_id;
  int32_t token;
  uint32_t status;
};
}  // namespace

struct llmopt_hip_ring {
  std::atomic<uint32_t> sq_head{0}, sq_tail{0}, cq_head{0}, cq_tail{0};
  Submission sq[kRingCapacity];
  Completion cq[kRingCapacity];
  pthread_mutex_t mutex;
  pthread_cond_t sq_cond, cq_cond;
  std::atomic<uint32_t> running{1};
  pthread_t worker;
  bool worker_started = false;
  // executor
  llmopt_hip_prebaked *plan = nullptr;
  llmopt_hip_ring_step step = nullptr;
  void *step_user = nullptr;
  int depth = 1;
  // steps queued on the GPU whose completion is not posted yet (depth > 1)
  int32_t *host_tokens = nullptr;  // pinned, one per slot
  hipEvent_t events[2] = {nullptr, nullptr};
};

namespace {

void post_completion(llmopt_hip_ring *q, uint32_t request_id, int32_t token, uint32_t status) {
  const uint32_t tail = q->cq_tail.load(std::memory_order_relaxed);
  q->cq[tail % kRingCapacity] = {request_id, token, status};
  q->cq_tail.store(tail + 1, std::memory_order_release);
  pthread_mutex_lock(&q->mutex);
  pthread_cond_signal(&q->cq_cond);
  pthread_mutex_unlock(&q->mutex);
}

struct Pending {
  bool valid = false;
  Submission entry;
  int slot = 0;
  int status = LLMOPT_OK;
};

void finish_pending(llmopt_hip_ring *q, Pending *pending) {
  if (!pending->valid) return;
  int32_t token = 0;
  uint32_t status = pending->status == LLMOPT_OK ? 0 : 1;
  if (status == 0) {
    if (q->plan != nullptr) {
      if (hipEventSynchronize(q->events[pending->slot]) != hipSuccess) status = 1;
      token = q->host_tokens[pending->slot];
    } else {
      token = q->host_tokens ? q->host_tokens[pending->slot] : 0;
    }
  }
  post_completion(q, pending->entry.request_id, token, status);
  pending->valid = false;
}

void *ring_worker(void *argument) {
  llmopt_hip_ring *q = static_cast<llmopt_hip_ring *>(argument);
  if (q->plan != nullptr) (void)hipSetDevice(q->plan->library->context->device);
  Pending previous;
  int32_t callback_tokens[2] = {0, 0};
  if (q->plan == nullptr) q->host_tokens = callback_tokens;
  while (q->running.load(std::memory_order_acquire)) {
    const uint32_t head = q->sq_head.load(std::memory_order_relaxed);
    uint32_t tail = q->sq_tail.load(std::memory_order_acquire);
    if (head == tail) {
      bool found = false;
      for (int i = 0; i < 1000 && !found; ++i) {
        tail = q->sq_tail.load(std::memory_order_acquire);
        found = head != tail;
        if (!found) sched_yield();
      }
      if (!found) {
        finish_pending(q, &previous);  // nothing to overlap it with
        pthread_mutex_lock(&q->mutex);
        while (q->sq_head.load(std::memory_order_relaxed) == q->sq_tail.load(std::memory_order_relaxed) &&
               q->running.load(std::memory_order_relaxed))
          pthread_cond_wait(&q->sq_cond, &q->mutex);
        pthread_mutex_unlock(&q->mutex);
        continue;
      }
    }
    const Submission entry = q->sq[head % kRingCapacity];
    q->sq_head.store(head + 1, std::memory_order_release);
    if (entry.flags == 2 || !q->running.load(std::memory_order_relaxed)) break;
    const int slot = (int)(head % 2);
    Pending current;
    current.valid = true;
    current.entry = entry;
    current.slot = slot;
    if (q->plan != nullptr) {
      // a negative token chains: the step reads the token the previous step produced, on the GPU
      current.status = enqueue_step(q->plan, entry.token, entry.token < 0, entry.past_tokens, &q->host_tokens[slot]);
      if (current.status == LLMOPT_OK &&
          hipEventRecord(q->events[slot], q->plan->library->context->stream) != hipSuccess)
        current.status = LLMOPT_ERR_FAILURE;
    } else {
      // host executor: a chained step needs the previous token now
      int64_t token = entry.token;
      if (entry.token < 0) {
        const int last = slot ^ 1;
        token = callback_tokens[last];
      }
      current.status = q->step(q->step_user, token, entry.past_tokens, &callback_tokens[slot]);
    }
    if (q->depth <= 1) {
      finish_pending(q, &current);
    } else {
      finish_pending(q, &previous);  // its successor is queued behind it already
      previous = current;
    }
  }
  finish_pending(q, &previous);
  if (q->plan == nullptr) q->host_tokens = nullptr;
  return nullptr;
}

int ring_depth_from_environment() {
  const char *text = getenv("LLMOPT_QUEUE_DEPTH");
  const int depth = text ? atoi(text) : 1;
  return depth >= 1 ? depth : 1;
}

int start_thread(llmopt_hip_ring *ring) {
  ring->depth = ring_depth_from_environment();
  ring->running.store(1, std::memory_order_release);
  if (pthread_create(&ring->worker, nullptr, ring_worker, ring) != 0)
    return fail(LLMOPT_ERR_FAILURE, "ring queue worker thread could not start");
  ring->worker_started = true;
  return LLMOPT_OK;
}

}  // namespace

extern "C" {

int llmopt_hip_ring_create(llmopt_hip_ring **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "ring output pointer is null");
  llmopt_hip_ring *ring = new llmopt_hip_ring();
  pthread_mutex_init(&ring->mutex, nullptr);
  pthread_cond_init(&ring->sq_cond, nullptr);
  pthread_cond_init(&ring->cq_cond, nullptr);
  *out = ring;
  return LLMOPT_OK;
}

int llmopt_hip_ring_submit(llmopt_hip_ring *ring, int64_t request_id, int64_t token, int64_t past_tokens,
                           int64_t flags) {
  if (ring == nullptr) return fail(LLMOPT_ERR_FAILURE, "ring queue has been finalized");
  const uint32_t tail = ring->sq_tail.load(std::memory_order_relaxed);
  const uint32_t head = ring->sq_head.load(std::memory_order_acquire);
  if (tail - head >= kRingCapacity) return 0;
  ring->sq[tail % kRingCapacity] = {(uint32_t)request_id, (int32_t)token, (int32_t)past_tokens, (uint32_t)flags};
  ring->sq_tail.store(tail + 1, std::memory_order_release);
  pthread_mutex_lock(&ring->mutex);
  pthread_cond_signal(&ring->sq_cond);
  pthread_mutex_unlock(&ring->mutex);
  return 1;
}

static int take_completion(llmopt_hip_ring *ring, int64_t *request_id, int64_t *token, int64_t *status) {
  const uint32_t head = ring->cq_head.load(std::memory_order_relaxed);
  const uint32_t tail = ring->cq_tail.load(std::memory_order_acquire);
  if (head == tail) return 0;
  const Completion entry = ring->cq[head % kRingCapacity];
  ring->cq_head.store(head + 1, std::memory_order_release);
  if (request_id) *request_id = entry.request_id;
  if (token) *token = entry.token;
  if (status) *status = entry.status;
  return 1;
}

int llmopt_hip_ring_wait_completion(llmopt_hip_ring *ring, int64_t *request_id, int64_t *token, int64_t *status) {
  if (ring == nullptr) return fail(LLMOPT_ERR_FAILURE, "ring queue has been finalized");
  if (ring->cq_head.load(std::memory_order_relaxed) == ring->cq_tail.load(std::memory_order_acquire)) {
    pthread_mutex_lock(&ring->mutex);
    while (ring->cq_head.load(std::memory_order_relaxed) == ring->cq_tail.load(std::memory_order_relaxed) &&
           ring->running.load(std::memory_order_relaxed))
      pthread_cond_wait(&ring->cq_cond, &ring->mutex);
    pthread_mutex_unlock(&ring->mutex);
  }
  if (take_completion(ring, request_id, token, status) == 0)
    return fail(LLMOPT_ERR_FAILURE, "Ring queue terminated with no completion");
  return LLMOPT_OK;
}

int llmopt_hip_ring_poll_completion(llmopt_hip_ring *ring, int64_t *request_id, int64_t *token, int64_t *status) {
  if (ring == nullptr) return fail(LLMOPT_ERR_FAILURE, "ring queue has been finalized");
  return take_completion(ring, request_id, token, status);
}

int llmopt_hip_ring_start_worker(llmopt_hip_ring *ring, llmopt_hip_library *library,
                                 const llmopt_hip_dispatch_item *items, size_t count, llmopt_hip_buffer *token_buffer,
                                 llmopt_hip_buffer *output_buffer) {
  if (ring == nullptr) return fail(LLMOPT_ERR_FAILURE, "ring queue has been finalized");
  if (ring->worker_started) return fail(LLMOPT_ERR_INVALID, "ring queue worker is already running");
  if (int status = llmopt_hip_prebaked_create(library, items, count, token_buffer, output_buffer, &ring->plan))
    return status;
  void *pinned = nullptr;
  if (hipHostMalloc(&pinned, 2 * sizeof(int32_t), hipHostMallocDefault) != hipSuccess ||
      hipEventCreateWithFlags(&ring->events[0], hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&ring->events[1], hipEventDisableTiming) != hipSuccess) {
    if (pinned) (void)hipHostFree(pinned);
    return fail(LLMOPT_ERR_FAILURE, "ring queue could not allocate its read-back slots");
  }
  ring->host_tokens = static_cast<int32_t *>(pinned);
  return start_thread(ring);
}

int llmopt_hip_ring_start_worker_with(llmopt_hip_ring *ring, llmopt_hip_ring_step step, void *user) {
  if (ring == nullptr) return fail(LLMOPT_ERR_FAILURE, "ring queue has been finalized");
  if (step == nullptr) return fail(LLMOPT_ERR_INVALID, "ring queue step function is null");
  if (ring->worker_started) return fail(LLMOPT_ERR_INVALID, "ring queue worker is already running");
  ring->step = step;
  ring->step_user = user;
  return start_thread(ring);
}

void llmopt_hip_ring_destroy(llmopt_hip_ring *ring) {
  if (ring == nullptr) return;
  ring->running.store(0, std::memory_order_release);
  pthread_mutex_lock(&ring->mutex);
  pthread_cond_broadcast(&ring->sq_cond);
  pthread_cond_broadcast(&ring->cq_cond);
  pthread_mutex_unlock(&ring->mutex);
  if (ring->worker_started) pthread_join(ring->worker, nullptr);
  if (ring->plan != nullptr) {
    llmopt_hip_release_prebaked(ring->plan);
    if (ring->host_tokens) (void)hipHostFree(ring->host_tokens);
    for (hipEvent_t event : ring->events)
      if (event) (void)hipEventDestroy(event);
  }
  pthread_mutex_destroy(&ring->mutex);
  pthread_cond_destroy(&ring->sq_cond);
  pthread_cond_destroy(&ring->cq_cond);
  delete ring;
}

}  // extern "C"
