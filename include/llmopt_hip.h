/*
 * llmopt_hip.h - flat C ABI of the MI355X (gfx950) backend for llmopt's
 * quantized-inference hot path.
 *
 * This is the boundary the reference crosses in lib/metal_native.ml:8-124
 * (`external ... = "caml_llmopt_metal_*"`, implemented for Apple GPUs in
 * native/ocaml_metal_stubs.m).  Every entry point below names the reference
 * symbol it stands in for.  The OCaml-value calling convention of the
 * reference is not part of this header: a thin CAMLprim shim unpacks OCaml
 * values, calls these functions and turns a non-zero status into `Failure` /
 * `Invalid_argument` carrying llmopt_hip_last_error().
 *
 * Conventions
 *  - Every function returns LLMOPT_OK (0) or a negative status; the message of
 *    the last failure on the calling thread is llmopt_hip_last_error().
 *    LLMOPT_ERR_INVALID corresponds to the reference's caml_invalid_argument,
 *    LLMOPT_ERR_FAILURE to caml_failwith (lib/metal_native.ml:126-129 maps
 *    both to `Error message`).
 *  - Kernels are addressed by the reference's entry-point names
 *    (Kernel_abi.Entry.name, lib/kernel_abi.ml:112-119), buffers are bound
 *    positionally in the reference's order and the parameter block is the
 *    reference's packed little-endian byte layout (lib/metal_parameters.ml).
 *  - grid is the reference's *thread* count (Metal dispatchThreads,
 *    native/ocaml_metal_stubs.m:1205) and group its threadgroup size.  They are
 *    validated (> 0) as the reference does but the launch geometry on gfx950 is
 *    derived from the parameter block, not from them.
 *  - One caller thread per context; work is ordered on the context's HIP stream
 *    (the reference encodes into one serial compute encoder,
 *    native/ocaml_metal_stubs.m:2473-2492).
 */
#ifndef LLMOPT_HIP_H
#define LLMOPT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLMOPT_OK 0
#define LLMOPT_ERR_FAILURE (-1) /* reference: caml_failwith */
#define LLMOPT_ERR_INVALID (-2) /* reference: caml_invalid_argument */

typedef struct llmopt_hip_context llmopt_hip_context;
typedef struct llmopt_hip_library llmopt_hip_library;
typedef struct llmopt_hip_buffer llmopt_hip_buffer;
typedef struct llmopt_hip_batch llmopt_hip_batch;
typedef struct llmopt_hip_prebaked llmopt_hip_prebaked;
typedef struct llmopt_hip_ring llmopt_hip_ring;

/* One recorded dispatch: the tuple of lib/metal_native.ml:61-65 and :117-124
 * (name, buffers, parameter bytes, grid xyz, threadgroup xyz, barrier flag). */
typedef struct llmopt_hip_dispatch_item {
  const char *name;
  llmopt_hip_buffer *const *buffers;
  uint32_t buffer_count;
  const void *parameters;
  uint32_t parameter_bytes;
  int64_t grid[3];
  int64_t group[3];
  int32_t barrier_before;
} llmopt_hip_dispatch_item;

/* Message of the last failed call on this thread ("" if none). */
const char *llmopt_hip_last_error(void);

/* ---- context / library ------------------------------------------------- */

/* caml_llmopt_metal_create_context (native/ocaml_metal_stubs.m:410-432).
 * device < 0 selects the current HIP device. */
int llmopt_hip_create_context(int device, llmopt_hip_context **out);
void llmopt_hip_release_context(llmopt_hip_context *context);

/* caml_llmopt_metal_device_name (:434-445); writes a NUL-terminated name. */
int llmopt_hip_device_name(llmopt_hip_context *context, char *out, size_t capacity);

/* Runs later work of this context on an existing HIP stream (hipStream_t
 * passed as void*), e.g. PyTorch's current stream.  No reference counterpart:
 * Metal command queues are private to the context. */
int llmopt_hip_context_set_stream(llmopt_hip_context *context, void *hip_stream);
/* Blocks until all work queued on the context's stream has finished. */
int llmopt_hip_context_synchronize(llmopt_hip_context *context);

/* caml_llmopt_metal_load_library (:613-665).  The gfx950 kernels are linked
 * into this shared library; `path` (the package's kernel artefact) is recorded
 * but not read, and may be NULL. */
int llmopt_hip_load_library(llmopt_hip_context *context, const char *path,
                            llmopt_hip_library **out);
void llmopt_hip_release_library(llmopt_hip_library *library);

/* caml_llmopt_metal_has_function (:667-682): 1 if the entry-point name is
 * implemented, 0 if not, negative on error. */
int llmopt_hip_has_function(llmopt_hip_library *library, const char *name);

/* caml_llmopt_metal_preload_pipeline (:1087-1098): fails with "... does not
 * contain the selected kernel" for an unknown name. */
int llmopt_hip_preload_pipeline(llmopt_hip_library *library, const char *name);

/* Number of implemented entry points and the i-th name (for package checks,
 * lib/metal_native.ml:271-284). */
int llmopt_hip_function_count(llmopt_hip_library *library);
const char *llmopt_hip_function_name(llmopt_hip_library *library, int index);

/* ---- buffers ------------------------------------------------------------ */

/* caml_llmopt_metal_buffer_of_bytes (:684-715): length 0 is invalid. */
int llmopt_hip_buffer_of_bytes(llmopt_hip_context *context, const void *bytes, size_t length,
                               llmopt_hip_buffer **out);
/* caml_llmopt_metal_create_buffer (:717-748): zero-filled; bytes <= 0 gives a
 * 16-byte buffer. */
int llmopt_hip_create_buffer(llmopt_hip_context *context, int64_t bytes, llmopt_hip_buffer **out);
/* caml_llmopt_metal_map_file (:863-943): the whole file becomes one device
 * buffer (tensor payloads keep their 256-byte alignment). */
int llmopt_hip_map_file(llmopt_hip_context *context, const char *path, llmopt_hip_buffer **out);
/* caml_llmopt_metal_buffer_view (:945-970): shares and retains the parent. */
int llmopt_hip_buffer_view(llmopt_hip_buffer *parent, int64_t offset, int64_t length,
                           llmopt_hip_buffer **out);
/* Wraps device memory owned by someone else (a PyTorch tensor); never freed
 * here.  No reference counterpart. */
int llmopt_hip_buffer_wrap(llmopt_hip_context *context, void *device_pointer, size_t length,
                           llmopt_hip_buffer **out);
void llmopt_hip_release_buffer(llmopt_hip_buffer *buffer);

/* caml_llmopt_metal_buffer_contents (:750-762): copies the whole buffer out
 * after draining the stream; capacity must be >= the buffer length. */
int llmopt_hip_buffer_contents(llmopt_hip_buffer *buffer, void *out, size_t capacity);
/* caml_llmopt_metal_buffer_length (:798-805); negative on error. */
int64_t llmopt_hip_buffer_length(llmopt_hip_buffer *buffer);
/* Device address of the first byte (for interop). */
void *llmopt_hip_buffer_device_pointer(llmopt_hip_buffer *buffer);
/* caml_llmopt_metal_buffer_copy (:807-822): lengths must be equal. */
int llmopt_hip_buffer_copy(llmopt_hip_buffer *source, llmopt_hip_buffer *destination);
/* Writes host bytes at a byte offset (the reference's engines write shared
 * memory directly; device memory needs an explicit upload). */
int llmopt_hip_buffer_write(llmopt_hip_buffer *buffer, int64_t offset, const void *bytes,
                            size_t length);
/* caml_llmopt_metal_buffer_set_int64 (:824-840). */
int llmopt_hip_buffer_set_int64(llmopt_hip_buffer *buffer, int64_t offset, int64_t value);
/* caml_llmopt_metal_buffer_set_u32_array (:842-861): values are OCaml ints
 * truncated to uint32. */
int llmopt_hip_buffer_set_u32_array(llmopt_hip_buffer *buffer, int64_t offset,
                                    const int64_t *values, size_t count);
/* caml_llmopt_metal_buffer_argmax_f16 (:764-796): argmax over the LAST row of
 * `vocabulary` fp16 logits; ties go to the lowest index. */
int llmopt_hip_buffer_argmax_f16(llmopt_hip_buffer *buffer, int64_t vocabulary, int64_t *out);

/* ---- host-side token selection --------------------------------------------- */

/* caml_llmopt_f16_argmax (native/ocaml_metal_stubs.m:2565-2579): index of the
 * first maximum of `count` fp16 logits in host memory (0 for an empty row). */
int llmopt_hip_f16_argmax(const uint16_t *logits, int64_t count, int64_t *out_index);
/* caml_llmopt_sample_f16_native (native/ocaml_metal_stubs.m:2629-2765; called by
 * Sampling.sample, lib/sampling.ml:193-207, on the last logits row in host memory):
 * greedy when temperature <= 1e-4 or top_k == 1; else top-k (0 -> 64, at most 256)
 * by a bounded min-heap, float32 softmax with temperature, min-p, top-p, and one
 * draw from xoroshiro128+ seeded with `seed` (0 = from the clock).  Same float32
 * operation order and tie handling as the reference: a seed gives the same token. */
int llmopt_hip_sample_f16(const uint16_t *logits, int64_t count, double temperature, int64_t top_k,
                          double top_p, double min_p, int64_t seed, int64_t *out_token);

/* ---- dispatch ------------------------------------------------------------ */

/* caml_llmopt_metal_dispatch (:1384-1454): launches one kernel and waits. */
int llmopt_hip_dispatch(llmopt_hip_library *library, const llmopt_hip_dispatch_item *item);

/* caml_llmopt_metal_begin_batch (:1132-1154).  A batch records dispatches and
 * copies; nothing runs before commit, so abort discards them, as discarding an
 * uncommitted Metal command buffer does. */
int llmopt_hip_begin_batch(llmopt_hip_library *library, llmopt_hip_batch **out);
void llmopt_hip_release_batch(llmopt_hip_batch *batch);
/* caml_llmopt_metal_batch_dispatch (:1156-1207). */
int llmopt_hip_batch_dispatch(llmopt_hip_batch *batch, llmopt_hip_library *library,
                              const llmopt_hip_dispatch_item *item);
/* caml_llmopt_metal_batch_dispatch_all (:1209-1274). */
int llmopt_hip_batch_dispatch_all(llmopt_hip_batch *batch, llmopt_hip_library *library,
                                  const llmopt_hip_dispatch_item *items, size_t count);
/* caml_llmopt_metal_batch_copy (:1276-1315): equal lengths, no overlap. */
int llmopt_hip_batch_copy(llmopt_hip_batch *batch, llmopt_hip_buffer *source,
                          llmopt_hip_buffer *destination);
/* caml_llmopt_metal_batch_barrier (:1317-1320): a no-op there and here
 * (launches on one stream are already ordered). */
int llmopt_hip_batch_barrier(llmopt_hip_batch *batch);
/* caml_llmopt_metal_commit_batch (:1322-1357): launches everything recorded,
 * in order, and waits. */
int llmopt_hip_commit_batch(llmopt_hip_batch *batch);
/* caml_llmopt_metal_commit_batch_async (:1359-1370): launches without waiting. */
int llmopt_hip_commit_batch_async(llmopt_hip_batch *batch);
/* Commit for measurement: the counterpart of committing under
 * LLMOPT_PROFILE_BATCH, where the reference reports the command buffer's GPU
 * time (native/ocaml_metal_stubs.m:1337-1347).  Runs the recorded work once
 * untimed, then `repeats` times between two HIP events on the context's
 * stream (as one HIP graph per repeat when use_graph != 0, so launches are
 * back to back) and returns the elapsed GPU milliseconds of the timed part.
 * use_graph = 2..4: the caller states that the recorded operations do not
 * depend on each other; the graph then has that many branches the GPU may
 * run side by side; every operation goes to the branch with the fewest bytes
 * of bound buffers so far (those that use the context's scratch memory stay
 * on the first, in recorded order). */
int llmopt_hip_commit_batch_profiled(llmopt_hip_batch *batch, int use_graph, int repeats,
                                     float *gpu_milliseconds);
/* The same commit with every one of the `repeats` timed runs measured on its own (a HIP
 * event between consecutive runs): gpu_milliseconds_each[0 .. repeats) receives their GPU
 * milliseconds, so that a caller can report a median.  No reference counterpart (the
 * reference reports one command buffer's GPU time per commit, :1337-1347). */
int llmopt_hip_commit_batch_profiled_each(llmopt_hip_batch *batch, int use_graph, int repeats,
                                          float *gpu_milliseconds_each);
/* caml_llmopt_metal_abort_batch (:1372-1382). */
int llmopt_hip_abort_batch(llmopt_hip_batch *batch);

/* ---- retained decode plan ------------------------------------------------ */

/* caml_llmopt_prebaked_create (:1879-2165): freezes a dispatch array; at most
 * 16 buffers and 256 parameter bytes per record.  The records are captured
 * into one HIP graph here (nothing runs): a later execute is a single graph
 * launch.  Paged attention records (names starting with
 * "llmopt_attention_q8_paged_", the batched extension excepted) read their
 * context length from a device word of the plan instead of parameter byte 12
 * and are sized for the capacity of their slot table (buffer 4), so one graph
 * serves every step; a plan that holds a masked one is replayed record by
 * record from the host instead, as the reference does.  Buffers the caller
 * rewrites between steps (rotary rows, slots, the lengths of the batched
 * extension) are read from device memory by the kernels, replay included. */
int llmopt_hip_prebaked_create(llmopt_hip_library *library,
                               const llmopt_hip_dispatch_item *items, size_t count,
                               llmopt_hip_buffer *token_buffer, llmopt_hip_buffer *output_buffer,
                               llmopt_hip_prebaked **out);
void llmopt_hip_release_prebaked(llmopt_hip_prebaked *plan);
/* caml_llmopt_prebaked_execute (:2167-2560): writes `token` (int64) at the
 * start of the token buffer, makes past_tokens the context length of every
 * paged attention record (:2182-2195) and `checkpoint` the slot of every
 * llmopt_cache_pack_checkpoint_q8_simd record (byte 0 of its parameter block,
 * :2186-2188), replays all records in order, waits, and returns the first
 * int32 of the output buffer in *out_token.
 * past_tokens beyond the slot tables' capacity is LLMOPT_ERR_INVALID.
 * Debug replays of the reference, switched on by the same environment
 * variables (:2203-2347): LLMOPT_PROFILE_BREAKDOWN runs the records one at a
 * time and prints GPU time by kernel name to stderr; LLMOPT_DEBUG_NAN_CHECK
 * (steps with past_tokens > 0, or every step under LLMOPT_CHECK_PREFILL)
 * reports the first record that leaves a NaN in a buffer that held none and
 * returns LLMOPT_ERR_FAILURE (the reference exits the process there). */
int llmopt_hip_prebaked_execute(llmopt_hip_prebaked *plan, int64_t token, int64_t past_tokens,
                                int64_t checkpoint, int64_t *out_token);
/* 1 when execute replays one HIP graph, 0 when it launches record by record
 * (no reference counterpart; for diagnostics and tests). */
int llmopt_hip_prebaked_is_single_submission(llmopt_hip_prebaked *plan);

/* ---- ring queue ------------------------------------------------------------ */

/* The submission / completion queues of lib/metal_native.ml:86-111 (256
 * entries each, one submitting thread, one worker thread).  The worker runs
 * one decode step of a retained plan per submission, in order, on the
 * context's stream; while it runs it is the context's caller thread.
 * LLMOPT_QUEUE_DEPTH (default 1, as lib/metal_native.ml:407-415) > 1 lets it
 * queue the next step on the GPU before it waits for the previous one. */

/* caml_llmopt_ring_create (native/ocaml_metal_stubs.m:1699-1710). */
int llmopt_hip_ring_create(llmopt_hip_ring **out);
/* caml_llmopt_ring_submit (:1712-1732): 1 when queued, 0 when 256 submissions
 * are waiting.  token < 0 chains: the step's input is the token the previous
 * step produced (:1546-1560).  flags == 2 stops the worker (:1538). */
int llmopt_hip_ring_submit(llmopt_hip_ring *ring, int64_t request_id, int64_t token,
                           int64_t past_tokens, int64_t flags);
/* caml_llmopt_ring_wait_completion (:1734-1767): blocks for the next
 * (request id, produced token, status 0 = ok / 1 = failed); fails with "Ring
 * queue terminated with no completion" when the ring stops first. */
int llmopt_hip_ring_wait_completion(llmopt_hip_ring *ring, int64_t *request_id, int64_t *token,
                                    int64_t *status);
/* caml_llmopt_ring_poll_completion (:1769-1797): 1 with a completion, 0 with
 * none (the reference's None), negative on error. */
int llmopt_hip_ring_poll_completion(llmopt_hip_ring *ring, int64_t *request_id, int64_t *token,
                                    int64_t *status);
/* caml_llmopt_ring_start_worker (:1799-1871): freezes the dispatch array as
 * llmopt_hip_prebaked_create does and starts the worker thread. */
int llmopt_hip_ring_start_worker(llmopt_hip_ring *ring, llmopt_hip_library *library,
                                 const llmopt_hip_dispatch_item *items, size_t count,
                                 llmopt_hip_buffer *token_buffer,
                                 llmopt_hip_buffer *output_buffer);
/* The same worker over a host function instead of a plan (no reference
 * counterpart: other executors, and tests of the queue without a GPU).  The
 * function gets the step's token (a chained step: the previous result) and
 * context length, stores the produced token and returns LLMOPT_OK or a
 * failure status. */
typedef int (*llmopt_hip_ring_step)(void *user, int64_t token, int64_t past_tokens,
                                    int32_t *out_token);
int llmopt_hip_ring_start_worker_with(llmopt_hip_ring *ring, llmopt_hip_ring_step step,
                                      void *user);
/* caml_llmopt_ring_destroy (finalize_ring, :296-329): stops and joins the
 * worker, releases the plan. */
void llmopt_hip_ring_destroy(llmopt_hip_ring *ring);

/* ---- the entry point that allocates nothing ---------------------------------- */

/* No counterpart in the reference.  For callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It is llmopt_attention_q8_paged_simd_* (one slot table for
 * all sequences, no mask) with plain device pointers: `parameters` is the
 * 64-byte Q8PagedAttentionParams block (lib/metal_cache_source.ml:352-369) in
 * host memory, the other pointers are device memory (query f16 [b, h, q, D],
 * current key / value f16 [b, kvh, q, D], the Q8 pool and its byte length,
 * `slot_count` u32 slot indices, output f16 [b, q, h, D]).  The work is queued
 * on `hip_stream` (a hipStream_t; NULL is the default stream) of the current
 * device and not waited for.
 * The partial results of the split-context kernels live in a fixed array of
 * LLMOPT_NO_ALLOC_SCRATCH_BYTES in the library's code object, one copy per
 * GPU, held until the process ends.  A call that needs more fails with
 * LLMOPT_ERR_INVALID and launches nothing.  No hipMalloc, hipFree or other
 * allocating routine is called.  All calls on one GPU share the array: calls
 * ordered on one stream are safe, calls that overlap on one GPU race.
 * llmopt_hip_create_context resolves the array's address for its device; on a
 * device with no context the first call does (do it before a capture). */
#define LLMOPT_NO_ALLOC_SCRATCH_BYTES (8u << 20)
int llmopt_hip_attention_q8_paged_no_alloc(void *hip_stream, const void *parameters,
                                           const void *query, const void *current_key,
                                           const void *current_value, const void *pool,
                                           size_t pool_bytes, const uint32_t *slots,
                                           size_t slot_count, void *output);

#ifdef __cplusplus
}
#endif

#endif /* LLMOPT_HIP_H */
