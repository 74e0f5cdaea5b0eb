// Implementation of include/llmopt_hip.h: the HIP counterpart of
// native/ocaml_metal_stubs.m's context / buffer / dispatch / batch / retained
// plan subset.  Error texts follow the reference's where a caller could match
// on them.
#include "runtime.h"

#include "kernels/kernels.h"

#include <fcntl.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <memory>

namespace llmopt {

// ---- errors ---------------------------------------------------------------
static thread_local std::string g_last_error;

int fail(int code, const char *format, ...) {
  char message[512];
  va_list args;
  va_start(args, format);
  vsnprintf(message, sizeof message, format, args);
  va_end(args);
  g_last_error = message;
  return code;
}

int fail_hip(hipError_t error, const char *what) {
  return fail(LLMOPT_ERR_FAILURE, "%s: %s", what, hipGetErrorString(error));
}

const char *last_error() { return g_last_error.c_str(); }
void clear_error() { g_last_error.clear(); }

void retain(RefCounted *object) {
  if (object) object->refs.fetch_add(1, std::memory_order_relaxed);
}

bool release(RefCounted *object) {
  return object && object->refs.fetch_sub(1, std::memory_order_acq_rel) == 1;
}

// ---- registry ---------------------------------------------------------------
void register_linear_kernels(std::vector<KernelEntryPoint> &table);
void register_cache_kernels(std::vector<KernelEntryPoint> &table);
void register_attention_kernels(std::vector<KernelEntryPoint> &table);
void register_glue_kernels(std::vector<KernelEntryPoint> &table);

const std::vector<KernelEntryPoint> &kernel_table() {
  static const std::vector<KernelEntryPoint> table = [] {
    std::vector<KernelEntryPoint> entries;
    register_linear_kernels(entries);
    register_cache_kernels(entries);
    register_attention_kernels(entries);
    register_glue_kernels(entries);
    return entries;
  }();
  return table;
}

const KernelEntryPoint *find_kernel(const char *name) {
  if (name == nullptr) return nullptr;
  for (const KernelEntryPoint &entry : kernel_table())
    if (strcmp(entry.name, name) == 0) return &entry;
  return nullptr;
}

// ---- handler helpers --------------------------------------------------------
int require_buffer_size(const BoundBuffer &buffer, uint64_t required, const char *name) {
  if ((uint64_t)buffer.length < required)
    return fail(LLMOPT_ERR_INVALID, "HIP %s buffer is too small: required=%llu actual=%llu", name,
                (unsigned long long)required, (unsigned long long)buffer.length);
  return LLMOPT_OK;
}

int require_buffer_count(const DispatchRecord &record, size_t expected) {
  if (record.buffers.size() != expected)
    return fail(LLMOPT_ERR_INVALID, "%s expects %zu buffers, got %zu", record.name.c_str(),
                expected, record.buffers.size());
  return LLMOPT_OK;
}

int require_parameter_bytes(const DispatchRecord &record, size_t expected) {
  if (record.parameters.size() != expected)
    return fail(LLMOPT_ERR_INVALID, "%s expects a %zu-byte parameter block, got %zu",
                record.name.c_str(), expected, record.parameters.size());
  return LLMOPT_OK;
}

uint32_t param_u32(const DispatchRecord &record, size_t byte_offset) {
  uint32_t value = 0;
  memcpy(&value, record.parameters.data() + byte_offset, 4);  // little-endian host
  return value;
}

float param_f32(const DispatchRecord &record, size_t byte_offset) {
  float value = 0;
  memcpy(&value, record.parameters.data() + byte_offset, 4);
  return value;
}

void *context_workspace(llmopt_hip_context *context, size_t bytes) {
  context->scratch_touched = true;
  if (bytes <= context->workspace_bytes) return context->workspace;
  if (context->sizing_capture) {
    // The launch being captured is never run: any non-null address will do.  Only for a launch that
    // really is being captured: one that would run (another thread using the context while a plan is
    // being captured, which the interface does not allow) must not get a placeholder for an address.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(context->stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusActive) {
      (void)hipGetLastError();
      fail(LLMOPT_ERR_FAILURE, "HIP context is capturing a plan on another thread: a context serves one thread at a time");
      return nullptr;
    }
    context->sizing_wanted = std::max(context->sizing_wanted, bytes);
    return context->workspace ? context->workspace : static_cast<void *>(context);
  }
  // Work already queued may still read the old block: drain before replacing.
  if (hipStreamSynchronize(context->stream) != hipSuccess) {
    fail(LLMOPT_ERR_FAILURE, "HIP stream synchronize failed while growing the workspace");
    return nullptr;
  }
  if (context->workspace) (void)hipFree(context->workspace);
  context->workspace = nullptr;
  context->workspace_bytes = 0;
  const size_t rounded = (bytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
  void *block = nullptr;
  hipError_t status = hipMalloc(&block, rounded);
  if (status != hipSuccess) {
    fail_hip(status, "HIP could not allocate the kernel workspace");
    return nullptr;
  }
  context->workspace = block;
  context->workspace_bytes = rounded;
  ++context->workspace_generation;
  return block;
}

uint32_t *context_counters(llmopt_hip_context *context, uint32_t *count) {
  constexpr uint32_t kCounters = 16384;
  context->scratch_touched = true;
  if (context->counters == nullptr) {
    void *block = nullptr;
    hipError_t status = hipMalloc(&block, kCounters * sizeof(uint32_t));
    if (status == hipSuccess) status = hipMemset(block, 0, kCounters * sizeof(uint32_t));
    if (status != hipSuccess) {
      if (block) (void)hipFree(block);
      fail_hip(status, "HIP could not allocate the tile counters");
      return nullptr;
    }
    context->counters = static_cast<uint32_t *>(block);
    context->counter_count = kCounters;
  }
  *count = context->counter_count;
  return context->counters;
}

static int positive_size(int64_t value, const char *name) {
  if (value <= 0) return fail(LLMOPT_ERR_INVALID, "HIP %s must be positive", name);
  return LLMOPT_OK;
}

int build_record(llmopt_hip_library *library, const llmopt_hip_dispatch_item *item,
                 DispatchRecord *out) {
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  if (item == nullptr || item->name == nullptr)
    return fail(LLMOPT_ERR_INVALID, "HIP dispatch item is missing");
  static const char *const grid_names[3] = {"grid width", "grid height", "grid depth"};
  static const char *const group_names[3] = {"threadgroup width", "threadgroup height",
                                             "threadgroup depth"};
  for (int i = 0; i < 3; ++i) {
    if (int status = positive_size(item->grid[i], grid_names[i])) return status;
    if (int status = positive_size(item->group[i], group_names[i])) return status;
  }
  if (find_kernel(item->name) == nullptr)
    return fail(LLMOPT_ERR_FAILURE, "HIP library does not contain the selected kernel");
  if (item->group[0] * item->group[1] * item->group[2] > 1024)
    return fail(LLMOPT_ERR_INVALID, "HIP threadgroup exceeds pipeline capacity");
  out->name = item->name;
  out->buffers.clear();
  out->retained.clear();
  for (uint32_t i = 0; i < item->buffer_count; ++i) {
    llmopt_hip_buffer *buffer = item->buffers[i];
    if (buffer == nullptr) {
      drop_record(out);
      return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
    }
    if (buffer->context != library->context) {
      drop_record(out);
      return fail(LLMOPT_ERR_INVALID, "HIP buffer belongs to a different device context");
    }
    retain(buffer);
    out->retained.push_back(buffer);
    out->buffers.push_back({buffer->device, buffer->length});
  }
  const uint8_t *bytes = static_cast<const uint8_t *>(item->parameters);
  out->parameters.assign(bytes, bytes + (bytes ? item->parameter_bytes : 0));
  for (int i = 0; i < 3; ++i) {
    out->grid[i] = item->grid[i];
    out->group[i] = item->group[i];
  }
  out->barrier_before = item->barrier_before != 0;
  return LLMOPT_OK;
}

int launch_record(llmopt_hip_context *context, const DispatchRecord &record) {
  const KernelEntryPoint *entry = find_kernel(record.name.c_str());
  if (entry == nullptr)
    return fail(LLMOPT_ERR_FAILURE, "HIP library does not contain the selected kernel");
  return entry->handler(context, record);
}

void drop_record(DispatchRecord *record) {
  for (llmopt_hip_buffer *buffer : record->retained) llmopt_hip_release_buffer(buffer);
  record->retained.clear();
  record->buffers.clear();
}

int use_device(llmopt_hip_context *context) {
  LLMOPT_HIP_TRY(hipSetDevice(context->device), "HIP could not select the context's device");
  return LLMOPT_OK;
}

}  // namespace llmopt

using namespace llmopt;

// ---- batch / plan objects ----------------------------------------------------
struct BatchOp {
  bool is_copy = false;
  DispatchRecord record;
  llmopt_hip_buffer *source = nullptr;
  llmopt_hip_buffer *destination = nullptr;
};

struct llmopt_hip_batch : llmopt::RefCounted {
  llmopt_hip_library *library = nullptr;
  std::vector<BatchOp> ops;
  bool finished = false;
};


extern "C" {

const char *llmopt_hip_last_error(void) { return last_error(); }

// ---- context ------------------------------------------------------------------
int llmopt_hip_create_context(int device, llmopt_hip_context **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "context output pointer is null");
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0)
    return fail(LLMOPT_ERR_FAILURE, "HIP has no default device");
  if (device < 0) {
    if (hipGetDevice(&device) != hipSuccess) device = 0;
  }
  if (device >= count) return fail(LLMOPT_ERR_INVALID, "HIP device index %d is out of range", device);
  LLMOPT_HIP_TRY(hipSetDevice(device), "HIP could not select the device");
  std::unique_ptr<llmopt_hip_context> context(new llmopt_hip_context());
  context->device = device;
  hipDeviceProp_t properties;
  LLMOPT_HIP_TRY(hipGetDeviceProperties(&properties, device), "HIP could not query the device");
  context->name = std::string(properties.name) + " (" + properties.gcnArchName + ")";
  context->compute_units = properties.multiProcessorCount > 0 ? properties.multiProcessorCount : 256;
  if (strncmp(properties.gcnArchName, "gfx950", 6) != 0)
    return fail(LLMOPT_ERR_FAILURE, "this library is built for gfx950 only, device is %s",
                properties.gcnArchName);
  LLMOPT_HIP_TRY(hipStreamCreateWithFlags(&context->stream, hipStreamNonBlocking),
                 "HIP could not create a stream");
  context->owns_stream = true;
  if (int status = no_alloc_prepare_current_device()) {
    (void)hipStreamDestroy(context->stream);
    return status;
  }
  *out = context.release();
  return LLMOPT_OK;
}

void llmopt_hip_release_context(llmopt_hip_context *context) {
  if (!release(context)) return;
  (void)hipSetDevice(context->device);
  if (context->stream) (void)hipStreamSynchronize(context->stream);
  if (context->workspace) (void)hipFree(context->workspace);
  if (context->counters) (void)hipFree(context->counters);
  if (context->owns_stream && context->stream) (void)hipStreamDestroy(context->stream);
  delete context;
}

int llmopt_hip_device_name(llmopt_hip_context *context, char *out, size_t capacity) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (out == nullptr || capacity == 0) return fail(LLMOPT_ERR_INVALID, "device name buffer is empty");
  snprintf(out, capacity, "%s", context->name.c_str());
  return LLMOPT_OK;
}

int llmopt_hip_context_set_stream(llmopt_hip_context *context, void *hip_stream) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (int status = use_device(context)) return status;
  LLMOPT_HIP_TRY(hipStreamSynchronize(context->stream), "HIP stream synchronize failed");
  if (context->owns_stream && context->stream) (void)hipStreamDestroy(context->stream);
  context->stream = static_cast<hipStream_t>(hip_stream);
  context->owns_stream = false;
  return LLMOPT_OK;
}

int llmopt_hip_context_synchronize(llmopt_hip_context *context) {
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (int status = use_device(context)) return status;
  LLMOPT_HIP_TRY(hipStreamSynchronize(context->stream), "HIP batch failed");
  return LLMOPT_OK;
}

// ---- library ------------------------------------------------------------------
int llmopt_hip_load_library(llmopt_hip_context *context, const char *path,
                            llmopt_hip_library **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "library output pointer is null");
  *out = nullptr;
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  llmopt_hip_library *library = new llmopt_hip_library();
  library->context = context;
  retain(context);
  library->path = path ? path : "";
  *out = library;
  return LLMOPT_OK;
}

void llmopt_hip_release_library(llmopt_hip_library *library) {
  if (!release(library)) return;
  llmopt_hip_release_context(library->context);
  delete library;
}

int llmopt_hip_has_function(llmopt_hip_library *library, const char *name) {
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  return find_kernel(name) != nullptr ? 1 : 0;
}

int llmopt_hip_preload_pipeline(llmopt_hip_library *library, const char *name) {
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  if (find_kernel(name) == nullptr)
    return fail(LLMOPT_ERR_FAILURE, "HIP library does not contain the selected kernel");
  return LLMOPT_OK;
}

int llmopt_hip_function_count(llmopt_hip_library *library) {
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  return (int)kernel_table().size();
}

const char *llmopt_hip_function_name(llmopt_hip_library *library, int index) {
  if (library == nullptr || index < 0 || index >= (int)kernel_table().size()) return nullptr;
  return kernel_table()[index].name;
}

// ---- buffers ------------------------------------------------------------------
static int allocate_buffer(llmopt_hip_context *context, size_t length, llmopt_hip_buffer **out) {
  if (int status = use_device(context)) return status;
  void *device = nullptr;
  if (hipMalloc(&device, length) != hipSuccess)
    return fail(LLMOPT_ERR_FAILURE, "HIP could not allocate a buffer");
  llmopt_hip_buffer *buffer = new llmopt_hip_buffer();
  buffer->context = context;
  retain(context);
  buffer->device = static_cast<uint8_t *>(device);
  buffer->length = length;
  buffer->owns_memory = true;
  *out = buffer;
  return LLMOPT_OK;
}

int llmopt_hip_buffer_of_bytes(llmopt_hip_context *context, const void *bytes, size_t length,
                               llmopt_hip_buffer **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "buffer output pointer is null");
  *out = nullptr;
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (length == 0 || bytes == nullptr) return fail(LLMOPT_ERR_INVALID, "HIP buffer cannot be empty");
  llmopt_hip_buffer *buffer = nullptr;
  if (int status = allocate_buffer(context, length, &buffer)) return status;
  hipError_t status = hipMemcpyAsync(buffer->device, bytes, length, hipMemcpyHostToDevice, context->stream);
  if (status == hipSuccess) status = hipStreamSynchronize(context->stream);
  if (status != hipSuccess) {
    llmopt_hip_release_buffer(buffer);
    return fail(LLMOPT_ERR_FAILURE, "HIP could not allocate and initialize a buffer");
  }
  *out = buffer;
  return LLMOPT_OK;
}

int llmopt_hip_create_buffer(llmopt_hip_context *context, int64_t bytes, llmopt_hip_buffer **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "buffer output pointer is null");
  *out = nullptr;
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  const size_t length = bytes <= 0 ? 16 : (size_t)bytes;
  llmopt_hip_buffer *buffer = nullptr;
  if (int status = allocate_buffer(context, length, &buffer)) return status;
  hipError_t status = hipMemsetAsync(buffer->device, 0, length, context->stream);
  if (status == hipSuccess) status = hipStreamSynchronize(context->stream);
  if (status != hipSuccess) {
    llmopt_hip_release_buffer(buffer);
    return fail(LLMOPT_ERR_FAILURE, "HIP could not allocate a buffer");
  }
  *out = buffer;
  return LLMOPT_OK;
}

int llmopt_hip_map_file(llmopt_hip_context *context, const char *path, llmopt_hip_buffer **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "buffer output pointer is null");
  *out = nullptr;
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (path == nullptr) return fail(LLMOPT_ERR_INVALID, "tensor store path is null");
  const int descriptor = open(path, O_RDONLY);
  if (descriptor < 0) return fail(LLMOPT_ERR_FAILURE, "cannot open tensor store %s: %s", path, strerror(errno));
  struct stat info;
  if (fstat(descriptor, &info) != 0) {
    const int saved = errno;
    close(descriptor);
    return fail(LLMOPT_ERR_FAILURE, "cannot stat tensor store %s: %s", path, strerror(saved));
  }
  if (info.st_size == 0) {
    close(descriptor);
    return fail(LLMOPT_ERR_FAILURE, "tensor store is empty");
  }
  const size_t length = (size_t)info.st_size;
  void *mapping = mmap(nullptr, length, PROT_READ, MAP_PRIVATE, descriptor, 0);
  close(descriptor);
  if (mapping == MAP_FAILED)
    return fail(LLMOPT_ERR_FAILURE, "cannot map tensor store %s: %s", path, strerror(errno));
  llmopt_hip_buffer *buffer = nullptr;
  int status = allocate_buffer(context, length, &buffer);
  if (status == LLMOPT_OK) {
    hipError_t copy = hipMemcpyAsync(buffer->device, mapping, length, hipMemcpyHostToDevice, context->stream);
    if (copy == hipSuccess) copy = hipStreamSynchronize(context->stream);
    if (copy != hipSuccess) {
      llmopt_hip_release_buffer(buffer);
      buffer = nullptr;
      status = fail(LLMOPT_ERR_FAILURE, "HIP could not upload the mapped tensor store");
    }
  }
  munmap(mapping, length);
  if (status != LLMOPT_OK) return status;
  *out = buffer;
  return LLMOPT_OK;
}

int llmopt_hip_buffer_view(llmopt_hip_buffer *parent, int64_t offset, int64_t length,
                           llmopt_hip_buffer **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "buffer output pointer is null");
  *out = nullptr;
  if (parent == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (offset < 0 || length <= 0 || (uint64_t)offset > parent->length ||
      (uint64_t)length > parent->length - (uint64_t)offset)
    return fail(LLMOPT_ERR_INVALID, "HIP buffer view is outside its parent buffer");
  llmopt_hip_buffer *view = new llmopt_hip_buffer();
  view->context = parent->context;
  retain(parent->context);
  view->parent = parent;
  retain(parent);
  view->device = parent->device + offset;
  view->length = (size_t)length;
  *out = view;
  return LLMOPT_OK;
}

int llmopt_hip_buffer_wrap(llmopt_hip_context *context, void *device_pointer, size_t length,
                           llmopt_hip_buffer **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "buffer output pointer is null");
  *out = nullptr;
  if (context == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP context has been finalized");
  if (device_pointer == nullptr || length == 0)
    return fail(LLMOPT_ERR_INVALID, "HIP buffer cannot be empty");
  llmopt_hip_buffer *buffer = new llmopt_hip_buffer();
  buffer->context = context;
  retain(context);
  buffer->device = static_cast<uint8_t *>(device_pointer);
  buffer->length = length;
  *out = buffer;
  return LLMOPT_OK;
}

void llmopt_hip_release_buffer(llmopt_hip_buffer *buffer) {
  if (!release(buffer)) return;
  if (buffer->owns_memory && buffer->device) {
    (void)hipSetDevice(buffer->context->device);
    (void)hipStreamSynchronize(buffer->context->stream);
    (void)hipFree(buffer->device);
  }
  if (buffer->parent) llmopt_hip_release_buffer(buffer->parent);
  llmopt_hip_release_context(buffer->context);
  delete buffer;
}

int llmopt_hip_buffer_contents(llmopt_hip_buffer *buffer, void *out, size_t capacity) {
  if (buffer == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (out == nullptr || capacity < buffer->length)
    return fail(LLMOPT_ERR_INVALID, "destination is smaller than the HIP buffer");
  if (int status = use_device(buffer->context)) return status;
  hipStream_t stream = buffer->context->stream;
  LLMOPT_HIP_TRY(hipMemcpyAsync(out, buffer->device, buffer->length, hipMemcpyDeviceToHost, stream),
                 "HIP could not read a buffer");
  LLMOPT_HIP_TRY(hipStreamSynchronize(stream), "HIP could not read a buffer");
  return LLMOPT_OK;
}

int64_t llmopt_hip_buffer_length(llmopt_hip_buffer *buffer) {
  if (buffer == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  return (int64_t)buffer->length;
}

void *llmopt_hip_buffer_device_pointer(llmopt_hip_buffer *buffer) {
  return buffer ? buffer->device : nullptr;
}

int llmopt_hip_buffer_copy(llmopt_hip_buffer *source, llmopt_hip_buffer *destination) {
  if (source == nullptr || destination == nullptr)
    return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (source->length != destination->length)
    return fail(LLMOPT_ERR_INVALID, "HIP copy requires equal buffer lengths");
  if (int status = use_device(source->context)) return status;
  hipStream_t stream = source->context->stream;
  LLMOPT_HIP_TRY(launch_copy_bytes(destination->device, source->device, source->length, stream),
                 "HIP buffer copy failed");
  LLMOPT_HIP_TRY(hipStreamSynchronize(stream), "HIP buffer copy failed");
  return LLMOPT_OK;
}

int llmopt_hip_buffer_write(llmopt_hip_buffer *buffer, int64_t offset, const void *bytes,
                            size_t length) {
  if (buffer == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (offset < 0 || (uint64_t)offset > buffer->length || length > buffer->length - (uint64_t)offset)
    return fail(LLMOPT_ERR_INVALID, "buffer offset out of bounds");
  if (length == 0) return LLMOPT_OK;
  if (int status = use_device(buffer->context)) return status;
  hipStream_t stream = buffer->context->stream;
  LLMOPT_HIP_TRY(hipMemcpyAsync(buffer->device + offset, bytes, length, hipMemcpyHostToDevice, stream),
                 "HIP buffer write failed");
  LLMOPT_HIP_TRY(hipStreamSynchronize(stream), "HIP buffer write failed");
  return LLMOPT_OK;
}

int llmopt_hip_buffer_set_int64(llmopt_hip_buffer *buffer, int64_t offset, int64_t value) {
  if (buffer == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (offset < 0 || (uint64_t)offset + 8 > buffer->length)
    return fail(LLMOPT_ERR_INVALID, "buffer offset out of bounds");
  return llmopt_hip_buffer_write(buffer, offset, &value, sizeof value);
}

int llmopt_hip_buffer_set_u32_array(llmopt_hip_buffer *buffer, int64_t offset,
                                    const int64_t *values, size_t count) {
  if (buffer == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (offset < 0 || (uint64_t)offset + (uint64_t)count * 4 > buffer->length)
    return fail(LLMOPT_ERR_INVALID, "buffer set_u32_array out of bounds");
  std::vector<uint32_t> narrowed(count);
  for (size_t i = 0; i < count; ++i) narrowed[i] = (uint32_t)values[i];
  return llmopt_hip_buffer_write(buffer, offset, narrowed.data(), count * 4);
}

int llmopt_hip_buffer_argmax_f16(llmopt_hip_buffer *buffer, int64_t vocabulary, int64_t *out) {
  if (buffer == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (vocabulary <= 0) return fail(LLMOPT_ERR_INVALID, "float16 logits vocabulary must be positive");
  const uint64_t row_bytes = (uint64_t)vocabulary * 2;
  if (buffer->length == 0 || buffer->length % row_bytes != 0)
    return fail(LLMOPT_ERR_INVALID, "float16 logits buffer does not contain complete rows");
  std::vector<uint16_t> row((size_t)vocabulary);
  if (int status = use_device(buffer->context)) return status;
  hipStream_t stream = buffer->context->stream;
  LLMOPT_HIP_TRY(hipMemcpyAsync(row.data(), buffer->device + buffer->length - row_bytes, row_bytes,
                                hipMemcpyDeviceToHost, stream),
                 "HIP could not read a buffer");
  LLMOPT_HIP_TRY(hipStreamSynchronize(stream), "HIP could not read a buffer");
  auto to_float = [](uint16_t bits) { return (float)__builtin_bit_cast(_Float16, bits); };
  float best = to_float(row[0]);
  int64_t best_index = 0;
  for (int64_t i = 1; i < vocabulary; ++i) {
    const float value = to_float(row[(size_t)i]);
    if (value > best) {
      best = value;
      best_index = i;
    }
  }
  if (out) *out = best_index;
  return LLMOPT_OK;
}

// ---- dispatch -------------------------------------------------------------------
int llmopt_hip_dispatch(llmopt_hip_library *library, const llmopt_hip_dispatch_item *item) {
  DispatchRecord record;
  if (int status = build_record(library, item, &record)) return status;
  llmopt_hip_context *context = library->context;
  int status = use_device(context);
  if (status == LLMOPT_OK) status = launch_record(context, record);
  if (status == LLMOPT_OK && hipStreamSynchronize(context->stream) != hipSuccess)
    status = fail(LLMOPT_ERR_FAILURE, "HIP dispatch failed");
  drop_record(&record);
  return status;
}

static int require_active_batch(llmopt_hip_batch *batch) {
  if (batch == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP batch has been finalized");
  if (batch->finished) return fail(LLMOPT_ERR_INVALID, "HIP batch is already finished");
  return LLMOPT_OK;
}

static void clear_batch(llmopt_hip_batch *batch) {
  for (BatchOp &op : batch->ops) {
    drop_record(&op.record);
    if (op.source) llmopt_hip_release_buffer(op.source);
    if (op.destination) llmopt_hip_release_buffer(op.destination);
  }
  batch->ops.clear();
}

int llmopt_hip_begin_batch(llmopt_hip_library *library, llmopt_hip_batch **out) {
  if (out == nullptr) return fail(LLMOPT_ERR_INVALID, "batch output pointer is null");
  *out = nullptr;
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  llmopt_hip_batch *batch = new llmopt_hip_batch();
  batch->library = library;
  retain(library);
  *out = batch;
  return LLMOPT_OK;
}

void llmopt_hip_release_batch(llmopt_hip_batch *batch) {
  if (!release(batch)) return;
  clear_batch(batch);
  llmopt_hip_release_library(batch->library);
  delete batch;
}

int llmopt_hip_batch_dispatch(llmopt_hip_batch *batch, llmopt_hip_library *library,
                              const llmopt_hip_dispatch_item *item) {
  if (int status = require_active_batch(batch)) return status;
  if (library == nullptr) return fail(LLMOPT_ERR_FAILURE, "HIP library has been finalized");
  if (library->context != batch->library->context)
    return fail(LLMOPT_ERR_INVALID, "HIP batch and dispatch runtime use different device contexts");
  BatchOp op;
  if (int status = build_record(library, item, &op.record)) return status;
  batch->ops.push_back(std::move(op));
  return LLMOPT_OK;
}

int llmopt_hip_batch_dispatch_all(llmopt_hip_batch *batch, llmopt_hip_library *library,
                                  const llmopt_hip_dispatch_item *items, size_t count) {
  for (size_t i = 0; i < count; ++i)
    if (int status = llmopt_hip_batch_dispatch(batch, library, &items[i])) return status;
  return LLMOPT_OK;
}

int llmopt_hip_batch_copy(llmopt_hip_batch *batch, llmopt_hip_buffer *source,
                          llmopt_hip_buffer *destination) {
  if (int status = require_active_batch(batch)) return status;
  if (source == nullptr || destination == nullptr)
    return fail(LLMOPT_ERR_FAILURE, "HIP buffer has been finalized");
  if (source->length != destination->length)
    return fail(LLMOPT_ERR_INVALID, "HIP copy requires equal buffer lengths");
  const uint8_t *a = source->device, *b = destination->device;
  if (a < b + destination->length && b < a + source->length)
    return fail(LLMOPT_ERR_INVALID, "batched HIP copy buffers overlap");
  BatchOp op;
  op.is_copy = true;
  op.source = source;
  op.destination = destination;
  retain(source);
  retain(destination);
  batch->ops.push_back(std::move(op));
  return LLMOPT_OK;
}

int llmopt_hip_batch_barrier(llmopt_hip_batch *batch) { return require_active_batch(batch); }

static int submit_batch(llmopt_hip_batch *batch, bool wait) {
  if (int status = require_active_batch(batch)) return status;
  llmopt_hip_context *context = batch->library->context;
  if (int status = use_device(context)) return status;
  batch->finished = true;
  int status = LLMOPT_OK;
  for (BatchOp &op : batch->ops) {
    if (op.is_copy) {
      if (launch_copy_bytes(op.destination->device, op.source->device, op.source->length, context->stream) !=
          hipSuccess)
        status = fail(LLMOPT_ERR_FAILURE, "HIP batched copy failed");
    } else {
      status = launch_record(context, op.record);
    }
    if (status != LLMOPT_OK) break;
  }
  // Buffers stay retained until the work has drained (or, for an async
  // commit, until the batch handle is released).
  if (wait || status != LLMOPT_OK) {
    if (hipStreamSynchronize(context->stream) != hipSuccess && status == LLMOPT_OK)
      status = fail(LLMOPT_ERR_FAILURE, "HIP batch failed");
    clear_batch(batch);
  }
  return status;
}

int llmopt_hip_commit_batch(llmopt_hip_batch *batch) { return submit_batch(batch, true); }
int llmopt_hip_commit_batch_async(llmopt_hip_batch *batch) { return submit_batch(batch, false); }

}  // extern "C"

namespace {

// The profiled commit: `each`, when not null, receives the GPU milliseconds of every one of the
// `repeats` timed runs (an event between consecutive runs); `total` their sum from first to last event.
int commit_profiled(llmopt_hip_batch *batch, int use_graph, int repeats, float *gpu_milliseconds, float *each) {
  if (int status = require_active_batch(batch)) return status;
  if (repeats <= 0) return fail(LLMOPT_ERR_INVALID, "profiled commit needs a positive repeat count");
  constexpr int kMaxBranches = 4;  // hardware queues a process gets by default
  if (use_graph < 0 || use_graph > kMaxBranches)
    return fail(LLMOPT_ERR_INVALID, "profiled commit takes 0 (host launches), 1 (one graph) or 2..%d graph branches",
                kMaxBranches);
  llmopt_hip_context *context = batch->library->context;
  if (int status = use_device(context)) return status;
  batch->finished = true;
  hipStream_t stream = context->stream;
  const int branches = use_graph >= 2 ? use_graph : 1;
  // Branch of every recorded operation.  One branch: the recorded order, as commit_batch runs it.
  // Several: the caller states that the operations do not depend on each other; each goes to the
  // branch with the fewest bytes so far (the bytes of its buffers stand for its duration: these
  // launches stream their operands once), except those that use the context's scratch memory
  // (kernel workspace, arrival counters), which share it and stay in recorded order on branch 0.
  // Dealt round-robin, the sweep's twelve launches left branch 0 with the split-K launch of every
  // step on top of its share, half as much again as the others.
  std::vector<int> branch_of(batch->ops.size(), 0);
  size_t branch_bytes[kMaxBranches] = {};
  hipStream_t side[kMaxBranches] = {stream};
  auto deal = [&](size_t index, size_t bytes, bool shares_scratch) {
    int chosen = 0;
    if (!shares_scratch)
      for (int b = 1; b < branches; ++b)
        if (branch_bytes[b] < branch_bytes[chosen]) chosen = b;
    // a launch also costs what its start and end take whatever it reads: about 2.5 us, or 12 MB of streaming
    branch_bytes[chosen] += bytes + ((size_t)12 << 20);
    branch_of[index] = chosen;
  };
  auto launch_all = [&](bool classify, bool forked) -> int {
    for (size_t i = 0; i < batch->ops.size(); ++i) {
      BatchOp &op = batch->ops[i];
      hipStream_t target = forked ? side[branch_of[i]] : stream;
      if (op.is_copy) {
        if (launch_copy_bytes(op.destination->device, op.source->device, op.source->length, target) != hipSuccess)
          return fail(LLMOPT_ERR_FAILURE, "HIP batched copy failed");
        if (classify) deal(i, 2 * op.source->length, false);
        continue;
      }
      context->scratch_touched = false;
      context->stream = target;
      const int status = launch_record(context, op.record);
      context->stream = stream;
      if (status != LLMOPT_OK) return status;
      if (classify) {
        size_t bytes = 0;
        for (const BoundBuffer &buffer : op.record.buffers) bytes += buffer.length;
        deal(i, bytes, context->scratch_touched);
      }
    }
    return LLMOPT_OK;
  };
  // One untimed pass: first-use allocations (kernel workspace) happen here, outside any stream
  // capture, and every operation shows whether it takes scratch memory.
  int status = launch_all(true, false);
  if (status == LLMOPT_OK && hipStreamSynchronize(stream) != hipSuccess)
    status = fail(LLMOPT_ERR_FAILURE, "HIP batch failed");
  hipGraph_t graph = nullptr;
  hipGraphExec_t executable = nullptr;
  hipEvent_t start = nullptr, stop = nullptr, fork = nullptr, joined[kMaxBranches] = {};
  std::vector<hipEvent_t> between;  // after every run but the last, when each run is timed
  if (status == LLMOPT_OK && use_graph) {
    for (int b = 1; b < branches && status == LLMOPT_OK; ++b)
      if (hipStreamCreateWithFlags(&side[b], hipStreamNonBlocking) != hipSuccess ||
          hipEventCreateWithFlags(&joined[b], hipEventDisableTiming) != hipSuccess)
        status = fail(LLMOPT_ERR_FAILURE, "HIP could not create a graph branch");
    if (status == LLMOPT_OK && branches > 1 && hipEventCreateWithFlags(&fork, hipEventDisableTiming) != hipSuccess)
      status = fail(LLMOPT_ERR_FAILURE, "HIP could not create a graph branch");
    if (status == LLMOPT_OK && hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
      status = fail(LLMOPT_ERR_FAILURE, "HIP stream capture could not begin");
    } else if (status == LLMOPT_OK) {
      // fork: the side streams join the capture by waiting for an event of the origin stream
      if (branches > 1) {
        if (hipEventRecord(fork, stream) != hipSuccess) status = fail(LLMOPT_ERR_FAILURE, "HIP graph fork failed");
        for (int b = 1; b < branches && status == LLMOPT_OK; ++b)
          if (hipStreamWaitEvent(side[b], fork, 0) != hipSuccess) status = fail(LLMOPT_ERR_FAILURE, "HIP graph fork failed");
      }
      if (status == LLMOPT_OK) status = launch_all(false, branches > 1);
      for (int b = 1; b < branches; ++b)
        if (hipEventRecord(joined[b], side[b]) != hipSuccess || hipStreamWaitEvent(stream, joined[b], 0) != hipSuccess) {
          if (status == LLMOPT_OK) status = fail(LLMOPT_ERR_FAILURE, "HIP graph join failed");
        }
      if (hipStreamEndCapture(stream, &graph) != hipSuccess && status == LLMOPT_OK)
        status = fail(LLMOPT_ERR_FAILURE, "HIP stream capture failed");
      if (status == LLMOPT_OK &&
          hipGraphInstantiate(&executable, graph, nullptr, nullptr, 0) != hipSuccess)
        status = fail(LLMOPT_ERR_FAILURE, "HIP graph instantiation failed");
    }
  }
  if (status == LLMOPT_OK &&
      (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess))
    status = fail(LLMOPT_ERR_FAILURE, "HIP could not create timing events");
  if (status == LLMOPT_OK && each != nullptr) {
    between.assign((size_t)repeats - 1, nullptr);
    for (hipEvent_t &event : between)
      if (status == LLMOPT_OK && hipEventCreate(&event) != hipSuccess)
        status = fail(LLMOPT_ERR_FAILURE, "HIP could not create timing events");
  }
  if (status == LLMOPT_OK) {
    (void)hipEventRecord(start, stream);
    for (int i = 0; i < repeats && status == LLMOPT_OK; ++i) {
      if (executable) {
        if (hipGraphLaunch(executable, stream) != hipSuccess)
          status = fail(LLMOPT_ERR_FAILURE, "HIP graph launch failed");
      } else {
        status = launch_all(false, false);
      }
      if (each != nullptr && i + 1 < repeats) (void)hipEventRecord(between[(size_t)i], stream);
    }
    (void)hipEventRecord(stop, stream);
    if (hipStreamSynchronize(stream) != hipSuccess && status == LLMOPT_OK)
      status = fail(LLMOPT_ERR_FAILURE, "HIP batch failed");
    float elapsed = 0.0f;
    if (status == LLMOPT_OK && hipEventElapsedTime(&elapsed, start, stop) != hipSuccess)
      status = fail(LLMOPT_ERR_FAILURE, "HIP could not read the timing events");
    if (gpu_milliseconds) *gpu_milliseconds = elapsed;
    for (int i = 0; i < repeats && status == LLMOPT_OK && each != nullptr; ++i) {
      hipEvent_t from = i == 0 ? start : between[(size_t)i - 1], to = i + 1 == repeats ? stop : between[(size_t)i];
      if (hipEventElapsedTime(&each[i], from, to) != hipSuccess)
        status = fail(LLMOPT_ERR_FAILURE, "HIP could not read the timing events");
    }
  }
  for (hipEvent_t event : between)
    if (event) (void)hipEventDestroy(event);
  if (start) (void)hipEventDestroy(start);
  if (stop) (void)hipEventDestroy(stop);
  if (executable) (void)hipGraphExecDestroy(executable);
  if (graph) (void)hipGraphDestroy(graph);
  (void)hipStreamSynchronize(stream);
  if (fork) (void)hipEventDestroy(fork);
  for (int b = 1; b < branches; ++b) {
    if (joined[b]) (void)hipEventDestroy(joined[b]);
    if (side[b]) (void)hipStreamDestroy(side[b]);
  }
  clear_batch(batch);
  return status;
}

}  // namespace

extern "C" {

int llmopt_hip_commit_batch_profiled(llmopt_hip_batch *batch, int use_graph, int repeats,
                                     float *gpu_milliseconds) {
  return commit_profiled(batch, use_graph, repeats, gpu_milliseconds, nullptr);
}

int llmopt_hip_commit_batch_profiled_each(llmopt_hip_batch *batch, int use_graph, int repeats,
                                          float *gpu_milliseconds_each) {
  if (gpu_milliseconds_each == nullptr) return fail(LLMOPT_ERR_INVALID, "profiled commit needs room for the timings");
  return commit_profiled(batch, use_graph, repeats, nullptr, gpu_milliseconds_each);
}

int llmopt_hip_abort_batch(llmopt_hip_batch *batch) {
  if (batch != nullptr && !batch->finished) {
    clear_batch(batch);
    batch->finished = true;
  }
  return LLMOPT_OK;
}

}  // extern "C"
