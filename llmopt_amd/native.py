"""ctypes binding of libllmopt_hip.so (include/llmopt_hip.h).

Mirrors the OCaml module lib/metal_native.ml of the reference: `Runtime`
(context + library), `Buffer`, `Batch`, `Prebaked`, `kernel_entry`, `dispatch`.
Failures of the C ABI surface as `LlmoptError(message)`, the counterpart of the
reference's `Error message` results (lib/metal_native.ml:126-129).

There is no CPU fallback: if the shared library is missing, importing the
handle raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Iterable, Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# LLMOPT_HIP_LIBRARY names another build of the same library (python -m llmopt_amd.build --host-ubsan)
LIBRARY_PATH = os.environ.get("LLMOPT_HIP_LIBRARY") or os.path.join(_HERE, "libllmopt_hip.so")


class LlmoptError(RuntimeError):
    """A failed call of the HIP backend; `.code` is the C status (-1 failure, -2 invalid)."""

    def __init__(self, message: str, code: int = -1):
        super().__init__(message)
        self.code = code


class DispatchItem(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char_p),
        ("buffers", ctypes.POINTER(ctypes.c_void_p)),
        ("buffer_count", ctypes.c_uint32),
        ("parameters", ctypes.c_void_p),
        ("parameter_bytes", ctypes.c_uint32),
        ("grid", ctypes.c_int64 * 3),
        ("group", ctypes.c_int64 * 3),
        ("barrier_before", ctypes.c_int32),
    ]


# llmopt_hip_ring_step: int (*)(void *user, int64 token, int64 past_tokens, int32 *out_token)
RING_STEP = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                             ctypes.POINTER(ctypes.c_int32))

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """The loaded shared library.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        raise LlmoptError(
            f"{LIBRARY_PATH} is missing: build it with `python -m llmopt_amd.build` "
            "(there is no CPU fallback)")
    handle = ctypes.CDLL(LIBRARY_PATH)
    vp, i64, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_size_t
    pp = ctypes.POINTER(ctypes.c_void_p)
    item_p = ctypes.POINTER(DispatchItem)
    signatures = {
        "llmopt_hip_last_error": (ctypes.c_char_p, []),
        "llmopt_hip_create_context": (ctypes.c_int, [ctypes.c_int, pp]),
        "llmopt_hip_release_context": (None, [vp]),
        "llmopt_hip_device_name": (ctypes.c_int, [vp, ctypes.c_char_p, sz]),
        "llmopt_hip_context_set_stream": (ctypes.c_int, [vp, vp]),
        "llmopt_hip_context_synchronize": (ctypes.c_int, [vp]),
        "llmopt_hip_load_library": (ctypes.c_int, [vp, ctypes.c_char_p, pp]),
        "llmopt_hip_release_library": (None, [vp]),
        "llmopt_hip_has_function": (ctypes.c_int, [vp, ctypes.c_char_p]),
        "llmopt_hip_preload_pipeline": (ctypes.c_int, [vp, ctypes.c_char_p]),
        "llmopt_hip_function_count": (ctypes.c_int, [vp]),
        "llmopt_hip_function_name": (ctypes.c_char_p, [vp, ctypes.c_int]),
        "llmopt_hip_buffer_of_bytes": (ctypes.c_int, [vp, vp, sz, pp]),
        "llmopt_hip_create_buffer": (ctypes.c_int, [vp, i64, pp]),
        "llmopt_hip_map_file": (ctypes.c_int, [vp, ctypes.c_char_p, pp]),
        "llmopt_hip_buffer_view": (ctypes.c_int, [vp, i64, i64, pp]),
        "llmopt_hip_buffer_wrap": (ctypes.c_int, [vp, vp, sz, pp]),
        "llmopt_hip_release_buffer": (None, [vp]),
        "llmopt_hip_buffer_contents": (ctypes.c_int, [vp, vp, sz]),
        "llmopt_hip_buffer_length": (i64, [vp]),
        "llmopt_hip_buffer_device_pointer": (vp, [vp]),
        "llmopt_hip_buffer_copy": (ctypes.c_int, [vp, vp]),
        "llmopt_hip_buffer_write": (ctypes.c_int, [vp, i64, vp, sz]),
        "llmopt_hip_buffer_set_int64": (ctypes.c_int, [vp, i64, i64]),
        "llmopt_hip_buffer_set_u32_array": (ctypes.c_int, [vp, i64, ctypes.POINTER(i64), sz]),
        "llmopt_hip_buffer_argmax_f16": (ctypes.c_int, [vp, i64, ctypes.POINTER(i64)]),
        "llmopt_hip_f16_argmax": (ctypes.c_int, [vp, i64, ctypes.POINTER(i64)]),
        "llmopt_hip_sample_f16": (ctypes.c_int, [vp, i64, ctypes.c_double, i64, ctypes.c_double, ctypes.c_double,
                                                 i64, ctypes.POINTER(i64)]),
        "llmopt_hip_dispatch": (ctypes.c_int, [vp, item_p]),
        "llmopt_hip_begin_batch": (ctypes.c_int, [vp, pp]),
        "llmopt_hip_release_batch": (None, [vp]),
        "llmopt_hip_batch_dispatch": (ctypes.c_int, [vp, vp, item_p]),
        "llmopt_hip_batch_dispatch_all": (ctypes.c_int, [vp, vp, item_p, sz]),
        "llmopt_hip_batch_copy": (ctypes.c_int, [vp, vp, vp]),
        "llmopt_hip_batch_barrier": (ctypes.c_int, [vp]),
        "llmopt_hip_commit_batch": (ctypes.c_int, [vp]),
        "llmopt_hip_commit_batch_async": (ctypes.c_int, [vp]),
        "llmopt_hip_commit_batch_profiled": (ctypes.c_int, [vp, ctypes.c_int, ctypes.c_int,
                                                           ctypes.POINTER(ctypes.c_float)]),
        "llmopt_hip_commit_batch_profiled_each": (ctypes.c_int, [vp, ctypes.c_int, ctypes.c_int,
                                                                ctypes.POINTER(ctypes.c_float)]),
        "llmopt_hip_abort_batch": (ctypes.c_int, [vp]),
        "llmopt_hip_prebaked_create": (ctypes.c_int, [vp, item_p, sz, vp, vp, pp]),
        "llmopt_hip_release_prebaked": (None, [vp]),
        "llmopt_hip_prebaked_execute": (ctypes.c_int, [vp, i64, i64, i64, ctypes.POINTER(i64)]),
        "llmopt_hip_prebaked_is_single_submission": (ctypes.c_int, [vp]),
        "llmopt_hip_ring_create": (ctypes.c_int, [pp]),
        "llmopt_hip_ring_submit": (ctypes.c_int, [vp, i64, i64, i64, i64]),
        "llmopt_hip_ring_wait_completion": (ctypes.c_int, [vp, ctypes.POINTER(i64), ctypes.POINTER(i64),
                                                           ctypes.POINTER(i64)]),
        "llmopt_hip_ring_poll_completion": (ctypes.c_int, [vp, ctypes.POINTER(i64), ctypes.POINTER(i64),
                                                           ctypes.POINTER(i64)]),
        "llmopt_hip_ring_start_worker": (ctypes.c_int, [vp, vp, item_p, sz, vp, vp]),
        "llmopt_hip_ring_start_worker_with": (ctypes.c_int, [vp, RING_STEP, vp]),
        "llmopt_hip_ring_destroy": (None, [vp]),
        "llmopt_hip_attention_q8_paged_no_alloc": (ctypes.c_int, [vp, vp, vp, vp, vp, vp, sz, vp, sz, vp]),
    }
    for name, (restype, argtypes) in signatures.items():
        function = getattr(handle, name)
        function.restype = restype
        function.argtypes = argtypes
    _lib = handle
    return handle


# Every symbol include/llmopt_hip.h declares (checked by the CPU test-suite).
EXPORTED_SYMBOLS = (
    "llmopt_hip_last_error", "llmopt_hip_create_context", "llmopt_hip_release_context",
    "llmopt_hip_device_name", "llmopt_hip_context_set_stream", "llmopt_hip_context_synchronize",
    "llmopt_hip_load_library", "llmopt_hip_release_library", "llmopt_hip_has_function",
    "llmopt_hip_preload_pipeline", "llmopt_hip_function_count", "llmopt_hip_function_name",
    "llmopt_hip_buffer_of_bytes", "llmopt_hip_create_buffer", "llmopt_hip_map_file",
    "llmopt_hip_buffer_view", "llmopt_hip_buffer_wrap", "llmopt_hip_release_buffer",
    "llmopt_hip_buffer_contents", "llmopt_hip_buffer_length", "llmopt_hip_buffer_device_pointer",
    "llmopt_hip_buffer_copy", "llmopt_hip_buffer_write", "llmopt_hip_buffer_set_int64",
    "llmopt_hip_buffer_set_u32_array", "llmopt_hip_buffer_argmax_f16", "llmopt_hip_f16_argmax",
    "llmopt_hip_sample_f16", "llmopt_hip_dispatch",
    "llmopt_hip_begin_batch", "llmopt_hip_release_batch", "llmopt_hip_batch_dispatch",
    "llmopt_hip_batch_dispatch_all", "llmopt_hip_batch_copy", "llmopt_hip_batch_barrier",
    "llmopt_hip_commit_batch", "llmopt_hip_commit_batch_async",
    "llmopt_hip_commit_batch_profiled", "llmopt_hip_commit_batch_profiled_each", "llmopt_hip_abort_batch",
    "llmopt_hip_prebaked_create", "llmopt_hip_release_prebaked", "llmopt_hip_prebaked_execute",
    "llmopt_hip_prebaked_is_single_submission",
    "llmopt_hip_ring_create", "llmopt_hip_ring_submit", "llmopt_hip_ring_wait_completion",
    "llmopt_hip_ring_poll_completion", "llmopt_hip_ring_start_worker", "llmopt_hip_ring_start_worker_with",
    "llmopt_hip_ring_destroy",
    "llmopt_hip_attention_q8_paged_no_alloc",
)


def _check(status: int) -> None:
    if status < 0:
        message = lib().llmopt_hip_last_error()
        raise LlmoptError(message.decode() if message else "unknown llmopt_hip failure", status)


class Buffer:
    """Device buffer handle (Metal_native.Buffer, lib/metal_native.ml:375-400)."""

    def __init__(self, handle: int, runtime: "Runtime"):
        self._handle = ctypes.c_void_p(handle)
        self.runtime = runtime

    @property
    def handle(self) -> ctypes.c_void_p:
        if not self._handle:
            raise LlmoptError("HIP buffer has been finalized")
        return self._handle

    def release(self) -> None:
        if self._handle:
            lib().llmopt_hip_release_buffer(self._handle)
            self._handle = ctypes.c_void_p(None)

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass

    @property
    def byte_length(self) -> int:
        length = lib().llmopt_hip_buffer_length(self.handle)
        _check(length)
        return int(length)

    @property
    def device_pointer(self) -> int:
        return int(lib().llmopt_hip_buffer_device_pointer(self.handle) or 0)

    def view(self, offset: int, nbytes: int) -> "Buffer":
        out = ctypes.c_void_p()
        _check(lib().llmopt_hip_buffer_view(self.handle, offset, nbytes, ctypes.byref(out)))
        return Buffer(out.value, self.runtime)

    def contents(self) -> bytes:
        length = self.byte_length
        out = ctypes.create_string_buffer(length)
        _check(lib().llmopt_hip_buffer_contents(self.handle, out, length))
        return out.raw

    def numpy(self, dtype, shape=None) -> np.ndarray:
        array = np.frombuffer(self.contents(), dtype=dtype).copy()
        return array if shape is None else array.reshape(shape)

    def write(self, data, offset: int = 0) -> None:
        raw = np.ascontiguousarray(data).tobytes() if not isinstance(data, (bytes, bytearray)) else bytes(data)
        _check(lib().llmopt_hip_buffer_write(self.handle, offset, raw, len(raw)))

    def copy_to(self, destination: "Buffer") -> None:
        _check(lib().llmopt_hip_buffer_copy(self.handle, destination.handle))

    def set_int64(self, offset: int, value: int) -> None:
        _check(lib().llmopt_hip_buffer_set_int64(self.handle, offset, value))

    def set_u32_array(self, offset: int, values: Sequence[int]) -> None:
        array = (ctypes.c_int64 * len(values))(*values)
        _check(lib().llmopt_hip_buffer_set_u32_array(self.handle, offset, array, len(values)))

    def argmax_f16(self, vocabulary: int) -> int:
        out = ctypes.c_int64()
        _check(lib().llmopt_hip_buffer_argmax_f16(self.handle, vocabulary, ctypes.byref(out)))
        return int(out.value)


def _make_item(name: str, buffers: Sequence[Buffer], parameters: bytes,
               grid=(1, 1, 1), group=(1, 1, 1), barrier_before: bool = False):
    """Builds a DispatchItem plus the objects that must outlive the call."""
    handles = (ctypes.c_void_p * max(1, len(buffers)))(*[b.handle for b in buffers])
    raw = ctypes.create_string_buffer(bytes(parameters), len(parameters)) if parameters else None
    encoded = name.encode()
    item = DispatchItem()
    item.name = encoded
    item.buffers = ctypes.cast(handles, ctypes.POINTER(ctypes.c_void_p))
    item.buffer_count = len(buffers)
    item.parameters = ctypes.cast(raw, ctypes.c_void_p) if raw is not None else None
    item.parameter_bytes = len(parameters) if parameters else 0
    item.grid = (ctypes.c_int64 * 3)(*grid)
    item.group = (ctypes.c_int64 * 3)(*group)
    item.barrier_before = int(barrier_before)
    return item, (handles, raw, encoded)


NO_ALLOC_SCRATCH_BYTES = 8 << 20  # LLMOPT_NO_ALLOC_SCRATCH_BYTES


def attention_q8_paged_no_alloc(parameters: bytes, query: Buffer, current_key: Buffer, current_value: Buffer,
                                pool: Buffer, slots: Buffer, output: Buffer, stream: int = 0) -> None:
    """llmopt_hip_attention_q8_paged_no_alloc: paged Q8 decode attention that allocates nothing
    (partial results in a fixed array of the library).  Queued on `stream`, not waited for."""
    raw = ctypes.create_string_buffer(bytes(parameters), len(parameters))
    if len(parameters) != 64:
        raise LlmoptError("Q8PagedAttentionParams is a 64-byte block", -2)
    _check(lib().llmopt_hip_attention_q8_paged_no_alloc(
        ctypes.c_void_p(stream), raw, query.device_pointer, current_key.device_pointer,
        current_value.device_pointer, pool.device_pointer, pool.byte_length, slots.device_pointer,
        slots.byte_length // 4, output.device_pointer))


class Runtime:
    """Context + library (the `t` of lib/metal_native.ml:130-135, minus the package)."""

    def __init__(self, device: int = -1, library_path: Optional[str] = None):
        self._context = ctypes.c_void_p()
        self._library = ctypes.c_void_p()
        _check(lib().llmopt_hip_create_context(device, ctypes.byref(self._context)))
        path = library_path.encode() if library_path else None
        _check(lib().llmopt_hip_load_library(self._context, path, ctypes.byref(self._library)))

    def close(self) -> None:
        if self._library:
            lib().llmopt_hip_release_library(self._library)
            self._library = ctypes.c_void_p()
        if self._context:
            lib().llmopt_hip_release_context(self._context)
            self._context = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def context(self):
        return self._context

    @property
    def library(self):
        return self._library

    def device_name(self) -> str:
        out = ctypes.create_string_buffer(256)
        _check(lib().llmopt_hip_device_name(self._context, out, 256))
        return out.value.decode()

    def set_stream(self, hip_stream: int) -> None:
        _check(lib().llmopt_hip_context_set_stream(self._context, ctypes.c_void_p(hip_stream)))

    def synchronize(self) -> None:
        _check(lib().llmopt_hip_context_synchronize(self._context))

    def has_function(self, name: str) -> bool:
        status = lib().llmopt_hip_has_function(self._library, name.encode())
        _check(status)
        return status == 1

    def preload_pipeline(self, name: str) -> None:
        _check(lib().llmopt_hip_preload_pipeline(self._library, name.encode()))

    def function_names(self) -> list[str]:
        count = lib().llmopt_hip_function_count(self._library)
        _check(count)
        return [lib().llmopt_hip_function_name(self._library, i).decode() for i in range(count)]

    # ---- buffers ----
    def buffer_of_bytes(self, data) -> Buffer:
        raw = data if isinstance(data, (bytes, bytearray)) else np.ascontiguousarray(data).tobytes()
        out = ctypes.c_void_p()
        _check(lib().llmopt_hip_buffer_of_bytes(self._context, bytes(raw), len(raw), ctypes.byref(out)))
        return Buffer(out.value, self)

    def create_buffer(self, nbytes: int) -> Buffer:
        out = ctypes.c_void_p()
        _check(lib().llmopt_hip_create_buffer(self._context, nbytes, ctypes.byref(out)))
        return Buffer(out.value, self)

    def map_file(self, path: str) -> Buffer:
        out = ctypes.c_void_p()
        _check(lib().llmopt_hip_map_file(self._context, path.encode(), ctypes.byref(out)))
        return Buffer(out.value, self)

    def wrap(self, device_pointer: int, nbytes: int) -> Buffer:
        out = ctypes.c_void_p()
        _check(lib().llmopt_hip_buffer_wrap(self._context, ctypes.c_void_p(device_pointer), nbytes,
                                            ctypes.byref(out)))
        return Buffer(out.value, self)

    # ---- dispatch ----
    def dispatch(self, name: str, buffers: Sequence[Buffer], parameters: bytes,
                 grid=(1, 1, 1), group=(1, 1, 1)) -> str:
        """Synchronous single dispatch (Metal_native.dispatch without a batch)."""
        item, keep = _make_item(name, buffers, parameters, grid, group)
        _check(lib().llmopt_hip_dispatch(self._library, ctypes.byref(item)))
        del keep
        return name

    def begin_batch(self) -> "Batch":
        return Batch(self)


class Batch:
    """Deferred dispatch list (Metal_native.Batch, lib/metal_native.ml:150-263)."""

    def __init__(self, runtime: Runtime):
        self.runtime = runtime
        self._handle = ctypes.c_void_p()
        _check(lib().llmopt_hip_begin_batch(runtime.library, ctypes.byref(self._handle)))
        self.kernels: list[str] = []

    def __del__(self):
        try:
            if self._handle:
                lib().llmopt_hip_release_batch(self._handle)
                self._handle = ctypes.c_void_p()
        except Exception:
            pass

    def dispatch(self, name: str, buffers: Sequence[Buffer], parameters: bytes,
                 grid=(1, 1, 1), group=(1, 1, 1)) -> str:
        item, keep = _make_item(name, buffers, parameters, grid, group)
        _check(lib().llmopt_hip_batch_dispatch(self._handle, self.runtime.library, ctypes.byref(item)))
        del keep
        self.kernels.append(name)
        return name

    def copy(self, source: Buffer, destination: Buffer) -> None:
        _check(lib().llmopt_hip_batch_copy(self._handle, source.handle, destination.handle))

    def barrier(self) -> None:
        _check(lib().llmopt_hip_batch_barrier(self._handle))

    def commit(self) -> None:
        _check(lib().llmopt_hip_commit_batch(self._handle))

    def commit_async(self) -> None:
        _check(lib().llmopt_hip_commit_batch_async(self._handle))

    def commit_profiled(self, repeats: int = 1, use_graph=True) -> float:
        """Runs the batch `repeats` times between HIP events; returns GPU milliseconds.
        use_graph: False (host launches), True (one graph, recorded order) or 2..4 (a graph of that
        many concurrent branches, for operations that do not depend on each other)."""
        elapsed = ctypes.c_float()
        _check(lib().llmopt_hip_commit_batch_profiled(self._handle, int(use_graph), repeats,
                                                      ctypes.byref(elapsed)))
        return float(elapsed.value)

    def commit_profiled_each(self, repeats: int = 3, use_graph=True) -> list[float]:
        """The same with every one of the `repeats` runs timed on its own: GPU milliseconds of each."""
        elapsed = (ctypes.c_float * repeats)()
        _check(lib().llmopt_hip_commit_batch_profiled_each(self._handle, int(use_graph), repeats, elapsed))
        return [float(value) for value in elapsed]

    def abort(self) -> None:
        _check(lib().llmopt_hip_abort_batch(self._handle))


class Prebaked:
    """Retained decode plan (Metal_native.Prebaked, lib/metal_native.ml:443-452)."""

    def __init__(self, runtime: Runtime, dispatches: Iterable[tuple], token_buffer: Buffer,
                 output_buffer: Buffer):
        self.runtime = runtime
        dispatches = list(dispatches)
        items = (DispatchItem * max(1, len(dispatches)))()
        keep = []
        for index, (name, buffers, parameters, grid, group) in enumerate(dispatches):
            item, alive = _make_item(name, buffers, parameters, grid, group)
            items[index] = item
            keep.append(alive)
        self._handle = ctypes.c_void_p()
        _check(lib().llmopt_hip_prebaked_create(runtime.library, items, len(dispatches),
                                                token_buffer.handle, output_buffer.handle,
                                                ctypes.byref(self._handle)))
        del keep

    def __del__(self):
        try:
            if self._handle:
                lib().llmopt_hip_release_prebaked(self._handle)
                self._handle = ctypes.c_void_p()
        except Exception:
            pass

    def execute(self, token: int, past_tokens: int, checkpoint: int = 0) -> int:
        out = ctypes.c_int64()
        _check(lib().llmopt_hip_prebaked_execute(self._handle, token, past_tokens, checkpoint,
                                                 ctypes.byref(out)))
        return int(out.value)

    @property
    def single_submission(self) -> bool:
        """True when a step replays one HIP graph."""
        status = lib().llmopt_hip_prebaked_is_single_submission(self._handle)
        _check(status)
        return status == 1


def _make_items(dispatches):
    dispatches = list(dispatches)
    items = (DispatchItem * max(1, len(dispatches)))()
    keep = []
    for index, (name, buffers, parameters, grid, group) in enumerate(dispatches):
        item, alive = _make_item(name, buffers, parameters, grid, group)
        items[index] = item
        keep.append(alive)
    return items, len(dispatches), keep


class Ring:
    """Submission / completion queues with one worker thread (Metal_native.Ring,
    lib/metal_native.ml:404-437)."""

    def __init__(self):
        self._handle = ctypes.c_void_p()
        self._callback = None
        _check(lib().llmopt_hip_ring_create(ctypes.byref(self._handle)))

    def submit(self, request_id: int, token: int, past_tokens: int, flags: int = 0) -> bool:
        status = lib().llmopt_hip_ring_submit(self._handle, request_id, token, past_tokens, flags)
        _check(status)
        return status == 1

    def wait_completion(self) -> tuple[int, int, int]:
        request, token, status = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        _check(lib().llmopt_hip_ring_wait_completion(self._handle, ctypes.byref(request), ctypes.byref(token),
                                                     ctypes.byref(status)))
        return int(request.value), int(token.value), int(status.value)

    def poll_completion(self) -> Optional[tuple[int, int, int]]:
        request, token, status = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        found = lib().llmopt_hip_ring_poll_completion(self._handle, ctypes.byref(request), ctypes.byref(token),
                                                      ctypes.byref(status))
        _check(found)
        return (int(request.value), int(token.value), int(status.value)) if found == 1 else None

    def start_worker(self, runtime: Runtime, dispatches: Iterable[tuple], token_buffer: Buffer,
                     output_buffer: Buffer) -> None:
        items, count, keep = _make_items(dispatches)
        _check(lib().llmopt_hip_ring_start_worker(self._handle, runtime.library, items, count,
                                                  token_buffer.handle, output_buffer.handle))
        del keep

    def start_worker_with(self, step) -> None:
        """`step(token, past_tokens) -> produced token` runs on the worker thread; an exception fails the step."""
        def trampoline(_user, token, past_tokens, out_token):
            try:
                out_token[0] = int(step(int(token), int(past_tokens)))
                return 0
            except Exception:
                return -1
        self._callback = RING_STEP(trampoline)
        _check(lib().llmopt_hip_ring_start_worker_with(self._handle, self._callback, None))

    def destroy(self) -> None:
        if self._handle:
            lib().llmopt_hip_ring_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
