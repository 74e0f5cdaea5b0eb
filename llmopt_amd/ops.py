"""The reference's dispatch_* operators (lib/metal_dispatch_linear.mli,
lib/metal_dispatch_attention.mli) over the HIP backend: a thin ctypes view of
the operator entry points declared in include/llmopt_hip_ops.h.

    ops = Operators(runtime)
    kernels = ops.w4a16_linear(m=1, n=1536, k=576, has_bias=False,
                               values=[Value(x, F16, (1, 576)), Value(w, U8, (1536, 288)),
                                       Value(s, F16, (1536, 9))],
                               output=Value(out, F16, (1, 1536)))

Each call returns the names of the kernels it dispatched (the reference's
`string list`) or raises LlmoptError with the reference's error string.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Sequence

from . import native
from .native import Batch, Buffer, LlmoptError, Runtime

F16, F32, U8, I32, I64, BOOL = range(6)


@dataclass
class Value:
    """An Ir.Value bound to its buffer: logical shape, dtype, device buffer."""
    buffer: Optional[Buffer]
    dtype: int
    shape: Sequence[int]


class _CValue(ctypes.Structure):
    _fields_ = [("buffer", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("rank", ctypes.c_uint32),
                ("dims", ctypes.c_int64 * 8)]


class _CKvLayer(ctypes.Structure):
    _fields_ = [("kv_heads", ctypes.c_int64), ("head_dim", ctypes.c_int64)]


class _CKvRegion(ctypes.Structure):
    _fields_ = [("key_offset", ctypes.c_int64), ("value_offset", ctypes.c_int64),
                ("segment_elements", ctypes.c_int64), ("segment_bytes", ctypes.c_int64)]


@dataclass(frozen=True)
class KvLayout:
    """Kv_cache.Layout of attention layers (lib/kv_cache.ml:52-61): token_elements int8 values per
    token, bytes_per_token (the pool slot stride) and (key_offset, value_offset, segment_elements,
    segment_bytes) per layer."""
    token_elements: int
    bytes_per_token: int
    regions: tuple


class _CPagedConfig(ctypes.Structure):
    _fields_ = [("token_elements", ctypes.c_int64), ("key_offset", ctypes.c_int64),
                ("value_offset", ctypes.c_int64), ("group_size", ctypes.c_int64),
                ("token_stride", ctypes.c_int64), ("scale", ctypes.c_double), ("window", ctypes.c_int64)]


OPERATOR_SYMBOLS = (
    "llmopt_op_context_create", "llmopt_op_context_release", "llmopt_op_context_set_batch",
    "llmopt_op_last_kernels", "llmopt_op_w4a16_linear", "llmopt_op_w4a16_qkv_linear",
    "llmopt_op_w4a16_swiglu_ffn", "llmopt_op_w4a16_lm_head_argmax", "llmopt_op_paged_attention_q8",
    "llmopt_op_attention",
    "llmopt_op_paged_attention_kernel_name", "llmopt_op_linear_f16_grid", "llmopt_op_simd_rows_grid",
    "llmopt_op_parameters_paged_attention_q8", "llmopt_op_kernel_operation",
    "llmopt_op_kv_bytes_for_elements", "llmopt_op_kv_layout",
)

_configured = False


def _lib() -> ctypes.CDLL:
    global _configured
    handle = native.lib()
    if not _configured:
        vp, i64, sz, dbl = ctypes.c_void_p, ctypes.c_int64, ctypes.c_size_t, ctypes.c_double
        values = ctypes.POINTER(_CValue)
        handle.llmopt_op_context_create.argtypes = [vp, vp, ctypes.POINTER(vp)]
        handle.llmopt_op_context_release.argtypes = [vp]
        handle.llmopt_op_context_release.restype = None
        handle.llmopt_op_context_set_batch.argtypes = [vp, vp]
        handle.llmopt_op_last_kernels.argtypes = [vp]
        handle.llmopt_op_last_kernels.restype = ctypes.c_char_p
        handle.llmopt_op_w4a16_linear.argtypes = [vp, i64, i64, i64, ctypes.c_int, values, sz, values]
        handle.llmopt_op_w4a16_qkv_linear.argtypes = [vp, i64, i64, i64, i64, i64, values, sz, values, values, sz]
        handle.llmopt_op_w4a16_swiglu_ffn.argtypes = [vp, i64, i64, i64, dbl, values, sz, values]
        handle.llmopt_op_w4a16_lm_head_argmax.argtypes = [vp, i64, i64, i64, dbl, values, sz, values, values, sz]
        handle.llmopt_op_paged_attention_q8.argtypes = [vp, ctypes.POINTER(_CPagedConfig), values, values,
                                                        values, values, values, values, sz, values]
        handle.llmopt_op_attention.argtypes = [vp, dbl, ctypes.c_int, values, values, values, values, values]
        handle.llmopt_op_paged_attention_kernel_name.argtypes = [ctypes.c_int, ctypes.c_int, i64, i64, i64]
        handle.llmopt_op_paged_attention_kernel_name.restype = ctypes.c_char_p
        handle.llmopt_op_linear_f16_grid.argtypes = [i64]
        handle.llmopt_op_linear_f16_grid.restype = i64
        handle.llmopt_op_simd_rows_grid.argtypes = [i64]
        handle.llmopt_op_simd_rows_grid.restype = i64
        handle.llmopt_op_parameters_paged_attention_q8.argtypes = [ctypes.c_char_p] + [i64] * 12 + [dbl] + [i64] * 3
        handle.llmopt_op_kernel_operation.argtypes = [ctypes.c_char_p]
        handle.llmopt_op_kernel_operation.restype = ctypes.c_char_p
        handle.llmopt_op_kv_bytes_for_elements.argtypes = [i64]
        handle.llmopt_op_kv_bytes_for_elements.restype = i64
        handle.llmopt_op_kv_layout.argtypes = [ctypes.POINTER(_CKvLayer), sz, ctypes.POINTER(_CKvRegion),
                                               ctypes.POINTER(i64), ctypes.POINTER(i64)]
        _configured = True
    return handle


# ---- pure helpers (no GPU needed) ---------------------------------------------------

def paged_attention_kernel_name(*, query_heads: int, kv_heads: int, head_dimension: int, split8: bool = False,
                                experimental_gqa3_split8: bool = False) -> str:
    """Paged_attention_tactic.kernel_name (lib/metal_dispatch_common.ml:41-57)."""
    return _lib().llmopt_op_paged_attention_kernel_name(int(experimental_gqa3_split8), int(split8), query_heads,
                                                        kv_heads, head_dimension).decode()


def linear_f16_grid(columns: int) -> int:
    """linear_f16_grid (lib/metal_dispatch_common.ml:64-70); raises on overflow."""
    grid = _lib().llmopt_op_linear_f16_grid(columns)
    if grid < 0:
        raise LlmoptError("Metal float16 linear grid dimension overflows")
    return grid


def parameters_paged_attention_q8(*, batches, query_heads, kv_heads, past_length, head_dimension, mask_batches,
                                  mask_heads, token_elements, key_offset, value_offset, group_size, token_stride,
                                  scale, mask_dtype, query_length=1, window=0) -> bytes:
    """Parameters.paged_attention_q8 (lib/metal_parameters.ml:119-140)."""
    out = ctypes.create_string_buffer(64)
    native._check(_lib().llmopt_op_parameters_paged_attention_q8(
        out, batches, query_heads, kv_heads, past_length, head_dimension, mask_batches, mask_heads,
        token_elements, key_offset, value_offset, group_size, token_stride, float(scale), mask_dtype,
        query_length, window))
    return out.raw


def kv_bytes_for_elements(elements: int) -> int:
    """Kv_cache.Format.bytes_for_elements (lib/kv_cache.ml:16-21)."""
    result = _lib().llmopt_op_kv_bytes_for_elements(elements)
    if result < 0:
        raise LlmoptError("KV element count cannot be negative" if elements < 0 else "Q8 KV byte length overflows")
    return result


def kv_layout(layers: Sequence[tuple]) -> KvLayout:
    """Kv_cache.Layout.create_heterogeneous over attention layers given as (kv_heads, head_dim)
    (lib/kv_cache.ml:80-166): where each layer's keys and values sit in a token's pool slot."""
    count = len(layers)
    c_layers = (_CKvLayer * max(1, count))(*[_CKvLayer(int(h), int(d)) for h, d in layers])
    regions = (_CKvRegion * max(1, count))()
    elements, stride = ctypes.c_int64(), ctypes.c_int64()
    native._check(_lib().llmopt_op_kv_layout(c_layers, count, regions, ctypes.byref(elements), ctypes.byref(stride)))
    return KvLayout(elements.value, stride.value,
                    tuple((r.key_offset, r.value_offset, r.segment_elements, r.segment_bytes)
                          for r in regions[:count]))


def kernel_operation(name: str) -> Optional[str]:
    """Kernel_abi.Operation.to_string of an implemented entry name, None if unknown."""
    result = _lib().llmopt_op_kernel_operation(name.encode())
    return result.decode() if result else None


# ---- operators ------------------------------------------------------------------------

def _values(items: Sequence[Value]):
    array = (_CValue * max(1, len(items)))()
    for slot, item in zip(array, items):
        slot.buffer = item.buffer.handle if item.buffer is not None else None
        slot.dtype = item.dtype
        slot.rank = len(item.shape)
        for axis, dim in enumerate(item.shape):
            slot.dims[axis] = dim
    return array


class Operators:
    """Metal_execution_state.context for the operator calls: runtime, open batch, scratch."""

    def __init__(self, runtime: Runtime):
        self.runtime = runtime
        handle = ctypes.c_void_p()
        native._check(_lib().llmopt_op_context_create(runtime.context, runtime.library, ctypes.byref(handle)))
        self._handle = handle
        self._batch: Optional[Batch] = None

    def close(self) -> None:
        if self._handle:
            _lib().llmopt_op_context_release(self._handle)
            self._handle = ctypes.c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_batch(self, batch: Optional[Batch]) -> None:
        """Operators record into `batch` until it is cleared (None = dispatch and wait)."""
        self._batch = batch
        native._check(_lib().llmopt_op_context_set_batch(self._handle, batch._handle if batch else None))

    def _done(self, status: int) -> list[str]:
        native._check(status)
        names = _lib().llmopt_op_last_kernels(self._handle).decode()
        return names.split("\n") if names else []

    def w4a16_linear(self, *, m, n, k, has_bias, values, output) -> list[str]:
        return self._done(_lib().llmopt_op_w4a16_linear(self._handle, m, n, k, int(has_bias), _values(values),
                                                        len(values), _values([output])))

    def w4a16_qkv_linear_command(self, *, m, k, n_q, n_k, n_v, extra_outputs, values, output) -> list[str]:
        return self._done(_lib().llmopt_op_w4a16_qkv_linear(
            self._handle, m, k, n_q, n_k, n_v, _values(values), len(values), _values([output]),
            _values(extra_outputs), len(extra_outputs)))

    def w4a16_swiglu_ffn_command(self, *, m, n, k, epsilon, values, output) -> list[str]:
        return self._done(_lib().llmopt_op_w4a16_swiglu_ffn(self._handle, m, n, k, float(epsilon),
                                                            _values(values), len(values), _values([output])))

    def w4a16_lm_head_argmax_command(self, *, m, n, k, epsilon, extra_outputs, values, output) -> list[str]:
        return self._done(_lib().llmopt_op_w4a16_lm_head_argmax(
            self._handle, m, n, k, float(epsilon), _values(values), len(values), _values([output]),
            _values(extra_outputs), len(extra_outputs)))

    def attention(self, *, scale: float, causal: bool, query, key, value, mask, output) -> list[str]:
        """dispatch_attention (lib/metal_dispatch_attention.ml:6-102): dense fp16 attention."""
        return self._done(_lib().llmopt_op_attention(
            self._handle, float(scale), int(bool(causal)), _values([query]), _values([key]), _values([value]),
            _values([mask]) if mask is not None else None, _values([output])))

    def paged_attention_q8(self, *, config: dict, query, current_key, current_value, pool, slots, mask_values,
                           output) -> list[str]:
        c = _CPagedConfig(config["token_elements"], config["key_offset"], config["value_offset"],
                          config.get("group_size", 64), config["token_stride"], float(config["scale"]),
                          config.get("window") or 0)
        return self._done(_lib().llmopt_op_paged_attention_q8(
            self._handle, ctypes.byref(c), _values([query]), _values([current_key]), _values([current_value]),
            _values([pool]), _values([slots]), _values(mask_values), len(mask_values), _values([output])))
