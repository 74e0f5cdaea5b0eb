"""ctypes access to the CPU oracle (test infrastructure only).

Only tests, the smoke check and the bench's CPU-baseline leg import this.
The shipped library never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile oracle/llmopt_cpu_oracle.c with gcc (see oracle/Makefile)."""
    source = os.path.join(_HERE, "llmopt_cpu_oracle.c")
    stale = (
        force
        or not os.path.exists(_LIB_PATH)
        or (os.path.exists(source)
            and os.path.getmtime(source) > os.path.getmtime(_LIB_PATH))
    )
    if stale:
        subprocess.run(["make", "-B", "-C", _HERE, "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


class CacheParams(ctypes.Structure):
    """AttentionCacheParams, lib/metal_cache_source.ml:9-20."""
    _fields_ = [(name, ctypes.c_uint32) for name in (
        "items", "segment_offset", "heads", "head_dim", "group_size",
        "token_elements", "token_groups", "token_stride", "source_items",
        "source_offset")]


class PagedParams(ctypes.Structure):
    """Q8PagedAttentionParams, lib/metal_cache_source.ml:352-369."""
    _fields_ = [
        ("batches", ctypes.c_uint32), ("query_heads", ctypes.c_uint32),
        ("kv_heads", ctypes.c_uint32), ("past_length", ctypes.c_uint32),
        ("head_dim", ctypes.c_uint32), ("mask_batches", ctypes.c_uint32),
        ("mask_heads", ctypes.c_uint32), ("token_elements", ctypes.c_uint32),
        ("key_offset", ctypes.c_uint32), ("value_offset", ctypes.c_uint32),
        ("group_size", ctypes.c_uint32), ("token_stride", ctypes.c_uint32),
        ("scale", ctypes.c_float), ("query_length", ctypes.c_uint32),
        ("mask_dtype", ctypes.c_uint32), ("window", ctypes.c_uint32)]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        handle = ctypes.CDLL(_LIB_PATH)
        p = ctypes.c_void_p
        i64 = ctypes.c_int64
        handle.oracle_f16_to_f32.restype = ctypes.c_float
        handle.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        handle.oracle_f32_to_f16.restype = ctypes.c_uint16
        handle.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        handle.oracle_w4_unpack.restype = ctypes.c_int
        handle.oracle_w4_unpack.argtypes = [p, i64, i64, i64]
        handle.oracle_w4_dequant.argtypes = [p, p, p, i64, i64]
        handle.oracle_w4a16_linear.argtypes = [p, p, p, p, p, i64, i64, i64]
        handle.oracle_add.argtypes = [p, i64, p, i64, p, i64, i64]
        handle.oracle_silu.argtypes = [p, p, i64]
        handle.oracle_silu_mul.argtypes = [p, p, p, i64]
        handle.oracle_attention.argtypes = [
            p, p, p, p, p, i64, i64, i64, i64, i64, i64, i64, ctypes.c_double,
            ctypes.c_int]
        handle.oracle_q8_pack.argtypes = [p, p, p, ctypes.POINTER(CacheParams)]
        handle.oracle_q8_unpack.argtypes = [p, p, p, ctypes.POINTER(CacheParams)]
        handle.oracle_paged_attention_q8.argtypes = [
            p, p, p, p, p, p, p, ctypes.POINTER(PagedParams), p, p]
        handle.oracle_rms_norm.argtypes = [p, p, p, i64, i64, ctypes.c_double]
        handle.oracle_rotary_h.argtypes = [p, p, p, p, i64, i64, i64]
        handle.oracle_argmax.restype = i64
        handle.oracle_argmax.argtypes = [p, i64]
        _lib = handle
    return _lib


def _ptr(array):
    return None if array is None else array.ctypes.data_as(ctypes.c_void_p)


def _f32(array):
    return np.ascontiguousarray(array, dtype=np.float32)


def w4_dequant(packed: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """packed u8 [N,K/2], scale f16 [N,K/64] -> f32 [N,K]."""
    n, half_k = packed.shape
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    scale32 = _f32(scale)
    out = np.empty((n, half_k * 2), dtype=np.float32)
    lib().oracle_w4_dequant(_ptr(packed), _ptr(scale32), _ptr(out), n, half_k * 2)
    return out


def w4a16_linear(x, packed, scale, bias=None) -> np.ndarray:
    """x f16 [M,K], packed u8 [N,K/2], scale f16 [N,K/64], bias f16 [N] -> f32 [M,N]."""
    x32 = _f32(x)
    m, k = x32.shape
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    n = packed.shape[0]
    assert packed.shape[1] * 2 == k
    scale32 = _f32(scale)
    assert scale32.shape == (n, k // 64)
    bias32 = None if bias is None else _f32(bias).reshape(-1)
    out = np.empty((m, n), dtype=np.float32)
    lib().oracle_w4a16_linear(_ptr(x32), _ptr(packed), _ptr(scale32), _ptr(bias32),
                              _ptr(out), m, n, k)
    return out


def add(left, right) -> np.ndarray:
    left32, right32 = _f32(left), _f32(right)
    rows = max(left32.shape[0], right32.shape[0])
    cols = left32.shape[1]
    out = np.empty((rows, cols), dtype=np.float32)
    lib().oracle_add(_ptr(left32), left32.shape[0], _ptr(right32), right32.shape[0],
                     _ptr(out), rows, cols)
    return out


def silu(x) -> np.ndarray:
    x32 = _f32(x)
    out = np.empty_like(x32)
    lib().oracle_silu(_ptr(x32), _ptr(out), x32.size)
    return out


def silu_mul(left, right) -> np.ndarray:
    left32, right32 = _f32(left), _f32(right)
    out = np.empty_like(left32)
    lib().oracle_silu_mul(_ptr(left32), _ptr(right32), _ptr(out), left32.size)
    return out


def attention(query, key, value, mask, scale: float, causal: bool = False) -> np.ndarray:
    """query [b,h,q,d], key/value [b,h,L,d], mask [mb,mh,q,L] -> f32 [b,h,q,d]."""
    q32, k32, v32, m32 = _f32(query), _f32(key), _f32(value), _f32(mask)
    b, h, ql, d = q32.shape
    kl = k32.shape[2]
    out = np.empty_like(q32)
    lib().oracle_attention(_ptr(q32), _ptr(k32), _ptr(v32), _ptr(m32), _ptr(out),
                           b, h, ql, kl, d, m32.shape[0], m32.shape[1],
                           float(scale), int(causal))
    return out


def q8_pack(source_f16: np.ndarray, slots: np.ndarray, pool: np.ndarray,
            params: CacheParams) -> None:
    """Quantise head-major f16 source into pool (uint8, modified in place)."""
    source = np.ascontiguousarray(source_f16, dtype=np.float16).view(np.uint16)
    slots = np.ascontiguousarray(slots, dtype=np.uint32)
    assert pool.dtype == np.uint8 and pool.flags.c_contiguous
    lib().oracle_q8_pack(_ptr(source), _ptr(slots), _ptr(pool), ctypes.byref(params))


def q8_unpack(pool: np.ndarray, slots: np.ndarray, params: CacheParams) -> np.ndarray:
    slots = np.ascontiguousarray(slots, dtype=np.uint32)
    out = np.empty((params.heads, params.items, params.head_dim), dtype=np.uint16)
    lib().oracle_q8_unpack(_ptr(pool), _ptr(slots), _ptr(out), ctypes.byref(params))
    return out.view(np.float16)


def paged_attention_q8(query, current_key, current_value, pool, slots, mask,
                       params: PagedParams, past_lengths=None,
                       slot_offsets=None) -> np.ndarray:
    """Returns f32 token-major [b,q,h,D]."""
    q32, ck32, cv32 = _f32(query), _f32(current_key), _f32(current_value)
    slots = np.ascontiguousarray(slots, dtype=np.uint32)
    q_len = max(1, params.query_length)
    out = np.empty((params.batches, q_len, params.query_heads, params.head_dim),
                   dtype=np.float32)
    if mask is not None:
        mask = np.ascontiguousarray(mask)
        mask = mask.view(np.uint8)
    if past_lengths is not None:
        past_lengths = np.ascontiguousarray(past_lengths, dtype=np.uint32)
        slot_offsets = np.ascontiguousarray(slot_offsets, dtype=np.uint32)
    lib().oracle_paged_attention_q8(
        _ptr(q32), _ptr(ck32), _ptr(cv32), _ptr(pool), _ptr(slots), _ptr(mask),
        _ptr(out), ctypes.byref(params), _ptr(past_lengths), _ptr(slot_offsets))
    return out


def rms_norm(x, weight, epsilon: float) -> np.ndarray:
    x32, w32 = _f32(x), _f32(weight)
    out = np.empty_like(x32)
    lib().oracle_rms_norm(_ptr(x32), _ptr(w32), _ptr(out), x32.shape[0], x32.shape[1],
                          float(epsilon))
    return out


def rotary_h(x, cos_table, sin_table) -> np.ndarray:
    """x [tokens, heads, d] -> [heads, tokens, d]."""
    x32, c32, s32 = _f32(x), _f32(cos_table), _f32(sin_table)
    tokens, heads, d = x32.shape
    out = np.empty((heads, tokens, d), dtype=np.float32)
    lib().oracle_rotary_h(_ptr(x32), _ptr(c32), _ptr(s32), _ptr(out), tokens, heads, d)
    return out


def argmax(values) -> int:
    v32 = _f32(values).reshape(-1)
    return int(lib().oracle_argmax(_ptr(v32), v32.size))


def f32_to_f16_bits(value: float) -> int:
    return int(lib().oracle_f32_to_f16(ctypes.c_float(value)))


def f16_bits_to_f32(bits: int) -> float:
    return float(lib().oracle_f16_to_f32(ctypes.c_uint16(bits)))
