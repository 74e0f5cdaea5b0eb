"""Token selection from fp16 logits, the host mirror of the reference's `Sampling` module
(lib/sampling.ml): `Float16Logits` (last_row / suppress / top), `Params`, `Greedy` and `sample`,
with the reference's argument meaning and error strings.  Errors are raised as `SamplingError`
where the reference returns `Error message`.

The arithmetic lives in the native library (`llmopt_hip_f16_argmax`, `llmopt_hip_sample_f16`,
the counterparts of the externals at lib/sampling.ml:173,193-195); there is no Python fallback:
without the library these calls raise.
"""
from __future__ import annotations

import ctypes
import math
import struct
from dataclasses import dataclass
from typing import Iterable, Sequence

from . import native

MAX_INT = (1 << 62) - 1  # OCaml's max_int on a 64-bit host


class SamplingError(ValueError):
    """Carries the reference's error string."""


def float16(bits: int) -> float:
    """`Sampling.float16` (lib/sampling.ml:1-13): the value of 16 raw bits."""
    return struct.unpack("<e", struct.pack("<H", bits & 0xFFFF))[0]


class Float16Logits:
    """`Sampling.Float16_logits` (lib/sampling.ml:15-84)."""

    @staticmethod
    def row_offset(vocabulary: int, data: bytes) -> tuple[int, int]:
        if vocabulary <= 0:
            raise SamplingError("float16 logits vocabulary must be positive")
        if vocabulary > MAX_INT // 2:
            raise SamplingError("float16 logits vocabulary byte length overflows")
        row_bytes = 2 * vocabulary
        length = len(data)
        if length == 0 or length % row_bytes != 0:
            raise SamplingError(
                f"float16 logits contain {length} bytes; expected complete {row_bytes}-byte rows")
        return length - row_bytes, row_bytes

    @staticmethod
    def last_row(vocabulary: int, data: bytes) -> bytes:
        offset, row_bytes = Float16Logits.row_offset(vocabulary, data)
        return bytes(data[offset:offset + row_bytes])

    @staticmethod
    def suppress(vocabulary: int, suppress_token_ids: Sequence[int], row: bytes) -> bytes:
        seen = [False] * vocabulary
        count = 0
        for token_id in suppress_token_ids:
            if token_id < 0 or token_id >= vocabulary:
                raise SamplingError(f"suppressed token id {token_id} is outside vocabulary [0,{vocabulary})")
            if not seen[token_id]:
                count += 1
            seen[token_id] = True
        if count >= vocabulary:
            raise SamplingError("cannot suppress the complete sampling vocabulary")
        if not suppress_token_ids:
            return row
        masked = bytearray(row)
        for token_id, suppressed in enumerate(seen):
            if suppressed:
                masked[2 * token_id:2 * token_id + 2] = b"\x00\xfc"  # -inf
        return bytes(masked)

    @staticmethod
    def top(count: int, vocabulary: int, data: bytes, suppress_token_ids: Sequence[int] = ()) -> list[tuple[int, float]]:
        if count <= 0:
            raise SamplingError("float16 logits top count must be positive")
        row = Float16Logits.last_row(vocabulary, data)
        row = Float16Logits.suppress(vocabulary, suppress_token_ids, row)
        values = struct.unpack(f"<{vocabulary}e", row)
        for token_id, value in enumerate(values):
            if math.isnan(value):
                raise SamplingError(f"float16 logits contain NaN at token {token_id}")
        ranked = sorted(range(vocabulary), key=lambda token_id: (-values[token_id], token_id))
        return [(token_id, values[token_id]) for token_id in ranked[:min(count, vocabulary)]]


@dataclass(frozen=True)
class Params:
    """`Sampling.Params` (lib/sampling.ml:86-118)."""
    temperature: float = 0.0
    top_k: int = 1
    top_p: float = 1.0
    min_p: float = 0.0
    seed: int = 0

    @staticmethod
    def greedy() -> "Params":
        return Params(temperature=0.0, top_k=1, top_p=1.0, min_p=0.0, seed=0)

    @staticmethod
    def create(temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, min_p: float = 0.0,
               seed: int = 0) -> "Params":
        return Params(temperature=max(0.0, temperature), top_k=max(0, top_k),
                      top_p=max(0.0, min(1.0, top_p)), min_p=max(0.0, min(1.0, min_p)), seed=seed)

    def is_greedy(self) -> bool:
        return self.temperature <= 0.0001 or self.top_k == 1


def _argmax(row: bytes, vocabulary: int) -> int:
    out = ctypes.c_int64(0)
    buffer = ctypes.create_string_buffer(row, len(row))
    native._check(native.lib().llmopt_hip_f16_argmax(ctypes.cast(buffer, ctypes.c_void_p), vocabulary,
                                                     ctypes.byref(out)))
    return int(out.value)


class Greedy:
    """`Sampling.Greedy` (lib/sampling.ml:120-191)."""

    @staticmethod
    def _token_at(data: bytes, offset: int) -> int:
        return struct.unpack_from("<I", data, offset)[0]

    @staticmethod
    def on_device(data: bytes) -> int:
        if len(data) != 4:
            raise SamplingError(f"on-device greedy token must contain 4 bytes; got {len(data)}")
        return Greedy._token_at(data, 0)

    @staticmethod
    def on_device_last(data: bytes) -> int:
        if len(data) == 0 or len(data) % 4 != 0:
            raise SamplingError(
                f"on-device greedy token rows contain {len(data)} bytes; expected a positive multiple of 4")
        return Greedy._token_at(data, len(data) - 4)

    @staticmethod
    def on_device_all(data: bytes) -> list[int]:
        if len(data) == 0 or len(data) % 4 != 0:
            raise SamplingError(
                f"on-device greedy token rows contain {len(data)} bytes; expected a positive multiple of 4")
        return [Greedy._token_at(data, 4 * index) for index in range(len(data) // 4)]

    @staticmethod
    def f16_last_row(vocabulary: int, data: bytes, suppress_token_ids: Sequence[int] = ()) -> int:
        row = Float16Logits.last_row(vocabulary, data)
        row = Float16Logits.suppress(vocabulary, suppress_token_ids, row)
        return _argmax(row, vocabulary)

    @staticmethod
    def f16_all_rows(vocabulary: int, data: bytes, suppress_token_ids: Sequence[int] = ()) -> list[int]:
        _, row_bytes = Float16Logits.row_offset(vocabulary, data)
        return [Greedy.f16_last_row(vocabulary, data[index * row_bytes:(index + 1) * row_bytes], suppress_token_ids)
                for index in range(len(data) // row_bytes)]


def sample(params: Params, vocabulary: int, data: bytes, suppress_token_ids: Iterable[int] = ()) -> int:
    """`Sampling.sample` (lib/sampling.ml:197-207): the last row of `data`, after suppression,
    through the greedy path or the seeded sampler."""
    suppress_token_ids = list(suppress_token_ids)
    row = Float16Logits.last_row(vocabulary, data)
    row = Float16Logits.suppress(vocabulary, suppress_token_ids, row)
    if params.is_greedy():
        return _argmax(row, vocabulary)
    out = ctypes.c_int64(0)
    buffer = ctypes.create_string_buffer(row, len(row))
    native._check(native.lib().llmopt_hip_sample_f16(ctypes.cast(buffer, ctypes.c_void_p), vocabulary,
                                                     params.temperature, params.top_k, params.top_p, params.min_p,
                                                     params.seed, ctypes.byref(out)))
    return int(out.value)
