"""`weights.llmopt` archives (magic LLMOPTWT, version 1): the reference's binary weight
container, read so that an engine directory built by the reference loads unchanged.

Layout (python/llmopt_backend/tensor_archive.py:19-118, lib/weight_archive.ml:165-296), all
little-endian:

    prefix   8s magic | u16 version = 1 | u16 flags = 0 | u32 tensor count | u64 index bytes
    entry    u32 name length | u8 dtype tag | u8 rank | u16 reserved = 0 | name (UTF-8)
             | rank x u64 dimension | u64 payload offset | u64 payload bytes
    padding  zero bytes up to `index bytes` (a multiple of 256)
    payload  every tensor at the next multiple of 256, in entry order, nothing after the last

Entries are strictly sorted by name.  The reader applies the same checks, with the same
messages, as lib/weight_archive.ml.  `WeightArchive` maps the file into one device buffer
(`Runtime.map_file`) and hands out 256-byte-aligned views of it, which is what the W4A16 and
glue kernels take as weight / scale / norm buffers.
"""
from __future__ import annotations

import os
import struct
from dataclasses import dataclass
from typing import Iterable, Mapping, Sequence

import numpy as np

MAGIC = b"LLMOPTWT"
VERSION = 1
ALIGNMENT = 256
_PREFIX = struct.Struct("<8sHHIQ")
_ENTRY_PREFIX = struct.Struct("<IBBH")

# tag order of python/llmopt_backend/tensor_archive.py:27-31
DTYPE_NAMES = (
    "float32", "float16", "bfloat16", "int64", "int32", "int8", "bool", "uint8",
    "Q8_0", "Q4_K", "Q5_K", "Q6_K", "Q5_0", "Q4_0", "IQ4_XS",
    "Tile32_Affine4", "Tile32_Affine8", "EXL3_4",
)
_ELEMENT_BYTES = {"float32": 4, "int32": 4, "float16": 2, "bfloat16": 2, "int64": 8, "int8": 1, "bool": 1,
                  "uint8": 1}
_NUMPY = {"float32": np.float32, "float16": np.float16, "int64": np.int64, "int32": np.int32, "int8": np.int8,
          "bool": np.bool_, "uint8": np.uint8, "bfloat16": np.uint16}


class ArchiveError(ValueError):
    """Carries the reference reader's error string."""


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: tuple[int, ...]
    offset: int
    byte_length: int


def _align(value: int) -> int:
    return (value + ALIGNMENT - 1) // ALIGNMENT * ALIGNMENT


def parse_index(data: bytes, file_size: int) -> list[TensorEntry]:
    """`data` = the first `index bytes` of the file (at least the 24-byte prefix to learn that length)."""
    if len(data) < _PREFIX.size:
        raise ArchiveError("weight archive file is too short")
    magic, version, flags, count, index_bytes = _PREFIX.unpack_from(data, 0)
    if magic != MAGIC:
        raise ArchiveError("invalid weight-archive magic")
    if version != VERSION:
        raise ArchiveError(f"unsupported weight-archive version: {version}")
    if flags != 0:
        raise ArchiveError(f"unsupported weight-archive flags: {flags}")
    if count == 0:
        raise ArchiveError("weight archive contains no tensors")
    if index_bytes < _PREFIX.size:
        raise ArchiveError("weight archive index is shorter than its prefix")
    if index_bytes % ALIGNMENT != 0:
        raise ArchiveError("weight archive index is not aligned")
    if index_bytes > file_size:
        raise ArchiveError("weight archive index extends beyond the file")
    if len(data) < index_bytes:
        raise ArchiveError("weight archive ended unexpectedly")
    cursor = _PREFIX.size
    entries: list[TensorEntry] = []
    previous = None

    def take(size: int) -> int:
        nonlocal cursor
        if cursor + size > index_bytes:
            raise ArchiveError("weight archive ended unexpectedly")
        cursor += size
        return cursor - size

    for _ in range(count):
        name_length, tag, rank, reserved = _ENTRY_PREFIX.unpack_from(data, take(_ENTRY_PREFIX.size))
        if tag >= len(DTYPE_NAMES):
            raise ArchiveError(f"unknown weight-archive dtype tag: {tag}")
        start = take(name_length)
        raw_name = data[start:start + name_length]
        if reserved != 0:
            raise ArchiveError("weight archive tensor reserved field is non-zero")
        if name_length == 0:
            raise ArchiveError("weight archive tensor name cannot be empty")
        if b"\x00" in raw_name:
            raise ArchiveError("weight archive tensor name contains a NUL byte")
        if previous is not None and previous >= raw_name:  # String.compare: byte order
            raise ArchiveError("weight archive tensor names are not strictly sorted")
        previous = raw_name
        name = raw_name.decode("utf-8", errors="replace")
        shape = struct.unpack_from(f"<{rank}Q", data, take(8 * rank)) if rank else ()
        offset, byte_length = struct.unpack_from("<QQ", data, take(16))
        elements = 1
        for dimension in shape:
            elements *= dimension
        if elements == 0 or byte_length == 0:
            raise ArchiveError(f"weight archive tensor {name} is empty")
        dtype = DTYPE_NAMES[tag]
        if dtype in _ELEMENT_BYTES and byte_length != elements * _ELEMENT_BYTES[dtype]:
            raise ArchiveError(f"weight archive tensor {name} byte length disagrees with its dtype and shape")
        if offset % ALIGNMENT != 0:
            raise ArchiveError(f"weight archive tensor {name} offset is not aligned")
        entries.append(TensorEntry(name, dtype, tuple(int(d) for d in shape), int(offset), int(byte_length)))
    if any(data[cursor:index_bytes]):
        raise ArchiveError("weight archive index padding contains non-zero bytes")
    cursor = index_bytes
    for entry in entries:
        expected = _align(cursor)
        if entry.offset != expected:
            raise ArchiveError(f"weight archive tensor {entry.name} has an unexpected payload offset")
        if expected > file_size or entry.byte_length > file_size - expected:
            raise ArchiveError(f"weight archive tensor {entry.name} exceeds the file")
        cursor = expected + entry.byte_length
    if cursor != file_size:
        raise ArchiveError("weight archive file has trailing or missing payload bytes")
    return entries


def read_index(path: str) -> list[TensorEntry]:
    if not os.path.isfile(path):
        raise ArchiveError("weight archive path is not a regular file: " + path)
    file_size = os.path.getsize(path)
    with open(path, "rb") as handle:
        prefix = handle.read(_PREFIX.size)
        if len(prefix) < _PREFIX.size:
            raise ArchiveError("weight archive file is too short")
        index_bytes = _PREFIX.unpack(prefix)[4]
        if index_bytes > file_size:
            raise ArchiveError("weight archive index extends beyond the file")
        rest = handle.read(max(0, index_bytes - _PREFIX.size))
    return parse_index(prefix + rest, file_size)


def write_archive(path: str, tensors: Mapping[str, np.ndarray], dtypes: Mapping[str, str] | None = None) -> list[
        TensorEntry]:
    """Writes `tensors` in the layout above (names sorted by their UTF-8 bytes).  `dtypes` names the
    archive dtype where numpy's does not say it (e.g. "bfloat16" held as uint16)."""
    if not tensors:
        raise ArchiveError("cannot write an empty llmopt weight archive")
    names = sorted(tensors, key=lambda name: name.encode("utf-8"))
    numpy_names = {np.dtype(v): k for k, v in _NUMPY.items() if k != "bfloat16"}
    specs = []
    index_bytes = _PREFIX.size
    for name in names:
        array = np.ascontiguousarray(tensors[name])
        dtype = (dtypes or {}).get(name) or numpy_names.get(array.dtype)
        if dtype is None:
            raise ArchiveError(f"tensor {name} has unsupported llmopt dtype {array.dtype}")
        if not name or "\x00" in name:
            raise ArchiveError(f"invalid llmopt tensor key: {name!r}")
        if array.nbytes == 0:
            raise ArchiveError(f"tensor {name} must contain at least one byte")
        specs.append((name, dtype, array))
        index_bytes += _ENTRY_PREFIX.size + len(name.encode("utf-8")) + 8 * array.ndim + 16
    data_start = _align(index_bytes)
    header = bytearray(_PREFIX.pack(MAGIC, VERSION, 0, len(specs), data_start))
    cursor = data_start
    entries = []
    for name, dtype, array in specs:
        cursor = _align(cursor)
        encoded = name.encode("utf-8")
        header += _ENTRY_PREFIX.pack(len(encoded), DTYPE_NAMES.index(dtype), array.ndim, 0) + encoded
        header += struct.pack(f"<{array.ndim}Q", *array.shape) + struct.pack("<QQ", cursor, array.nbytes)
        entries.append(TensorEntry(name, dtype, tuple(array.shape), cursor, array.nbytes))
        cursor += array.nbytes
    header += b"\x00" * (data_start - len(header))
    with open(path, "wb") as handle:
        handle.write(header)
        position = data_start
        for (name, dtype, array), entry in zip(specs, entries):
            handle.write(b"\x00" * (entry.offset - position))
            handle.write(array.tobytes())
            position = entry.offset + entry.byte_length
    return entries


class WeightArchive:
    """A `weights.llmopt` file mapped into device memory; `buffer(name)` is a view of its payload."""

    def __init__(self, runtime, path: str):
        self.entries = {entry.name: entry for entry in read_index(path)}
        self._runtime = runtime
        self._mapped = runtime.map_file(path)

    def names(self) -> Sequence[str]:
        return list(self.entries)

    def entry(self, name: str) -> TensorEntry:
        if name not in self.entries:
            raise KeyError(f"weight archive has no tensor {name}")
        return self.entries[name]

    def buffer(self, name: str):
        entry = self.entry(name)
        return self._mapped.view(entry.offset, entry.byte_length)

    def numpy(self, name: str) -> np.ndarray:
        entry = self.entry(name)
        if entry.dtype not in _NUMPY:
            raise ArchiveError(f"tensor {name} has no numpy dtype ({entry.dtype})")
        return self.buffer(name).numpy(_NUMPY[entry.dtype], entry.shape)

    def w4a16_pair(self, weight_name: str, scale_name: str):
        """(packed uint8 [N, K/2], f16 scales [N, K/64]) views after the shape checks of
        Tile.w4a16_linear (lib/tile.ml:106-160)."""
        weight, scale = self.entry(weight_name), self.entry(scale_name)
        if weight.dtype != "uint8" or len(weight.shape) != 2:
            raise ArchiveError(f"tensor {weight_name} is not a packed uint8 [N, K/2] weight")
        n, half_k = weight.shape
        if (2 * half_k) % 64 != 0:
            raise ArchiveError(f"tensor {weight_name}: K must be a multiple of 64")
        if scale.dtype != "float16" or scale.shape != (n, 2 * half_k // 64):
            raise ArchiveError(f"tensor {scale_name} is not the float16 [N, K/64] scale of {weight_name}")
        return self.buffer(weight_name), self.buffer(scale_name)
