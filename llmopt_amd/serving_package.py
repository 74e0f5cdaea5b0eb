"""`package.llmopt`: the serving-package manifest of the reference (lib/serving_package.ml).

The manifest names the kernel artefact, the kernels a backend must provide (entry-point name,
operation, input / output dtype, threadgroup), the tensor store (`weights.llmopt`), the radix
cache page size, and carries the schedule and its memory plan.  This module reads and writes the
container byte for byte (lib/serving_package.ml:294-352 over the primitives of lib/binary.ml:
little-endian, strings as u32 length + bytes, blobs as u64 length + bytes) with the reference's
checks and error texts, and checks a manifest's kernel list against a loaded backend the way
Metal_native does before it serves a package (lib/metal_native.ml:271-284).

The schedule and the memory plan are Model Program IR (lib/serving_schedule_codec.ml,
lib/serving_memory_plan.ml): this backend executes dispatch lists, not IR, so the two blobs are
carried through unparsed and written back unchanged.
"""
from __future__ import annotations

import os
import stat
import struct
from dataclasses import dataclass, field
from typing import Optional

MAGIC = b"LLMOPTPK"
ABI_VERSION = 27  # lib/serving_package.ml:75

# lib/serving_package.ml:152-186 (tag) with lib/kernel_abi.ml:37-70 (name)
OPERATION_TAGS = {
    0: "matmul", 1: "fused-linear", 2: "linear", 5: "rms-norm", 6: "short-conv", 7: "attention", 8: "embedding",
    9: "arange", 10: "diff", 11: "cumsum", 12: "fill", 13: "gather2", 14: "cast", 15: "pointwise", 16: "movement",
    17: "reduction", 18: "update-slice", 19: "cache", 23: "rms-rope", 24: "short-conv-step",
    25: "short-conv-prefill", 26: "w4a16-lm-head-argmax", 27: "w4a16-linear-g64", 28: "w4a16-swiglu-ffn-g64",
    29: "w4a16-qkv-linear-g64", 30: "rms-rope-qk", 31: "triangular-recurrence", 32: "eye", 33: "batched-matmul",
    34: "gated-delta", 35: "gated-linear", 36: "rotary-qk", 37: "moe-swiglu-ffn",
}
OPERATION_OF_NAME = {name: tag for tag, name in OPERATION_TAGS.items()}

# lib/serving_package.ml:224-242 (tag) with Ir.Dtype.to_string (lib/ir.ml:22-61: name)
DTYPE_TAGS = {
    0: "f32", 1: "f16", 2: "bf16", 3: "i64", 4: "i32", 5: "i8", 6: "bool", 7: "u8",
    8: "Q8_0", 9: "Q4_K", 10: "Q5_K", 11: "Q6_K", 12: "Q5_0", 13: "Q4_0", 14: "IQ4_XS", 15: "Tile32_Affine4",
    16: "Tile32_Affine8", 17: "EXL3_4",
}
DTYPE_OF_NAME = {name: tag for tag, name in DTYPE_TAGS.items()}


class PackageError(ValueError):
    """The reference's `Error message` for a manifest that does not decode or validate."""


def artifact(path: str) -> str:
    """Serving_package.Artifact.create (lib/serving_package.ml:14-27): a canonical relative path."""
    path = path.strip()
    if path == "":
        raise PackageError("serving-package artifact path cannot be empty")
    if path.startswith("/"):
        raise PackageError("serving-package artifact path must be relative: " + path)
    if "\0" in path:
        raise PackageError("serving-package artifact path contains a NUL byte")
    if any(component in ("", ".", "..") for component in path.split("/")):
        raise PackageError("serving-package artifact path is not canonical: " + path)
    return path


@dataclass(frozen=True)
class KernelEntry:
    """Kernel_abi.Entry without a tile (lib/kernel_abi.ml:112-135; the manifest stores none)."""
    name: str
    operation: str
    input_dtype: str
    output_dtype: str
    threadgroup: tuple[int, int, int]

    def __post_init__(self):
        if self.name.strip() == "":
            raise PackageError("kernel entry-point name cannot be empty")
        if any(extent <= 0 for extent in self.threadgroup):
            raise PackageError("kernel threadgroup dimensions must be positive")
        if self.operation not in OPERATION_OF_NAME:
            raise PackageError("unsupported kernel operation: " + self.operation)
        if self.input_dtype not in DTYPE_OF_NAME or self.output_dtype not in DTYPE_OF_NAME:
            raise PackageError("unsupported kernel dtype")


@dataclass
class Package:
    """Serving_package.t (lib/serving_package.ml:63-73)."""
    stage: str                       # "compiled-graph" | "serving"
    kernel_library: str              # Files.metal_library: the kernel artefact's relative path
    kernels: list[KernelEntry]
    schedule: bytes                  # Serving_schedule.to_bytes, carried unparsed
    memory_plan: bytes               # Serving_memory_plan.to_bytes, carried unparsed
    model: Optional[str] = None
    tensor_store: Optional[str] = None   # Tensor_store.Weights { file }
    page_size: int = 1               # Cache.default
    abi_version: int = field(default=ABI_VERSION)

    def validate(self) -> None:
        """lib/serving_package.ml:77-94, minus the check that needs the parsed schedule (a serving
        package whose schedule has no tensor-store inputs)."""
        if self.stage not in ("compiled-graph", "serving"):
            raise PackageError("unknown serving-package stage: " + self.stage)
        if self.model is not None and self.model.strip() == "":
            raise PackageError("serving-package model identifier cannot be empty")
        if not self.kernels:
            raise PackageError("serving-package must declare at least one kernel")
        names = [kernel.name for kernel in self.kernels]
        if len(names) != len(set(names)):
            raise PackageError("serving-package kernel entry-point names must be unique")
        if self.stage == "compiled-graph" and self.tensor_store is not None:
            raise PackageError("compiled-graph package cannot declare a tensor store")
        if self.stage == "serving" and self.tensor_store is None:
            raise PackageError("serving-stage package must declare a tensor store")
        if self.page_size <= 0:
            raise PackageError("serving-package radix page_size must be positive")
        artifact(self.kernel_library)
        if self.tensor_store is not None:
            artifact(self.tensor_store)

    # ---- encoding (lib/serving_package.ml:294-311) ----
    def to_bytes(self) -> bytes:
        self.validate()
        out = bytearray(MAGIC)
        out += struct.pack("<HBB", self.abi_version, 0 if self.stage == "compiled-graph" else 1, 0)
        out += _option(self.model, _string)
        out += _string(self.kernel_library)
        if len(self.kernels) > 0xFFFF:
            raise PackageError("binary u16 value is out of range: %d" % len(self.kernels))
        out += struct.pack("<H", len(self.kernels))
        for kernel in self.kernels:
            out += _string(kernel.name)
            out += struct.pack("<BBB", OPERATION_OF_NAME[kernel.operation], DTYPE_OF_NAME[kernel.input_dtype],
                               DTYPE_OF_NAME[kernel.output_dtype])
            out += struct.pack("<III", *kernel.threadgroup)
        out += _option(self.tensor_store, lambda file: b"\x00" + _string(file))
        out += struct.pack("<I", self.page_size)
        out += struct.pack("<Q", len(self.schedule)) + bytes(self.schedule)
        out += struct.pack("<Q", len(self.memory_plan)) + bytes(self.memory_plan)
        return bytes(out)

    def write_file(self, path: str) -> None:
        try:
            with open(path, "wb") as handle:
                handle.write(self.to_bytes())
        except OSError as error:
            raise PackageError("cannot write serving package: " + str(error)) from error

    # ---- files and kernels a backend must have ----
    def validate_files(self, root: str) -> None:
        """Serving_package.validate_files (lib/serving_package.ml:392-419)."""
        for relative in [self.kernel_library] + ([self.tensor_store] if self.tensor_store else []):
            try:
                info = os.stat(os.path.join(root, relative))
            except OSError as error:
                raise PackageError("cannot access serving-package artifact %s: %s" % (relative, error.strerror))
            if not stat.S_ISREG(info.st_mode):
                raise PackageError("serving-package artifact is not a regular file: " + relative)

    def validate_declared_functions(self, runtime) -> None:
        """validate_declared_functions + preload_declared_pipelines (lib/metal_native.ml:271-284): every
        declared kernel must be an entry point of the loaded library."""
        for kernel in self.kernels:
            if not runtime.has_function(kernel.name):
                raise PackageError("HIP library does not define declared kernel: " + kernel.name)
        for kernel in self.kernels:
            runtime.preload_pipeline(kernel.name)


def _string(value: str) -> bytes:
    raw = value.encode()
    return struct.pack("<I", len(raw)) + raw


def _option(value, encode) -> bytes:
    return b"\x00" if value is None else b"\x01" + encode(value)


class _Reader:
    """Binary.Reader (lib/binary.ml:72-183) with its error texts."""

    def __init__(self, data: bytes):
        self.data, self.offset = bytes(data), 0

    def take(self, length: int) -> bytes:
        remaining = len(self.data) - self.offset
        if length > remaining:
            raise PackageError("truncated binary input at byte %d: need %d bytes, have %d"
                               % (self.offset, length, remaining))
        value = self.data[self.offset:self.offset + length]
        self.offset += length
        return value

    def u8(self) -> int:
        return self.take(1)[0]

    def u16(self) -> int:
        return struct.unpack("<H", self.take(2))[0]

    def u32(self) -> int:
        return struct.unpack("<I", self.take(4))[0]

    def u64(self) -> int:
        value = struct.unpack("<q", self.take(8))[0]
        if value < 0:
            raise PackageError("binary u64 value exceeds signed host range")
        return value

    def string(self) -> str:
        return self.take(self.u32()).decode()

    def blob(self) -> bytes:
        return self.take(self.u64())

    def option(self, read):
        tag = self.u8()
        if tag == 0:
            return None
        if tag == 1:
            return read()
        raise PackageError("unknown serving-package option tag: %d" % tag)

    def finish(self) -> None:
        remaining = len(self.data) - self.offset
        if remaining != 0:
            raise PackageError("binary input has %d trailing bytes" % remaining)


def of_bytes(data: bytes) -> Package:
    """Serving_package.of_bytes (lib/serving_package.ml:313-366)."""
    reader = _Reader(data)
    if reader.take(len(MAGIC)) != MAGIC:
        raise PackageError("invalid serving-package magic")
    version = reader.u16()
    if version != ABI_VERSION:
        raise PackageError("unsupported serving-package version: %d" % version)
    stage_tag = reader.u8()
    if stage_tag not in (0, 1):
        raise PackageError("unknown serving-package stage tag: %d" % stage_tag)
    target = reader.u8()
    if target != 0:
        raise PackageError("unsupported serving-package target tag: %d" % target)
    model = reader.option(reader.string)
    kernel_library = artifact(reader.string())
    kernels = []
    for _ in range(reader.u16()):
        name = reader.string()
        operation_tag, input_tag, output_tag = reader.u8(), reader.u8(), reader.u8()
        if operation_tag not in OPERATION_TAGS:
            raise PackageError("unknown kernel operation tag: %d" % operation_tag)
        for tag in (input_tag, output_tag):
            if tag not in DTYPE_TAGS:
                raise PackageError("unknown kernel dtype tag: %d" % tag)
        threadgroup = (reader.u32(), reader.u32(), reader.u32())
        kernels.append(KernelEntry(name, OPERATION_TAGS[operation_tag], DTYPE_TAGS[input_tag], DTYPE_TAGS[output_tag],
                                   threadgroup))

    def tensor_store():
        tag = reader.u8()
        if tag != 0:
            raise PackageError("unknown tensor-store tag: %d" % tag)
        return artifact(reader.string())

    store = reader.option(tensor_store)
    page_size = reader.u32()
    schedule = reader.blob()
    memory_plan = reader.blob()
    reader.finish()
    package = Package(stage="compiled-graph" if stage_tag == 0 else "serving", kernel_library=kernel_library,
                      kernels=kernels, schedule=schedule, memory_plan=memory_plan, model=model, tensor_store=store,
                      page_size=page_size)
    package.validate()
    return package


def of_file(path: str) -> Package:
    try:
        with open(path, "rb") as handle:
            return of_bytes(handle.read())
    except OSError as error:
        raise PackageError("cannot read serving package: " + str(error)) from error
