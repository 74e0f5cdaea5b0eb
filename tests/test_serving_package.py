"""`package.llmopt` manifests (llmopt_amd/serving_package.py) against the container layout of
lib/serving_package.ml:294-366: a manifest assembled here byte by byte from that description
decodes to the expected fields and encodes back to the same bytes; the reference's checks and
messages; the kernel list of a decode-step package against this backend's entry points.

The reference holds no package bytes (its tests round-trip in memory, test/exl3_runtime.ml:39-47),
so the byte-level vector below is written from the format's definition."""
import os
import struct

import pytest

from llmopt_amd import serving_package as sp


def s(text):
    raw = text.encode()
    return struct.pack("<I", len(raw)) + raw


def hand_built(version=27, stage=1, target=0, trailing=b""):
    out = b"LLMOPTPK" + struct.pack("<HBB", version, stage, target)
    out += b"\x01" + s("smollm2-135m")                       # Some model
    out += s("kernels/llmopt.hsaco")                         # kernel artefact
    out += struct.pack("<H", 2)
    out += s("llmopt_w4a16_linear_f16_g64") + bytes([27, 1, 1]) + struct.pack("<III", 256, 1, 1)
    out += s("llmopt_attention_q8_paged_simd_h64_gqa3") + bytes([7, 5, 1]) + struct.pack("<III", 32, 8, 1)
    out += (b"\x01" + b"\x00" + s("weights.llmopt")) if stage == 1 else b"\x00"
    out += struct.pack("<I", 16)                              # radix page size
    out += struct.pack("<Q", 5) + b"SCHED"
    out += struct.pack("<Q", 3) + b"MEM"
    return out + trailing


def test_hand_built_manifest_decodes_and_reencodes():
    raw = hand_built()
    package = sp.of_bytes(raw)
    assert package.stage == "serving" and package.model == "smollm2-135m"
    assert package.kernel_library == "kernels/llmopt.hsaco" and package.tensor_store == "weights.llmopt"
    assert package.page_size == 16 and package.schedule == b"SCHED" and package.memory_plan == b"MEM"
    assert package.kernels == [
        sp.KernelEntry("llmopt_w4a16_linear_f16_g64", "w4a16-linear-g64", "f16", "f16", (256, 1, 1)),
        sp.KernelEntry("llmopt_attention_q8_paged_simd_h64_gqa3", "attention", "i8", "f16", (32, 8, 1)),
    ]
    assert package.to_bytes() == raw


def test_compiled_graph_stage_has_no_tensor_store(tmp_path):
    package = sp.of_bytes(hand_built(stage=0))
    assert package.stage == "compiled-graph" and package.tensor_store is None
    path = tmp_path / "package.llmopt"
    package.write_file(str(path))
    assert sp.of_file(str(path)) == package


@pytest.mark.parametrize("raw,message", [
    (b"LLMOPTPX" + hand_built()[8:], "invalid serving-package magic"),
    (hand_built(version=26), "unsupported serving-package version: 26"),
    (hand_built(stage=2), "unknown serving-package stage tag: 2"),
    (hand_built(target=1), "unsupported serving-package target tag: 1"),
    (hand_built(trailing=b"xy"), "binary input has 2 trailing bytes"),
    (hand_built()[:40], "truncated binary input at byte 33: need 20 bytes, have 7"),
])
def test_decoder_rejects_with_the_reference_messages(raw, message):
    with pytest.raises(sp.PackageError) as error:
        sp.of_bytes(raw)
    assert str(error.value) == message


def test_unknown_tags_are_rejected():
    raw = bytearray(hand_built())
    at = raw.index(b"llmopt_w4a16_linear_f16_g64") + len("llmopt_w4a16_linear_f16_g64")
    for offset, value, message in ((0, 3, "unknown kernel operation tag: 3"), (1, 18, "unknown kernel dtype tag: 18")):
        broken = bytearray(raw)
        broken[at + offset] = value
        with pytest.raises(sp.PackageError) as error:
            sp.of_bytes(bytes(broken))
        assert str(error.value) == message


def test_validation_rules():
    kernel = sp.KernelEntry("k", "linear", "f16", "f16", (1, 1, 1))
    base = dict(kernel_library="k.hsaco", kernels=[kernel], schedule=b"", memory_plan=b"")
    cases = [
        (dict(base, stage="serving"), "serving-stage package must declare a tensor store"),
        (dict(base, stage="compiled-graph", tensor_store="w"), "compiled-graph package cannot declare a tensor store"),
        (dict(base, stage="compiled-graph", kernels=[]), "serving-package must declare at least one kernel"),
        (dict(base, stage="compiled-graph", kernels=[kernel, kernel]),
         "serving-package kernel entry-point names must be unique"),
        (dict(base, stage="compiled-graph", model="  "), "serving-package model identifier cannot be empty"),
        (dict(base, stage="compiled-graph", page_size=0), "serving-package radix page_size must be positive"),
        (dict(base, stage="compiled-graph", kernel_library="/abs/k"), "serving-package artifact path must be relative: /abs/k"),
        (dict(base, stage="compiled-graph", kernel_library="a/../k"), "serving-package artifact path is not canonical: a/../k"),
    ]
    for fields, message in cases:
        with pytest.raises(sp.PackageError) as error:
            sp.Package(**fields).to_bytes()
        assert str(error.value) == message
    with pytest.raises(sp.PackageError, match="kernel threadgroup dimensions must be positive"):
        sp.KernelEntry("k", "linear", "f16", "f16", (0, 1, 1))
    with pytest.raises(sp.PackageError, match="kernel entry-point name cannot be empty"):
        sp.KernelEntry(" ", "linear", "f16", "f16", (1, 1, 1))


def test_operation_and_dtype_tables_match_the_reference_tags():
    # spot values of lib/serving_package.ml:152-186,224-242
    assert sp.OPERATION_OF_NAME["w4a16-linear-g64"] == 27 and sp.OPERATION_OF_NAME["w4a16-qkv-linear-g64"] == 29
    assert sp.OPERATION_OF_NAME["w4a16-swiglu-ffn-g64"] == 28 and sp.OPERATION_OF_NAME["w4a16-lm-head-argmax"] == 26
    assert sp.OPERATION_OF_NAME["attention"] == 7 and sp.OPERATION_OF_NAME["cache"] == 19
    assert sp.OPERATION_OF_NAME["rotary-qk"] == 36 and sp.OPERATION_OF_NAME["embedding"] == 8
    assert len(sp.OPERATION_TAGS) == 33 and set(range(38)) - set(sp.OPERATION_TAGS) == {3, 4, 20, 21, 22}
    assert sp.DTYPE_OF_NAME["f16"] == 1 and sp.DTYPE_OF_NAME["i8"] == 5 and sp.DTYPE_OF_NAME["EXL3_4"] == 17


def test_validate_files(tmp_path):
    package = sp.of_bytes(hand_built())
    with pytest.raises(sp.PackageError, match="cannot access serving-package artifact kernels/llmopt.hsaco"):
        package.validate_files(str(tmp_path))
    os.makedirs(tmp_path / "kernels")
    (tmp_path / "kernels" / "llmopt.hsaco").write_bytes(b"x")
    os.makedirs(tmp_path / "weights.llmopt")
    with pytest.raises(sp.PackageError, match="serving-package artifact is not a regular file: weights.llmopt"):
        package.validate_files(str(tmp_path))
    os.rmdir(tmp_path / "weights.llmopt")
    (tmp_path / "weights.llmopt").write_bytes(b"x")
    package.validate_files(str(tmp_path))


class FakeRuntime:
    def __init__(self, names):
        self.names, self.preloaded = set(names), []

    def has_function(self, name):
        return name in self.names

    def preload_pipeline(self, name):
        self.preloaded.append(name)


def test_declared_kernels_are_checked_against_the_backend():
    package = sp.of_bytes(hand_built())
    names = [kernel.name for kernel in package.kernels]
    runtime = FakeRuntime(names)
    package.validate_declared_functions(runtime)
    assert runtime.preloaded == names
    with pytest.raises(sp.PackageError) as error:
        package.validate_declared_functions(FakeRuntime(names[:1]))
    assert str(error.value) == "HIP library does not define declared kernel: " + names[1]


@pytest.mark.gpu
def test_decode_step_package_is_served_by_the_library():
    """Every kernel of the decode step, declared in a manifest, is an entry point of the built library."""
    from llmopt_amd.native import Runtime
    runtime = Runtime()
    names = ["llmopt_embedding_f16", "llmopt_rms_norm_f16_simd", "llmopt_w4a16_qkv_linear_f16_g64",
             "llmopt_rotary_qk_f16_simd_h64", "llmopt_cache_pack_attention_q8_pair_simd",
             "llmopt_attention_q8_paged_simd_h64_gqa3", "llmopt_w4a16_linear_f16_g64",
             "llmopt_w4a16_dual_swiglu_f16_g64", "llmopt_w4a16_down_add_f16_g64", "llmopt_w4a16_lm_head_argmax_f16"]
    package = sp.Package(stage="serving", kernel_library="llmopt.hsaco", tensor_store="weights.llmopt",
                         kernels=[sp.KernelEntry(name, "linear", "f16", "f16", (256, 1, 1)) for name in names],
                         schedule=b"", memory_plan=b"")
    sp.of_bytes(package.to_bytes()).validate_declared_functions(runtime)
    bad = sp.Package(stage="serving", kernel_library="llmopt.hsaco", tensor_store="weights.llmopt",
                     kernels=[sp.KernelEntry("llmopt_conv2d_f16", "short-conv", "f16", "f16", (256, 1, 1))],
                     schedule=b"", memory_plan=b"")
    with pytest.raises(sp.PackageError, match="does not define declared kernel: llmopt_conv2d_f16"):
        bad.validate_declared_functions(runtime)
    runtime.close()
