"""Host logic of the operator layer that needs no GPU: kernel selection, grids,
parameter blocks and the operation tags of the implemented entry names, checked
against the reference's own expectations."""
import struct

import pytest

from llmopt_amd import ops


def test_paged_kernel_selection_matches_the_reference_table(golden):
    """test/test_schedule.ml:1714-1755."""
    for case in golden["paged_kernel_selection"]["cases"]:
        assert ops.paged_attention_kernel_name(
            query_heads=case["query_heads"], kv_heads=case["kv_heads"], head_dimension=case["head_dim"],
            split8=case["split8"], experimental_gqa3_split8=case["experimental_gqa3_split8"]) == case["name"]


def test_benchmark_shapes_select_the_expected_kernels():
    # the 9/3 x 64 decode model and the 32/8 x 128 attention benchmark
    assert ops.paged_attention_kernel_name(query_heads=9, kv_heads=3, head_dimension=64) \
        == "llmopt_attention_q8_paged_simd_h64_gqa3"
    assert ops.paged_attention_kernel_name(query_heads=32, kv_heads=8, head_dimension=128) \
        == "llmopt_attention_q8_paged_simd_generic"
    assert ops.paged_attention_kernel_name(query_heads=8, kv_heads=8, head_dimension=512) \
        == "llmopt_attention_q8_paged_simd_h512"


def test_linear_f16_grid():
    """lib/metal_dispatch_common.ml:64-70: columns rounded up to 8 simdgroups of 32 threads."""
    assert ops.linear_f16_grid(1) == 256
    assert ops.linear_f16_grid(8) == 256
    assert ops.linear_f16_grid(9) == 512
    assert ops.linear_f16_grid(1536) == 1536 * 32
    with pytest.raises(ops.LlmoptError, match="overflows"):
        ops.linear_f16_grid((1 << 62) - 1)


def test_paged_attention_parameter_block_layout():
    """Offsets of Q8PagedAttentionParams (lib/metal_cache_source.ml:352-369): past_length at
    byte 12 (patched per step by the prebaked plan), scale f32 at 48, window at 60."""
    raw = ops.parameters_paged_attention_q8(
        batches=16, query_heads=32, kv_heads=8, past_length=4352, head_dimension=128, mask_batches=0,
        mask_heads=0, token_elements=2048, key_offset=0, value_offset=1024, group_size=64, token_stride=2112,
        scale=128 ** -0.5, mask_dtype=0, query_length=1, window=7)
    assert len(raw) == 64
    fields = struct.unpack("<12IfIII", raw)
    assert fields[:12] == (16, 32, 8, 4352, 128, 0, 0, 2048, 0, 1024, 64, 2112)
    assert struct.unpack_from("<I", raw, 12)[0] == 4352
    assert fields[12] == struct.unpack("<f", struct.pack("<f", 128 ** -0.5))[0]
    assert fields[13:] == (1, 0, 7)
    with pytest.raises(ops.LlmoptError, match="does not fit uint32"):
        ops.parameters_paged_attention_q8(
            batches=-1, query_heads=1, kv_heads=1, past_length=0, head_dimension=64, mask_batches=0,
            mask_heads=0, token_elements=128, key_offset=0, value_offset=64, group_size=64, token_stride=132,
            scale=1.0, mask_dtype=0)


def test_operation_tags_of_entry_names():
    """Kernel_abi.Operation.to_string (lib/kernel_abi.ml:37-70) per entry."""
    expected = {
        "llmopt_w4a16_linear_f16_g64": "w4a16-linear-g64",
        "llmopt_w4a16_linear_f16_g64_m4": "w4a16-linear-g64",
        "llmopt_w4a16_qkv_linear_f16_g64": "w4a16-qkv-linear-g64",
        "llmopt_w4a16_swiglu_rms_f16_g64": "w4a16-swiglu-ffn-g64",
        "llmopt_w4a16_dual_swiglu_f16_g64_m4": "w4a16-swiglu-ffn-g64",
        "llmopt_w4a16_down_add_f16_g64": "w4a16-swiglu-ffn-g64",
        "llmopt_w4a16_lm_head_argmax_stage1_f16": "w4a16-lm-head-argmax",
        "llmopt_w4a16_lm_head_reduce": "w4a16-lm-head-argmax",
        "llmopt_attention_q8_paged_simd_h64_gqa3": "attention",
        "llmopt_cache_pack_attention_q8_pair_simd": "cache",
        "llmopt_rms_norm_f16_simd": "rms-norm",
        "llmopt_rotary_qk_f16_simd_h64": "rotary-qk",
        "llmopt_embedding_f16": "embedding",
        "llmopt_add_f16": "pointwise",
    }
    for name, operation in expected.items():
        assert ops.kernel_operation(name) == operation, name
    assert ops.kernel_operation("llmopt_matmul_f32") is None


def test_operator_symbols_are_exported():
    import ctypes
    from llmopt_amd import native
    handle = ctypes.CDLL(native.LIBRARY_PATH)
    assert [name for name in ops.OPERATOR_SYMBOLS if not hasattr(handle, name)] == []


def test_header_and_python_list_the_same_operator_symbols():
    import os
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(root, "include", "llmopt_hip_ops.h")).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(llmopt_op_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(ops.OPERATOR_SYMBOLS)
