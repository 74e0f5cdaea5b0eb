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


def test_kv_layout_matches_the_reference_gemma_numbers():
    """test/test_cache.ml:183-320: 48 layers, every sixth one global (1 KV head of 512), the others
    sliding (8 KV heads of 256): 172 032 elements and 177 408 bytes per token, layer 5's keys at
    20 480 and values at 20 992, layer 6's keys at 21 504, a pool of 8 tokens 1 419 264 bytes."""
    import json
    import os
    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
    layers = [(1, 512) if (layer + 1) % 6 == 0 else (8, 256) for layer in range(48)]
    layout = ops.kv_layout(layers)
    assert layout.token_elements == golden["kv_layout_gemma"]["token_elements"] == 172032
    assert layout.bytes_per_token == golden["kv_layout_gemma"]["bytes_per_token"] == 177408
    assert layout.regions[5][:2] == (20480, 20992)
    assert layout.regions[6][0] == 21504
    assert layout.regions[5][2:] == (512, 512 + 2 * 8) and layout.regions[0][2:] == (2048, 2048 + 2 * 32)
    assert 8 * layout.bytes_per_token == 1419264


def test_kv_layout_of_the_benchmark_shapes_and_its_errors():
    from llmopt_amd.decode_step import DecodeConfig
    # C4: one layer of 8 KV heads of 128 -> 2048 + 64 bytes; C5: 30 layers of 3 KV heads of 64 -> 11 520 + 360
    assert ops.kv_layout([(8, 128)]).bytes_per_token == 2112
    config = DecodeConfig()
    assert (config.token_elements, config.token_stride, config.layer_elements) == (11520, 11880, 384)
    assert config.kv_layout.regions[7][:2] == (7 * 384, 7 * 384 + 192)
    # Kv_cache.Format.bytes_for_elements (lib/kv_cache.ml:10-21): a partial last group has a scale of its own
    assert [ops.kv_bytes_for_elements(n) for n in (0, 1, 64, 65, 128)] == [0, 3, 66, 69, 132]
    for layers, message in (([(0, 64)], "attention KV layer requires positive kv_heads"),
                            ([(2, 0)], "attention KV layer requires positive head_dim"),
                            ([(2, 96)], "Q8 KV group_size must divide each attention head dimension"),
                            ([(2 ** 40, 2 ** 30)], "attention KV layer element count overflows")):
        with pytest.raises(ops.LlmoptError, match=message):
            ops.kv_layout(layers)
    with pytest.raises(ops.LlmoptError):
        ops.kv_bytes_for_elements(-1)
