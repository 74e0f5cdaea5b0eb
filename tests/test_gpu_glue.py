"""GPU parity of the decode-step glue kernels (RMSNorm, RoPE, embedding, add,
LM-head argmax, buffer copy) through the C ABI.  Float results are compared
with the CPU oracle at the path's tolerance; where the reference kernel fixes
the rounding of every operation (half-precision RoPE, half add, gathers,
copies) the result must also equal IEEE half arithmetic bit for bit."""
import struct

import numpy as np
import pytest

import oracle
from tests.gpu_util import assert_close_to_oracle, linear_grid, u32s, w4_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def rms_params(rows, width, epsilon):
    return struct.pack("<IIf", rows, width, epsilon)


def test_rms_norm_reference_vector(runtime, golden):
    x = np.array([[1, 0, 0, 0], [0, 1, 0, 0]], dtype=np.float16)
    w = np.ones(4, dtype=np.float16)
    out = runtime.buffer_of_bytes(np.zeros_like(x))
    runtime.dispatch("llmopt_rms_norm_f16_simd", [runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(w), out],
                     rms_params(2, 4, 0.0), grid=(256, 1, 1), group=(256, 1, 1))
    assert out.numpy(np.uint16, (8,)).tolist() == golden["rms_norm"]["expected_output_bits"]


@pytest.mark.parametrize("rows,width", [(1, 576), (5, 576), (32, 4096), (3, 100)])
def test_rms_norm_matches_oracle(runtime, rows, width):
    rng = np.random.default_rng(rows * 1000 + width)
    x = (rng.standard_normal((rows, width)) * 3).astype(np.float16)
    w = rng.uniform(0.5, 1.5, width).astype(np.float16)
    out = runtime.buffer_of_bytes(np.full((rows, width), np.nan, dtype=np.float16))
    runtime.dispatch("llmopt_rms_norm_f16_simd", [runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(w), out],
                     rms_params(rows, width, 1e-5), grid=(((rows + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    assert_close_to_oracle(out.numpy(np.float16, (rows, width)), oracle.rms_norm(x, w, 1e-5), "rms_norm")


@pytest.mark.parametrize("dtype,name", [(np.float16, "llmopt_w4a16_swiglu_rms_f16_g64"),
                                        (np.float32, "llmopt_w4a16_swiglu_rms_f32_g64")])
def test_swiglu_rms_stage(runtime, dtype, name):
    rng = np.random.default_rng(11)
    m, n, k = 3, 1536, 576
    x = rng.standard_normal((m, k)).astype(dtype)
    w = rng.uniform(0.5, 1.5, k).astype(np.float16)
    out = runtime.buffer_of_bytes(np.full((m, k), np.nan, dtype=np.float16))
    runtime.dispatch(name, [runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(w), out],
                     u32s(m, n, k) + struct.pack("<f", 1e-5), grid=(m * 256, 1, 1), group=(256, 1, 1))
    assert_close_to_oracle(out.numpy(np.float16, (m, k)), oracle.rms_norm(x, w, 1e-5), name)


def rope_tables(tokens, d, rng):
    """cos/sin rows duplicated into both halves (lib/serving_rope_table.ml:156-172)."""
    inv_freq = (10000.0 ** (-np.arange(0, d, 2) / d)).astype(np.float32)
    positions = rng.integers(0, 4096, tokens)
    angle = (inv_freq[None, :] * positions[:, None].astype(np.float32)).astype(np.float32).astype(np.float64)
    cos = np.concatenate([np.cos(angle), np.cos(angle)], axis=1).astype(np.float32).astype(np.float16)
    sin = np.concatenate([np.sin(angle), np.sin(angle)], axis=1).astype(np.float32).astype(np.float16)
    return cos, sin


def half_rope(x, cos, sin):
    """The kernel's arithmetic in IEEE half: out = half(half(x*cos) + half(rot*sin)),
    token-major [t, heads, d] -> head-major [heads, t, d]."""
    tokens, heads, d = x.shape
    h = d // 2
    rotated = np.concatenate([-x[..., h:], x[..., :h]], axis=-1)
    direct = (x * cos[:, None, :]).astype(np.float16)
    turned = (rotated * sin[:, None, :]).astype(np.float16)
    return (direct + turned).astype(np.float16).transpose(1, 0, 2).copy()


@pytest.mark.parametrize("batches,tokens,q_heads,k_heads", [(1, 1, 9, 3), (1, 7, 9, 3), (3, 2, 4, 4)])
def test_rotary_qk_h64(runtime, batches, tokens, q_heads, k_heads):
    rng = np.random.default_rng(batches * 100 + tokens)
    d = 64
    q = rng.standard_normal((batches, tokens, q_heads, d)).astype(np.float16)
    k = rng.standard_normal((batches, tokens, k_heads, d)).astype(np.float16)
    cos, sin = rope_tables(tokens, d, rng)  # shared by all batches: trig_batches = 1
    q_out = runtime.buffer_of_bytes(np.full(q.size, np.nan, dtype=np.float16))
    k_out = runtime.buffer_of_bytes(np.full(k.size, np.nan, dtype=np.float16))
    rows = batches * (q_heads + k_heads) * tokens
    runtime.dispatch("llmopt_rotary_qk_f16_simd_h64",
                     [runtime.buffer_of_bytes(q), runtime.buffer_of_bytes(k), runtime.buffer_of_bytes(cos),
                      runtime.buffer_of_bytes(sin), q_out, k_out],
                     u32s(batches, tokens, q_heads, k_heads, d, d // 2, 1),
                     grid=(((rows + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    got_q = q_out.numpy(np.float16, (batches, q_heads, tokens, d))
    got_k = k_out.numpy(np.float16, (batches, k_heads, tokens, d))
    for b in range(batches):
        for got, source in ((got_q[b], q[b]), (got_k[b], k[b])):
            np.testing.assert_array_equal(got.view(np.uint16), half_rope(source, cos, sin).view(np.uint16))
            # the double-precision restatement differs only by the three half roundings
            expected = oracle.rotary_h(source, cos, sin)
            error = np.abs(got.astype(np.float64) - expected)
            assert float(error.max()) <= 3 * 2.0 ** -11 * max(1.0, float(np.abs(expected).max()))


@pytest.mark.parametrize("batches,q_heads,k_heads,d,trig_batches", [(1, 9, 3, 64, 1), (5, 9, 3, 64, 5),
                                                                     (33, 32, 8, 128, 33), (2, 4, 4, 128, 1)])
def test_rotary_pack_in_one_launch_equals_the_two_launches(runtime, batches, q_heads, k_heads, d, trig_batches):
    """The decode step's fused extension against the kernels it stands for, bit for bit: rotated
    queries and keys, and the Q8 bytes and scales of the new token's keys and values in the pool."""
    rng = np.random.default_rng(batches * 1000 + d)
    layers = 2
    elements = layers * 2 * k_heads * d
    stride = elements + 2 * (elements // 64)
    key_offset, value_offset = 2 * k_heads * d, 3 * k_heads * d  # the second layer's segments
    capacity = batches + 3
    q = rng.standard_normal((batches, 1, q_heads, d)).astype(np.float16)
    k = rng.standard_normal((batches, 1, k_heads, d)).astype(np.float16)
    v = rng.standard_normal((batches, k_heads, d)).astype(np.float16)
    v[0, 0, :64] = 0  # an all-zero group stores scale 1.0
    cos = np.concatenate([rope_tables(1, d, rng)[0] for _ in range(trig_batches)])
    sin = np.concatenate([rope_tables(1, d, rng)[1] for _ in range(trig_batches)])
    slots = rng.permutation(capacity)[:batches].astype(np.uint32)
    start = rng.integers(0, 256, size=capacity * stride, dtype=np.uint8)
    rotary_params = u32s(batches, 1, q_heads, k_heads, d, d // 2, trig_batches)
    pack_params = u32s(batches, key_offset, value_offset, k_heads, d, 64, elements, elements // 64, stride,
                       batches, 0)
    inputs = [runtime.buffer_of_bytes(x) for x in (q, k, cos, sin)]
    v_buffer, slot_buffer = runtime.buffer_of_bytes(v), runtime.buffer_of_bytes(slots)

    def outputs():
        return (runtime.buffer_of_bytes(np.full(q.size, np.nan, dtype=np.float16)),
                runtime.buffer_of_bytes(np.full(k.size, np.nan, dtype=np.float16)),
                runtime.buffer_of_bytes(start))

    q_two, k_two, pool_two = outputs()
    rows = batches * (q_heads + k_heads)
    runtime.dispatch("llmopt_rotary_qk_f16_simd_h64", [*inputs, q_two, k_two], rotary_params,
                     grid=(((rows + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    runtime.dispatch("llmopt_cache_pack_attention_q8_pair_batched", [k_two, v_buffer, slot_buffer, pool_two],
                     pack_params, grid=(batches * k_heads * (d // 64) * 64, 1, 1), group=(256, 1, 1))
    q_one, k_one, pool_one = outputs()
    runtime.dispatch("llmopt_rotary_qk_pack_q8_batched",
                     [*inputs, q_one, k_one, v_buffer, slot_buffer, pool_one], rotary_params + pack_params,
                     grid=(((batches * (q_heads + 2 * k_heads) + 3) // 4) * 256, 1, 1), group=(256, 1, 1))
    np.testing.assert_array_equal(q_one.numpy(np.uint16, (q.size,)), q_two.numpy(np.uint16, (q.size,)))
    np.testing.assert_array_equal(k_one.numpy(np.uint16, (k.size,)), k_two.numpy(np.uint16, (k.size,)))
    got = pool_one.numpy(np.uint8, (capacity, stride))
    np.testing.assert_array_equal(got, pool_two.numpy(np.uint8, (capacity, stride)))
    # and the two launches did write: the new slots differ from the starting bytes, the others do not
    before = start.reshape(capacity, stride)
    untouched = np.setdiff1d(np.arange(capacity), slots)
    np.testing.assert_array_equal(got[untouched], before[untouched])
    assert all((got[slot] != before[slot]).any() for slot in slots)
    # the values of the first sequence against the quantiser's definition
    first = got[slots[0]]
    scales = first[elements:].view(np.float16)
    assert scales[value_offset // 64] == np.float16(1.0) and not first[value_offset:value_offset + 64].any()
    group = v[0, 0, 64:128] if d == 128 else v[0, 1, :64]
    scale = np.float16(np.float32(np.abs(group).max()) / np.float32(127.0))
    assert scales[value_offset // 64 + 1] == scale
    expected = np.clip(np.rint(group.astype(np.float32) / np.float32(scale)), -127, 127).astype(np.int8)
    np.testing.assert_array_equal(first[value_offset + 64:value_offset + 128].view(np.int8), expected)


@pytest.mark.parametrize("batches,tokens,q_heads,k_heads,d,trig_batches", [(1, 37, 9, 3, 64, 1), (2, 5, 8, 2, 128, 2),
                                                                            (1, 300, 9, 3, 64, 1)])
def test_rotary_pack_of_a_prompt_equals_the_separate_launches(runtime, batches, tokens, q_heads, k_heads, d,
                                                              trig_batches):
    """Several tokens per sequence (a prefill): token-major Q, K and V in, head-major rotated Q and K
    out as llmopt_rotary_qk_f16_simd_h64 leaves them, and every token's K and V in its pool slot as
    two llmopt_cache_pack_attention_q8_simd launches leave them (K from the head-major rotated rows,
    V - token-major - as one head of k_heads * d values) - bit for bit."""
    rng = np.random.default_rng(tokens * 100 + d)
    elements = 2 * 2 * k_heads * d  # two layers; the second one is written
    stride = elements + 2 * (elements // 64)
    key_offset, value_offset = 2 * k_heads * d, 3 * k_heads * d
    items = batches * tokens
    capacity = items + 4
    q = rng.standard_normal((batches, tokens, q_heads, d)).astype(np.float16)
    k = rng.standard_normal((batches, tokens, k_heads, d)).astype(np.float16)
    v = rng.standard_normal((batches, tokens, k_heads, d)).astype(np.float16)
    cos = np.concatenate([rope_tables(tokens, d, rng)[0] for _ in range(trig_batches)])
    sin = np.concatenate([rope_tables(tokens, d, rng)[1] for _ in range(trig_batches)])
    slots = rng.permutation(capacity)[:items].astype(np.uint32)
    start = rng.integers(0, 256, size=capacity * stride, dtype=np.uint8)
    rotary_params = u32s(batches, tokens, q_heads, k_heads, d, d // 2, trig_batches)
    inputs = [runtime.buffer_of_bytes(x) for x in (q, k, cos, sin)]
    v_buffer, slot_buffer = runtime.buffer_of_bytes(v), runtime.buffer_of_bytes(slots)

    def outputs():
        return (runtime.buffer_of_bytes(np.full(q.size, np.nan, dtype=np.float16)),
                runtime.buffer_of_bytes(np.full(k.size, np.nan, dtype=np.float16)),
                runtime.buffer_of_bytes(start))

    q_two, k_two, pool_two = outputs()
    rows = items * (q_heads + k_heads)
    runtime.dispatch("llmopt_rotary_qk_f16_simd_h64", [*inputs, q_two, k_two], rotary_params,
                     grid=(((rows + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    # K head-major [k_heads, tokens, d] per sequence; V token-major as one head of k_heads * d values
    for b in range(batches):
        seq_slots = runtime.buffer_of_bytes(slots[b * tokens:(b + 1) * tokens])
        k_rows = k_two.view(b * k_heads * tokens * d * 2, k_heads * tokens * d * 2)
        v_rows = v_buffer.view(b * tokens * k_heads * d * 2, tokens * k_heads * d * 2)
        runtime.dispatch("llmopt_cache_pack_attention_q8_simd", [k_rows, seq_slots, pool_two],
                         u32s(tokens, key_offset, k_heads, d, 64, elements, elements // 64, stride, tokens, 0),
                         grid=(tokens * k_heads * (d // 64) * 64, 1, 1), group=(256, 1, 1))
        runtime.dispatch("llmopt_cache_pack_attention_q8_simd", [v_rows, seq_slots, pool_two],
                         u32s(tokens, value_offset, 1, k_heads * d, 64, elements, elements // 64, stride, tokens, 0),
                         grid=(tokens * k_heads * (d // 64) * 64, 1, 1), group=(256, 1, 1))
    q_one, k_one, pool_one = outputs()
    pack_params = u32s(items, key_offset, value_offset, k_heads, d, 64, elements, elements // 64, stride, items, 0)
    runtime.dispatch("llmopt_rotary_qk_pack_q8_batched",
                     [*inputs, q_one, k_one, v_buffer, slot_buffer, pool_one], rotary_params + pack_params,
                     grid=(((items * (q_heads + 2 * k_heads) + 3) // 4) * 256, 1, 1), group=(256, 1, 1))
    np.testing.assert_array_equal(q_one.numpy(np.uint16, (q.size,)), q_two.numpy(np.uint16, (q.size,)))
    np.testing.assert_array_equal(k_one.numpy(np.uint16, (k.size,)), k_two.numpy(np.uint16, (k.size,)))
    np.testing.assert_array_equal(pool_one.numpy(np.uint8, (capacity, stride)), pool_two.numpy(np.uint8, (capacity, stride)))


def test_rotary_pack_rejects_blocks_that_disagree(runtime):
    d, batches, heads = 64, 2, 3
    elements = 2 * heads * d
    stride = elements + 2 * (elements // 64)
    half = lambda count: runtime.buffer_of_bytes(np.zeros(count, dtype=np.float16))
    buffers = [half(batches * 9 * d), half(batches * heads * d), half(2 * d), half(2 * d), half(batches * 9 * d),
               half(batches * heads * d), half(batches * heads * d),
               runtime.buffer_of_bytes(np.arange(batches, dtype=np.uint32)),
               runtime.buffer_of_bytes(np.zeros(batches * stride, dtype=np.uint8))]
    pack = lambda items, kv: u32s(items, 0, heads * d, kv, d, 64, elements, elements // 64, stride, items, 0)
    for rotary, cache in ((u32s(batches, 1, 9, heads, d, d // 2, 1), pack(batches, 2)),
                          (u32s(batches, 1, 9, heads, d, d // 2, 1), pack(1, heads)),
                          (u32s(1, 1, 9, heads, d, d // 2, 1), pack(batches, heads))):
        with pytest.raises(Exception, match="requires the same tokens"):
            runtime.dispatch("llmopt_rotary_qk_pack_q8_batched", buffers, rotary + cache,
                             grid=(256, 1, 1), group=(256, 1, 1))


def test_embedding_gather_and_out_of_range(runtime):
    rng = np.random.default_rng(5)
    vocabulary, width = 1000, 576
    table = rng.standard_normal((vocabulary, width)).astype(np.float16)
    indices = np.array([0, 999, 17, -1, 1000, 500], dtype=np.int64)
    out = runtime.buffer_of_bytes(np.full((len(indices), width), np.nan, dtype=np.float16))
    count = len(indices) * width
    runtime.dispatch("llmopt_embedding_f16", [runtime.buffer_of_bytes(indices), runtime.buffer_of_bytes(table), out],
                     u32s(len(indices), vocabulary, width), grid=(((count + 255) // 256) * 256, 1, 1),
                     group=(256, 1, 1))
    expected = np.zeros((len(indices), width), dtype=np.float16)
    for i, index in enumerate(indices):
        if 0 <= index < vocabulary:
            expected[i] = table[index]
    np.testing.assert_array_equal(out.numpy(np.uint16, expected.shape), expected.view(np.uint16))


def pointwise_params(output_shape, left_shape, right_shape, left_scalar=None, right_scalar=None):
    """Parameters.pointwise (lib/metal_parameters.ml:350-380)."""
    rank = len(output_shape)
    align = lambda shape: [1] * (rank - len(shape)) + list(shape)
    pad = lambda shape: list(shape) + [1] * (8 - rank)
    block = bytearray(136)
    struct.pack_into("<4I", block, 0, int(np.prod(output_shape)), rank,
                     int(left_scalar is not None), int(right_scalar is not None))
    struct.pack_into("<8I", block, 16, *pad(output_shape))
    struct.pack_into("<8I", block, 48, *pad(align(left_shape)))
    struct.pack_into("<8I", block, 80, *pad(align(right_shape)))
    if left_scalar is not None:
        struct.pack_into("<f", block, 128, left_scalar)
    if right_scalar is not None:
        struct.pack_into("<f", block, 132, right_scalar)
    return bytes(block)


@pytest.mark.parametrize("left_shape,right_shape", [((4, 576), (4, 576)), ((3, 5, 7), (5, 1)), ((2, 9), (1,)),
                                                    ((1, 576), (6, 576))])
def test_add_f16_broadcast(runtime, left_shape, right_shape):
    rng = np.random.default_rng(len(left_shape) * 10 + len(right_shape))
    left = rng.standard_normal(left_shape).astype(np.float16)
    right = rng.standard_normal(right_shape).astype(np.float16)
    expected = (left + right).astype(np.float16)  # one rounding to half, like the kernel's half add
    out = runtime.buffer_of_bytes(np.full(expected.shape, np.nan, dtype=np.float16))
    runtime.dispatch("llmopt_add_f16", [runtime.buffer_of_bytes(left), runtime.buffer_of_bytes(right), out],
                     pointwise_params(expected.shape, left_shape, right_shape),
                     grid=(((expected.size + 255) // 256) * 256, 1, 1), group=(256, 1, 1))
    np.testing.assert_array_equal(out.numpy(np.uint16, expected.shape), expected.view(np.uint16))
    assert_close_to_oracle(out.numpy(np.float16, expected.shape),
                           oracle.add(np.broadcast_to(left, expected.shape).reshape(1, -1).copy(),
                                      np.broadcast_to(right, expected.shape).reshape(1, -1).copy()), "add")


def test_add_f16_scalar_operand(runtime):
    left = np.linspace(-4, 4, 100).astype(np.float16)
    out = runtime.buffer_of_bytes(np.zeros(100, dtype=np.float16))
    runtime.dispatch("llmopt_add_f16", [runtime.buffer_of_bytes(left), runtime.buffer_of_bytes(left), out],
                     pointwise_params((100,), (100,), (100,), right_scalar=0.5),
                     grid=(256, 1, 1), group=(256, 1, 1))
    np.testing.assert_array_equal(out.numpy(np.float16, (100,)), (left + np.float16(0.5)).astype(np.float16))


def test_add_rejects_non_broadcastable(runtime):
    from llmopt_amd.native import LlmoptError
    a = runtime.create_buffer(64)
    with pytest.raises(LlmoptError, match="not broadcastable"):
        runtime.dispatch("llmopt_add_f16", [a, a, a], pointwise_params((4, 4), (4, 4), (3,)),
                         grid=(256, 1, 1), group=(256, 1, 1))


@pytest.mark.parametrize("nbytes", [1, 15, 16, 4096 + 3, 1 << 20])
def test_buffer_copy_is_exact(runtime, nbytes):
    rng = np.random.default_rng(nbytes)
    data = rng.integers(0, 256, nbytes, dtype=np.uint8)
    source = runtime.buffer_of_bytes(data)
    destination = runtime.create_buffer(nbytes)
    source.copy_to(destination)
    np.testing.assert_array_equal(destination.numpy(np.uint8, (nbytes,)), data)
    # the batched form, from an unaligned view
    if nbytes > 16:
        batch = runtime.begin_batch()
        target = runtime.create_buffer(nbytes - 1)
        batch.copy(source.view(1, nbytes - 1), target)
        batch.commit()
        np.testing.assert_array_equal(target.numpy(np.uint8, (nbytes - 1,)), data[1:])


# ---- LM head -------------------------------------------------------------------

def lm_head_oracle(x, norm_weight, packed, scale, epsilon):
    normalized = oracle.rms_norm(x, norm_weight, epsilon)
    return oracle.w4a16_linear(normalized, packed, scale, None)


def run_lm_head(runtime, x, norm_weight, packed, scale, epsilon, extra=False, staged=False):
    m, k = x.shape
    n = packed.shape[0]
    suffix = "f32" if x.dtype == np.float32 else "f16"
    buffers = [runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(norm_weight), runtime.buffer_of_bytes(packed),
               runtime.buffer_of_bytes(scale)]
    tokens = runtime.buffer_of_bytes(np.full(m, 0xFFFFFFFF, dtype=np.uint32))
    logits = runtime.buffer_of_bytes(np.full((m, n), np.nan, dtype=np.float16)) if extra else None
    params = u32s(m, n, k) + struct.pack("<f", epsilon)
    tail = [logits] if extra else []
    if staged:
        candidates = runtime.create_buffer(m * 256 * 8)
        name = f"llmopt_w4a16_lm_head_argmax_stage1_{'extra_' if extra else ''}{suffix}"
        batch = runtime.begin_batch()
        batch.dispatch(name, buffers + [candidates] + tail, params, grid=(64 * 256, m, 1), group=(256, 1, 1))
        batch.dispatch("llmopt_w4a16_lm_head_reduce", [candidates, tokens], u32s(m),
                       grid=(m * 256, 1, 1), group=(256, 1, 1))
        batch.commit()
    else:
        name = f"llmopt_w4a16_lm_head_argmax_{'extra_' if extra else ''}{suffix}"
        runtime.dispatch(name, buffers + [tokens] + tail, params, grid=(m * 256, 1, 1), group=(256, 1, 1))
    return tokens.numpy(np.uint32, (m,)), (logits.numpy(np.float16, (m, n)) if extra else None)


def check_tokens(tokens, expected_logits):
    """The chosen column must hold the oracle's maximum; only logits closer than float32
    accumulation can separate (1e-5 x RMS) may swap."""
    rms = float(np.sqrt(np.mean(expected_logits.astype(np.float64) ** 2)))
    for row, token in enumerate(tokens):
        best = float(expected_logits[row].max())
        assert 0 <= token < expected_logits.shape[1]
        assert float(expected_logits[row, token]) >= best - 1e-5 * rms, (row, token)
        margin = np.partition(expected_logits[row], -2)[-2]
        if best - margin > 1e-5 * rms:
            assert token == oracle.argmax(expected_logits[row])


@pytest.mark.parametrize("m,n,k,dtype,extra,staged", [
    (1, 49152, 576, np.float16, False, True),   # the decode LM head, two-stage form
    (1, 1000, 576, np.float16, True, False),
    (2, 16400, 576, np.float16, True, False),   # a wide head with its logits
    (3, 2048, 640, np.float32, True, True),
    (8, 520, 2048, np.float16, False, False),
    (11, 300, 128, np.float16, True, False),    # more rows than one GEMV launch of eight takes: three row groups
    (32, 49152, 576, np.float16, False, False),  # the decode LM head at batch 32: 64 rows, eight row groups, one launch
    (70, 1024, 576, np.float16, True, False),   # 140 rows: two launches of row groups
    (9, 1040, 5120, np.float16, True, False),   # K split over workgroups: groups of eight rows, a launch each
])
def test_lm_head_argmax(runtime, m, n, k, dtype, extra, staged):
    rng = np.random.default_rng(m * 7 + n)
    x, packed, scale, _ = w4_case(rng, m, n, k)
    x = (x.astype(np.float32) * 2.5).astype(dtype)
    norm_weight = rng.uniform(0.5, 1.5, k).astype(np.float16)
    tokens, logits = run_lm_head(runtime, x, norm_weight, packed, scale, 1e-5, extra=extra, staged=staged)
    expected = lm_head_oracle(x, norm_weight, packed, scale, 1e-5)
    check_tokens(tokens, expected)
    if extra:
        assert_close_to_oracle(logits, expected, "lm head logits")


def test_lm_head_tie_goes_to_lowest_index(runtime):
    """lib/metal_w4a16_source.ml:1116-1117: equal logits -> lowest column."""
    rng = np.random.default_rng(3)
    m, n, k = 2, 700, 576
    x = np.abs(rng.standard_normal((m, k))).astype(np.float16)      # positive activations
    packed = np.full((n, k // 2), 0x88, dtype=np.uint8)             # every weight -8: very negative logits
    winner = np.full(k // 2, 0x77, dtype=np.uint8)                  # every weight +7: the maximum
    for column in (650, 123, 400):
        packed[column] = winner
    scale = np.full((n, k // 64), 0.01, dtype=np.float16)
    norm_weight = np.ones(k, dtype=np.float16)
    for staged in (False, True):
        tokens, _ = run_lm_head(runtime, x, norm_weight, packed, scale, 1e-5, staged=staged)
        assert tokens.tolist() == [123, 123]


def test_swiglu_ffn_three_stage_chain(runtime):
    """dispatch_w4a16_swiglu_ffn_command's launches (lib/metal_dispatch_linear.ml:346-395):
    RMSNorm -> half, silu(gate)*up -> half, down + residual -> half."""
    rng = np.random.default_rng(21)
    m, n, k = 1, 1536, 576
    x, gate_w, gate_s, _ = w4_case(rng, m, n, k)
    _, up_w, up_s, _ = w4_case(rng, m, n, k)
    _, down_w, down_s, _ = w4_case(rng, m, k, n)
    residual = rng.standard_normal((m, k)).astype(np.float16)
    norm_weight = rng.uniform(0.5, 1.5, k).astype(np.float16)
    params = u32s(m, n, k) + struct.pack("<f", 1e-5)
    b = runtime.buffer_of_bytes
    normalized, product = runtime.create_buffer(m * k * 2), runtime.create_buffer(m * n * 2)
    out = b(np.full((m, k), np.nan, dtype=np.float16))
    batch = runtime.begin_batch()
    batch.dispatch("llmopt_w4a16_swiglu_rms_f16_g64", [b(x), b(norm_weight), normalized], params,
                   grid=(m * 256, 1, 1), group=(256, 1, 1))
    batch.dispatch("llmopt_w4a16_dual_swiglu_f16_g64", [normalized, b(gate_w), b(gate_s), b(up_w), b(up_s), product],
                   params, grid=(linear_grid(m * n), 1, 1), group=(256, 1, 1))
    batch.dispatch("llmopt_w4a16_down_add_f16_g64", [product, b(down_w), b(down_s), b(residual), out], params,
                   grid=(linear_grid(m * k), 1, 1), group=(256, 1, 1))
    batch.commit()
    # oracle with the same half roundings between the stages
    norm = oracle.rms_norm(x, norm_weight, 1e-5).astype(np.float16)
    gate = oracle.w4a16_linear(norm, gate_w, gate_s, None)
    up = oracle.w4a16_linear(norm, up_w, up_s, None)
    prod = oracle.silu_mul(gate, up).astype(np.float16)
    expected = oracle.add(oracle.w4a16_linear(prod, down_w, down_s, None), residual.astype(np.float32))
    assert_close_to_oracle(out.numpy(np.float16, (m, k)), expected, "swiglu ffn chain")
