"""The fused decode-step launches (llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64,
llmopt_rms_w4a16_swiglu_down_partial_f16_g64, llmopt_sum_rms_w4a16_swiglu_down_partial_f16_g64,
llmopt_attention_q8_paged_batched_w4a16_partial_g64) against the launches they stand for and against
the CPU oracle, and the decode step built from them against the oracle's chain."""
import math
import struct

import numpy as np
import pytest

import oracle
from oracle import CacheParams
from oracle.chain import decode_chain, f16, rope_rows
from tests.gpu_util import assert_close_to_oracle, u32s

pytestmark = pytest.mark.gpu

GROUP = (256, 1, 1)


def drawn_cases():
    """Seeded random shapes for the fused entries, beside the hand-picked ones: rows, widths, head counts and
    pending sums anywhere the entries accept them."""
    rng = np.random.default_rng(20240607)
    qkv, ffn, summing, projecting = [], [], [], []
    for _ in range(10):
        kv = int(rng.integers(1, 5))
        qkv.append((int(rng.integers(1, 41)), 64 * int(rng.integers(1, 33)), (kv * int(rng.integers(1, 5)), kv, kv),
                    int(rng.integers(0, 33))))
        ffn.append((int(rng.integers(1, 41)), 64 * int(rng.integers(1, 33)), 64 * int(rng.integers(1, 24))))
        summing.append((int(rng.integers(1, 41)), 64 * int(rng.integers(1, 33)), 64 * int(rng.integers(1, 22)),
                        int(rng.integers(0, 33))))
        kv = int(rng.integers(1, 5))
        projecting.append((int(rng.integers(1, 41)), kv * int(rng.integers(1, 7)), kv, 64 * int(rng.integers(1, 17)),
                           int(rng.integers(64, 700))))
    return qkv, ffn, summing, projecting


DRAWN_QKV, DRAWN_FFN, DRAWN_SUMMING, DRAWN_PROJECTING = drawn_cases()


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def random_w4(rng, n, k):
    return (rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8),
            rng.uniform(0.005, 0.02, size=(n, k // 64)).astype(np.float16))


def pending_stream(rng, m, k, partial_count):
    """A residual stream as the fused launches hand it over: rows plus pending float32 partial sums,
    and the rows a reader forms from them (sums in ascending order, float32, one rounding to half)."""
    x = rng.standard_normal((m, k)).astype(np.float16)
    partials = (rng.standard_normal((max(1, partial_count), m, k)) * 0.2).astype(np.float32)
    total = np.zeros((m, k), dtype=np.float32)
    for p in range(partial_count):
        total = total + partials[p]
    stream = (total + x.astype(np.float32)).astype(np.float16) if partial_count else x
    return x, partials, stream


@pytest.mark.parametrize("m,k,heads,partial_count", [(1, 576, (9, 3, 3), 0), (1, 576, (9, 3, 3), 24), (3, 576, (9, 3, 3), 24),
                                                     (8, 576, (9, 3, 3), 24), (5, 1024, (4, 2, 2), 7), (2, 2048, (2, 1, 1), 32),
                                                     (40, 576, (9, 3, 3), 24), (37, 1536, (3, 1, 1), 3), (2, 64, (1, 1, 1), 1),
                                                     (1, 576, (9, 3, 3), 48), (8, 576, (9, 3, 3), 48), (23, 576, (9, 3, 3), 48),
                                                     (3, 1024, (4, 2, 2), 48)]
                         + DRAWN_QKV)
def test_fused_qkv_rotary_pack_against_separate_launches_and_oracle(runtime, m, k, heads, partial_count):
    rng = np.random.default_rng(1000 * m + k + partial_count)
    q_heads, k_heads, v_heads = heads
    assert k_heads == v_heads
    n = [64 * q_heads, 64 * k_heads, 64 * v_heads]
    layers, layer = 3, 1  # the new token's K / V go into the middle layer of a three-layer slot
    layer_elements = 2 * n[1]
    token_elements = layers * layer_elements
    stride = token_elements + 2 * (token_elements // 64)
    key_offset, value_offset = layer * layer_elements, layer * layer_elements + n[1]
    capacity = m + 3
    new_slots = rng.permutation(capacity).astype(np.uint32)[:m]
    pool = rng.integers(0, 256, size=capacity * stride, dtype=np.uint8)
    x, partials, stream = pending_stream(rng, m, k, partial_count)
    gain = rng.uniform(0.5, 1.5, k).astype(np.float16)
    weights = [random_w4(rng, count, k) for count in n]
    positions = rng.integers(0, 5000, size=m)

    class Rope:
        head_dim, rope_theta = 64, 10000.0
    cos, sin = rope_rows(Rope, positions)
    b = runtime.buffer_of_bytes
    device_w = [(b(w), b(s)) for w, s in weights]
    outputs = {name: b(np.full(m * width, np.nan, dtype=np.float16)) for name, width in zip("qkv", n)}
    stream_out = b(np.full(m * k, np.nan, dtype=np.float16))
    device_pool = b(pool)
    epsilon = 1e-5
    runtime.dispatch("llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64",
                     [b(x), b(partials), stream_out, b(gain), *device_w[0], *device_w[1], *device_w[2],
                      b(np.concatenate([cos, sin])), outputs["q"], outputs["k"], outputs["v"], b(new_slots), device_pool],
                     u32s(m, k, *n) + struct.pack("<f", epsilon) +
                     u32s(partial_count, key_offset, value_offset, token_elements, stride), grid=(256, 1, 1), group=GROUP)
    # the stream the launch formed and stored: the partial sums are added in float32 in a fixed order of
    # the kernel's own (groups of threads share them), then rounded once: the half nearest the exact sum,
    # or its neighbour where float32 rounding moved a sum across a rounding boundary
    got_stream = stream_out.numpy(np.float16, (m, k))
    assert np.all(np.isfinite(got_stream))
    step = np.spacing(np.abs(stream)).astype(np.float64)  # one half ulp step at the expected value
    # (where the operands cancel, the float32 rounding of another summation order - 2^-23 of the operands -
    # is itself several steps of the small result)
    operands = np.abs(x).astype(np.float64) + np.abs(partials[:partial_count]).astype(np.float64).sum(axis=0)
    assert np.all(np.abs(got_stream.astype(np.float64) - stream.astype(np.float64)) <= step + 4e-7 * operands)
    assert np.mean(got_stream != stream) < 0.01
    stream = got_stream  # what the rest of the launch worked on
    got = {name: outputs[name].numpy(np.float16, (m, width)) for name, width in zip("qkv", n)}
    got_pool = device_pool.numpy(np.uint8, (capacity, stride))

    # the launches it stands for, on the same stream
    separate = {name: b(np.zeros(m * width, dtype=np.float16)) for name, width in zip("qkv", n)}
    rotated = {name: b(np.zeros(m * width, dtype=np.float16)) for name, width in zip("qk", n)}
    separate_pool = b(pool)
    runtime.dispatch("llmopt_rms_w4a16_qkv_linear_f16_g64",
                     [b(stream), b(gain), *device_w[0], *device_w[1], *device_w[2], separate["q"], separate["k"],
                      separate["v"]], u32s(m, k, *n) + struct.pack("<f", epsilon), grid=(256, 1, 1), group=GROUP)
    runtime.dispatch("llmopt_rotary_qk_pack_q8_batched",
                     [separate["q"], separate["k"], b(cos), b(sin), rotated["q"], rotated["k"], separate["v"],
                      b(new_slots), separate_pool],
                     u32s(m, 1, q_heads, k_heads, 64, 32, m) +
                     u32s(m, key_offset, value_offset, k_heads, 64, 64, token_elements, token_elements // 64, stride, m, 0),
                     grid=(256, 1, 1), group=GROUP)
    want = {"q": rotated["q"].numpy(np.float16, (m, n[0])), "k": rotated["k"].numpy(np.float16, (m, n[1])),
            "v": separate["v"].numpy(np.float16, (m, n[2]))}
    for name in "qkv":
        # the same arithmetic but for the order of the float32 sums over K: a last half bit here and there
        assert_close_to_oracle(got[name], want[name].astype(np.float32), f"{name} vs separate launches", rel_l2_tol=3e-4)
    want_pool = separate_pool.numpy(np.uint8, (capacity, stride))
    untouched = np.setdiff1d(np.arange(capacity), new_slots)
    np.testing.assert_array_equal(got_pool[untouched], pool.reshape(capacity, stride)[untouched])
    segment = slice(key_offset, key_offset + 2 * n[1])
    difference = got_pool[new_slots, segment].view(np.int8).astype(np.int32) - \
        want_pool[new_slots, segment].view(np.int8).astype(np.int32)
    assert np.abs(difference).max() <= 1
    # the other layers' bytes of the new tokens' slots stay what they were
    for lo, hi in ((0, key_offset), (key_offset + 2 * n[1], token_elements)):
        np.testing.assert_array_equal(got_pool[new_slots, lo:hi], pool.reshape(capacity, stride)[new_slots, lo:hi])
    scale_lo, scale_hi = token_elements + 2 * (key_offset // 64), token_elements + 2 * ((key_offset + 2 * n[1]) // 64)
    got_scales = got_pool[new_slots, scale_lo:scale_hi].copy().view(np.uint16).astype(np.int32)
    want_scales = want_pool[new_slots, scale_lo:scale_hi].copy().view(np.uint16).astype(np.int32)
    assert np.abs(got_scales - want_scales).max() <= 2
    np.testing.assert_array_equal(got_pool[new_slots, token_elements:scale_lo],
                                  pool.reshape(capacity, stride)[new_slots, token_elements:scale_lo])

    # the oracle on the same stream; the cache bytes are exactly the quantiser's for the K / V this launch stored
    normalised = f16(oracle.rms_norm(stream, gain, epsilon))
    for name, (packed, scale), count in zip("qkv", weights, heads):
        projected = f16(oracle.w4a16_linear(normalised, packed, scale, None)).reshape(m, count, 64)
        if name != "v":
            projected = f16(oracle.rotary_h(projected, cos, sin)).transpose(1, 0, 2)  # back to [m, heads, 64]
        assert_close_to_oracle(got[name], projected.reshape(m, -1).astype(np.float32), f"{name} vs oracle")
    exact_pool = pool.copy()
    for name, offset in (("k", key_offset), ("v", value_offset)):
        source = np.ascontiguousarray(got[name].reshape(m, k_heads, 64).transpose(1, 0, 2))
        oracle.q8_pack(source, new_slots, exact_pool,
                       CacheParams(items=m, segment_offset=offset, heads=k_heads, head_dim=64, group_size=64,
                                   token_elements=token_elements, token_groups=token_elements // 64,
                                   token_stride=stride, source_items=m, source_offset=0))
    np.testing.assert_array_equal(got_pool, exact_pool.reshape(capacity, stride))


@pytest.mark.parametrize("m,n,k", [(1, 1536, 576), (2, 1536, 576), (8, 1536, 576), (33, 1536, 576), (3, 2048, 1024),
                                   (5, 128, 1408), (2, 64, 64), (4, 1024, 704)] + DRAWN_FFN)
@pytest.mark.parametrize("width", [64, 32], ids=["slices_of_64", "slices_of_32"])
def test_fused_ffn_partial_sums_against_separate_launches_and_oracle(runtime, m, n, k, width):
    if n // width > 48:
        pytest.skip("more slices than a reader takes partial sums")
    rng = np.random.default_rng(7 * m + n + k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    gain = rng.uniform(0.5, 1.5, k).astype(np.float16)
    gate, up, down = random_w4(rng, n, k), random_w4(rng, n, k), random_w4(rng, k, n)
    b = runtime.buffer_of_bytes
    device = [b(a) for pair in (gate, up, down) for a in pair]
    slices = n // width
    partials = b(np.full(slices * m * k, np.nan, dtype=np.float32))
    params = u32s(m, n, k) + struct.pack("<f", 1e-5)
    runtime.dispatch("llmopt_rms_w4a16_swiglu_down_partial_f16_g64", [b(x), b(gain), *device, partials],
                     params + u32s(width), grid=(256, 1, 1), group=GROUP)
    got_partials = partials.numpy(np.float32, (slices, m, k))
    assert np.all(np.isfinite(got_partials))
    total = np.zeros((m, k), dtype=np.float32)
    for p in range(slices):
        total = total + got_partials[p]
    got = (total + x.astype(np.float32)).astype(np.float16)  # what the next reader of the stream forms

    product = b(np.zeros(m * n, dtype=np.float16))
    separate = b(np.zeros(m * k, dtype=np.float16))
    runtime.dispatch("llmopt_rms_w4a16_dual_swiglu_f16_g64", [b(x), b(gain), *device[:4], product], params,
                     grid=(256, 1, 1), group=GROUP)
    runtime.dispatch("llmopt_w4a16_down_add_f16_g64" + ("" if m == 1 else "_m4"),
                     [product, *device[4:], b(x), separate], params, grid=(256, 1, 1), group=GROUP)
    assert_close_to_oracle(got, separate.numpy(np.float16, (m, k)).astype(np.float32), "vs separate launches",
                           rel_l2_tol=3e-4)

    normalised = f16(oracle.rms_norm(x, gain, 1e-5))
    want_product = f16(oracle.silu_mul(oracle.w4a16_linear(normalised, *gate, None),
                                       oracle.w4a16_linear(normalised, *up, None)))
    want = oracle.add(oracle.w4a16_linear(want_product, *down, None), x.astype(np.float32))
    assert_close_to_oracle(got, want, "vs oracle")
    # every partial sum is its own slice of the contraction (slices of 32: half a scale group, the group's scale)
    for p in sorted({0, slices // 2, slices - 1}):
        columns = slice(width * p, width * p + width)
        packed = np.ascontiguousarray(down[0][:, width // 2 * p:width // 2 * p + width // 2])
        scale = np.ascontiguousarray(down[1][:, width * p // 64:width * p // 64 + 1])
        if width == 32:  # as a 64-wide group whose other half is zero
            packed = np.concatenate([packed, np.zeros_like(packed)], axis=1)
            padded_product = np.concatenate([want_product[:, columns], np.zeros((m, 32), dtype=np.float16)], axis=1)
            want_partial = oracle.w4a16_linear(padded_product, packed, scale, None)
        else:
            want_partial = oracle.w4a16_linear(want_product[:, columns], packed, scale, None)
        error = np.linalg.norm(got_partials[p] - want_partial) / max(np.linalg.norm(want_partial), 1e-30)
        assert error <= 2e-3, f"partial sum {p}: {error:.3e}"  # the product's half rounding carries over


@pytest.mark.parametrize("m,n,k,pending", [(1, 1536, 576, 9), (2, 1536, 576, 9), (8, 1536, 576, 9), (5, 128, 1024, 32),
                                           (3, 256, 704, 1), (16, 1536, 576, 9), (4, 64, 576, 0)] + DRAWN_SUMMING)
@pytest.mark.parametrize("width", [64, 32], ids=["slices_of_64", "slices_of_32"])
def test_summing_ffn_forms_the_stream_and_leaves_the_partial_sums_of_the_plain_entry(runtime, m, n, k, pending, width):
    if n // width > 48:
        pytest.skip("more slices than a reader takes partial sums")
    rng = np.random.default_rng(11 * m + n + k + pending)
    x, pending_sums, stream = pending_stream(rng, m, k, pending)
    gain = rng.uniform(0.5, 1.5, k).astype(np.float16)
    b = runtime.buffer_of_bytes
    device = [b(a) for pair in (random_w4(rng, n, k), random_w4(rng, n, k), random_w4(rng, k, n)) for a in pair]
    slices = n // width
    params = u32s(m, n, k) + struct.pack("<f", 1e-5)
    stream_out = b(np.full(m * k, np.nan, dtype=np.float16))
    partials = b(np.full(slices * m * k, np.nan, dtype=np.float32))
    runtime.dispatch("llmopt_sum_rms_w4a16_swiglu_down_partial_f16_g64",
                     [b(x), b(pending_sums), stream_out, b(gain), *device, partials], params + u32s(pending, width),
                     grid=(256, 1, 1), group=GROUP)
    got_stream = stream_out.numpy(np.float16, (m, k))
    assert np.all(np.isfinite(got_stream))
    step = np.spacing(np.abs(stream)).astype(np.float64)
    operands = np.abs(x).astype(np.float64) + np.abs(pending_sums[:pending]).astype(np.float64).sum(axis=0)
    assert np.all(np.abs(got_stream.astype(np.float64) - stream.astype(np.float64)) <= step + 4e-7 * operands)
    assert np.mean(got_stream != stream) < 0.01
    # the plain entry on the stream this launch formed: the same kernel from there on, bit for bit
    plain = b(np.full(slices * m * k, np.nan, dtype=np.float32))
    runtime.dispatch("llmopt_rms_w4a16_swiglu_down_partial_f16_g64", [b(got_stream), b(gain), *device, plain],
                     params + u32s(width), grid=(256, 1, 1), group=GROUP)
    np.testing.assert_array_equal(partials.numpy(np.uint32, (slices, m, k)), plain.numpy(np.uint32, (slices, m, k)))


def paged_case(rng, batch, q_heads, kv_heads, lengths):
    """A ragged batch over a pool of one layer's slots: (pool, slots, offsets, stride, token_elements)."""
    token_elements = 2 * kv_heads * 64
    stride = token_elements + 2 * (token_elements // 64)
    total = int(np.sum(lengths))
    capacity = total + 5
    slots = rng.permutation(capacity).astype(np.uint32)[:total]
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    pool = np.zeros((capacity, stride), dtype=np.uint8)
    pool[:, :token_elements] = np.clip(np.rint(rng.standard_normal((capacity, token_elements)) * 38), -127, 127) \
        .astype(np.int8).view(np.uint8)
    pool[:, token_elements:] = rng.uniform(0.02, 0.035, (capacity, token_elements // 64)).astype(np.float16) \
        .view(np.uint8).reshape(capacity, -1)
    return pool, slots, offsets, stride, token_elements


@pytest.mark.parametrize("batch,q_heads,kv_heads,hidden,longest", [(1, 9, 3, 576, 2048), (1, 9, 3, 576, 64), (2, 9, 3, 576, 300),
                                                                   (8, 9, 3, 576, 2048), (5, 8, 2, 1024, 700),
                                                                   (16, 9, 3, 576, 500), (3, 4, 4, 64, 150),
                                                                   (33, 2, 1, 704, 260)] + DRAWN_PROJECTING)
def test_projecting_attention_leaves_each_heads_share_of_the_output_projection(runtime, batch, q_heads, kv_heads, hidden,
                                                                               longest):
    rng = np.random.default_rng(batch * 1000 + hidden + longest)
    lengths = rng.integers(1, longest + 1, size=batch).astype(np.uint32)
    lengths[rng.integers(0, batch)] = longest
    pool, slots, offsets, stride, token_elements = paged_case(rng, batch, q_heads, kv_heads, lengths)
    width = q_heads * 64
    query = rng.standard_normal((batch, width)).astype(np.float16)
    key = rng.standard_normal((batch, kv_heads * 64)).astype(np.float16)
    value = rng.standard_normal((batch, kv_heads * 64)).astype(np.float16)
    projection = random_w4(rng, hidden, width)
    b = runtime.buffer_of_bytes
    shared = [b(query), b(key), b(value), b(pool), b(slots)]
    tail = [b(lengths), b(offsets)]
    device_projection = [b(a) for a in projection]
    params = struct.pack("<12IfIII", batch, q_heads, kv_heads, 0, 64, 0, 0, token_elements, 0, kv_heads * 64, 64, stride,
                         1.0 / math.sqrt(64), 1, 0, 0) + struct.pack("<I", longest)
    rows = b(np.full(batch * width, np.nan, dtype=np.float16))
    runtime.dispatch("llmopt_attention_q8_paged_batched", [*shared, shared[4], rows, *tail], params, grid=(256, 1, 1), group=GROUP)
    attention = rows.numpy(np.float16, (batch, width))
    partials = b(np.full(q_heads * batch * hidden, np.nan, dtype=np.float32))
    runtime.dispatch("llmopt_attention_q8_paged_batched_w4a16_partial_g64",
                     [*shared, shared[4], partials, *tail, *device_projection], params + u32s(hidden), grid=(256, 1, 1), group=GROUP)
    got = partials.numpy(np.float32, (q_heads, batch, hidden))
    assert np.all(np.isfinite(got))
    # every head's 64 columns of the contraction, on the rows the plain entry stores (the same merge, rounded to half)
    for head in range(q_heads):
        packed = np.ascontiguousarray(projection[0][:, 32 * head:32 * head + 32])
        scale = np.ascontiguousarray(projection[1][:, head:head + 1])
        want = oracle.w4a16_linear(attention[:, 64 * head:64 * head + 64], packed, scale, None)
        error = np.linalg.norm(got[head] - want) / max(np.linalg.norm(want), 1e-30)
        # (the two instantiations of the merge may round an element of a row to neighbouring halves: 5e-4 of
        # one element in 64)
        assert error <= 2e-4, f"head {head}: {error:.3e}"
    # and their sum in ascending order against the output-projection launch
    total = np.zeros((batch, hidden), dtype=np.float32)
    for head in range(q_heads):
        total = total + got[head]
    projected = b(np.zeros(batch * hidden, dtype=np.float16))
    runtime.dispatch("llmopt_w4a16_linear_f16_g64" + ("" if batch == 1 else "_m4"), [rows, *device_projection, rows, projected],
                     u32s(batch, hidden, width, 0, hidden), grid=(256, 1, 1), group=GROUP)
    assert_close_to_oracle(total.astype(np.float16), projected.numpy(np.float16, (batch, hidden)).astype(np.float32),
                           "sum of the shares vs the projection launch", rel_l2_tol=3e-4)


def test_fused_entries_reject_what_they_cannot_take(runtime):
    from llmopt_amd.native import LlmoptError
    b = runtime.buffer_of_bytes
    any_buffer = b(np.zeros(4096, dtype=np.uint8))
    with pytest.raises(LlmoptError, match="k <= 1472,"):
        runtime.dispatch("llmopt_rms_w4a16_swiglu_down_partial_f16_g64", [any_buffer] * 9,
                         u32s(1, 64, 4096) + struct.pack("<f", 1e-5) + u32s(64), grid=(256, 1, 1), group=GROUP)
    with pytest.raises(LlmoptError, match="slices of 32 or 64"):
        runtime.dispatch("llmopt_rms_w4a16_swiglu_down_partial_f16_g64", [any_buffer] * 9,
                         u32s(1, 64, 64) + struct.pack("<f", 1e-5) + u32s(48), grid=(256, 1, 1), group=GROUP)
    with pytest.raises(LlmoptError, match="whole heads of 64"):
        runtime.dispatch("llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64", [any_buffer] * 16,
                         u32s(1, 64, 64, 32, 32) + struct.pack("<f", 1e-5) + u32s(0, 0, 64, 128, 132),
                         grid=(256, 1, 1), group=GROUP)
    with pytest.raises(LlmoptError, match="contexts of 64 tokens and more"):
        big = b(np.zeros(1 << 16, dtype=np.uint8))
        runtime.dispatch("llmopt_attention_q8_paged_batched_w4a16_partial_g64", [big] * 11,
                         struct.pack("<12IfIII", 1, 1, 1, 0, 64, 0, 0, 128, 0, 64, 64, 132, 0.125, 1, 0, 0) + u32s(10, 64),
                         grid=(256, 1, 1), group=GROUP)
    with pytest.raises(LlmoptError, match="at most 48 pending"):
        runtime.dispatch("llmopt_sum_rms_w4a16_swiglu_down_partial_f16_g64", [any_buffer] * 11,
                         u32s(1, 64, 64) + struct.pack("<f", 1e-5) + u32s(49, 64), grid=(256, 1, 1), group=GROUP)
    with pytest.raises(LlmoptError, match="two buffers"):
        big = b(np.zeros(1 << 16, dtype=np.uint8))
        runtime.dispatch("llmopt_rms_w4a16_qkv_rotary_pack_q8_f16_g64", [big] * 16,
                         u32s(1, 64, 64, 64, 64) + struct.pack("<f", 1e-5) + u32s(0, 0, 64, 128, 132),
                         grid=(256, 1, 1), group=GROUP)


@pytest.mark.parametrize("batch", [1, 2, 8, 32])
def test_fused_step_leaves_what_the_unfused_step_leaves(runtime, batch):
    """The same step as three or four launches a layer and as six: hidden state and cache within
    the half roundings the two orders of float32 sums allow; three layers, so that the partial sums
    pass from layer to layer twice and the last layer's whole stream feeds the LM head."""
    from llmopt_amd.decode_step import DecodeConfig, DecodeStep, random_weights
    rng = np.random.default_rng(40 + batch)
    config = DecodeConfig(layers=3, vocabulary=1000)
    weights = random_weights(config, rng)
    lengths = [int(v) for v in rng.integers(1, 200, size=batch)]
    lengths[0] = max(lengths[0], 70)  # long enough for the projecting attention
    total = sum(lengths)
    capacity = total + batch
    order = rng.permutation(capacity).astype(np.uint32)
    slots, new_slots = order[:total], order[total:]
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    stride, elements = config.token_stride, config.token_elements
    pool = np.zeros((capacity, stride), dtype=np.uint8)
    pool[:, :elements] = np.clip(np.rint(rng.standard_normal((capacity, elements)) * 38), -127, 127) \
        .astype(np.int8).view(np.uint8)
    pool[:, elements:] = rng.uniform(0.02, 0.035, (capacity, elements // 64)).astype(np.float16) \
        .view(np.uint8).reshape(capacity, -1)
    tokens = rng.integers(0, config.vocabulary, batch)
    results = {}
    # six launches a layer, four, and three (the last layer of a fused step: five)
    launches = {"unfused": 2 + 6 * config.layers, "fused_qkv": 2 + 5 * config.layers, "fused": 2 + 4 * config.layers + 1,
                "projecting": 2 + 3 * (config.layers - 1) + 5}
    for mode in launches:
        device_pool = runtime.buffer_of_bytes(pool)
        step = DecodeStep(runtime, config, weights, batch, device_pool, runtime.buffer_of_bytes(slots), offsets,
                          lengths, new_slots, lengths, fused=mode in ("fused", "projecting"), projecting=mode == "projecting",
                          fused_qkv=mode == "fused_qkv")
        assert step.fused == (mode in ("fused", "projecting")) and step.projecting == (mode == "projecting")
        assert len(step.dispatches) == launches[mode]
        got_tokens = step.run(tokens)
        results[mode] = (got_tokens, step.work["x"][0].numpy(np.float16, (batch, config.hidden)),
                         device_pool.numpy(np.uint8, (capacity, stride)))
    for mode in ("fused_qkv", "fused", "projecting"):
        assert_close_to_oracle(results[mode][1], results["unfused"][1].astype(np.float32), f"{mode} vs unfused hidden state",
                               rel_l2_tol=2e-3)
        difference = results[mode][2][:, :elements].view(np.int8).astype(np.int32) - \
            results["unfused"][2][:, :elements].view(np.int8).astype(np.int32)
        assert np.abs(difference).max() <= 1
    hidden, logits, _ = decode_chain(config, weights, pool.reshape(-1), slots, offsets, lengths, new_slots, lengths, tokens)
    # three layers of chained kernels that each store half: 2e-3 a layer in relative L2, as the two-layer
    # chains are held to 4e-3, and the largest single difference at 1e-2 x RMS a layer
    want = hidden.astype(np.float64)
    rms_hidden = float(np.sqrt(np.mean(want ** 2)))
    for mode in launches:
        difference = results[mode][1].astype(np.float64) - want
        assert np.linalg.norm(difference) <= 6e-3 * np.linalg.norm(want), mode
        assert np.abs(difference).max() <= 3e-2 * rms_hidden, mode
    rms = float(np.sqrt(np.mean(logits.astype(np.float64) ** 2)))
    for mode in launches:
        for b in range(batch):
            assert float(logits[b, results[mode][0][b]]) >= float(logits[b].max()) - 2e-2 * rms, mode
