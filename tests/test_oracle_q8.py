"""Pins the CPU oracle's Q8 cache and attention functions (restating
lib/metal_cache_source.ml:46-81,184-211,382-401,493-583 and lib/cpu.ml:606-717)
against the reference's golden vectors, closed forms and brute force."""
import math

import numpy as np
import pytest

import oracle
from oracle import CacheParams, PagedParams


def _f16(bits):
    return np.array(bits, dtype=np.uint16).view(np.float16)


def _layout(kv_heads, head_dim, layers=1):
    """Kv_cache.Layout arithmetic (lib/kv_cache.ml:16-21,126-166)."""
    segment = kv_heads * head_dim
    token_elements = 2 * segment * layers
    token_stride = token_elements + 2 * (token_elements // 64)
    return token_elements, token_stride


def test_layout_matches_reference_gemma_numbers(golden):
    case = golden["kv_layout_gemma"]
    elements = case["token_elements"]
    assert elements + 2 * (elements // 64) == case["bytes_per_token"]


def _pack_params(items, segment_offset, heads, head_dim, token_elements, token_stride,
                 source_items=None, source_offset=0):
    return CacheParams(items=items, segment_offset=segment_offset, heads=heads,
                       head_dim=head_dim, group_size=64, token_elements=token_elements,
                       token_groups=token_elements // 64, token_stride=token_stride,
                       source_items=source_items or items, source_offset=source_offset)


def test_reference_round_trip_vector(golden):
    cycle = golden["q8_round_trip"]["value_bits_cycle"]
    token_elements, stride = _layout(1, 64)
    items = 3
    source = _f16([cycle[i % 4] for i in range(items * 64)]).reshape(1, items, 64)
    slots = np.array([2, 0, 3], dtype=np.uint32)
    pool = np.zeros(4 * stride, dtype=np.uint8)
    for offset in (0, 64):
        params = _pack_params(items, offset, 1, 64, token_elements, stride)
        oracle.q8_pack(source, slots, pool, params)
        back = oracle.q8_unpack(pool, slots, params)
        np.testing.assert_array_equal(back.view(np.uint16), source.view(np.uint16))
    # stored bytes are exactly +-127 / +-1 and every scale is 1.0
    token = pool[2 * stride:3 * stride]
    assert token[:4].view(np.int8).tolist() == [127, -127, 1, -1]
    assert token[token_elements:].view(np.uint16).tolist() == [0x3c00, 0x3c00]


def test_pack_closed_forms():
    token_elements, stride = _layout(2, 64)
    pool = np.full(stride, 0xAA, dtype=np.uint8)
    source = np.zeros((2, 1, 64), dtype=np.float16)
    # head 0: all zero -> scale 1.0, bytes 0.
    # head 1: maximum 2.0 -> scale half(2/127); ties: x/scale = k + 0.5 rounds to even.
    source[1, 0, 0] = 2.0
    source[1, 0, 1] = -2.0
    source[1, 0, 2] = 1.0
    params = _pack_params(1, 0, 2, 64, token_elements, stride)
    oracle.q8_pack(source, np.zeros(1, dtype=np.uint32), pool, params)
    scale_bits = pool[token_elements:token_elements + 4].view(np.uint16)
    assert scale_bits[0] == 0x3c00
    expected_scale = np.float16(np.float32(2.0) / np.float32(127.0))
    assert scale_bits[1] == expected_scale.view(np.uint16)
    q = pool[64:128].view(np.int8)
    s = np.float32(expected_scale)
    assert q[0] == min(127, int(np.rint(np.float32(2.0) / s)))
    assert q[1] == -q[0]
    assert q[2] == int(np.rint(np.float32(1.0) / s))
    assert np.all(pool[:64] == 0) and np.all(q[3:] == 0)
    # bytes outside the written segment (V half of the token, V scales) are untouched
    assert np.all(pool[128:token_elements] == 0xAA)
    assert np.all(pool[token_elements + 4:] == 0xAA)


def test_pack_round_half_even_and_clamp():
    token_elements, stride = _layout(1, 64)
    pool = np.zeros(stride, dtype=np.uint8)
    source = np.zeros((1, 1, 64), dtype=np.float16)
    source[0, 0, 0] = 127.0    # scale = 1.0 exactly
    source[0, 0, 1] = 0.5      # tie -> 0
    source[0, 0, 2] = 1.5      # tie -> 2
    source[0, 0, 3] = 2.5      # tie -> 2
    source[0, 0, 4] = -0.5     # tie -> -0
    source[0, 0, 5] = -3.5     # tie -> -4
    source[0, 0, 6] = 126.5    # tie -> 126
    oracle.q8_pack(source, np.zeros(1, dtype=np.uint32), pool,
                   _pack_params(1, 0, 1, 64, token_elements, stride))
    assert pool[:7].view(np.int8).tolist() == [127, 0, 2, 2, 0, -4, 126]
    assert pool[token_elements:token_elements + 2].view(np.uint16)[0] == 0x3c00


def test_pack_matches_vectorised_numpy_and_error_bound():
    rng = np.random.default_rng(3)
    heads, dim, items = 4, 128, 6
    token_elements, stride = _layout(heads, dim)
    source = rng.standard_normal((heads, 9, dim)).astype(np.float16)
    slots = rng.permutation(16)[:items].astype(np.uint32)
    pool = np.zeros(16 * stride, dtype=np.uint8)
    params = _pack_params(items, heads * dim, heads, dim, token_elements, stride,
                          source_items=9, source_offset=2)
    oracle.q8_pack(source, slots, pool, params)
    chosen = source[:, 2:2 + items, :].astype(np.float32).reshape(heads, items, dim // 64, 64)
    maximum = np.abs(chosen).max(axis=-1)
    scale = (maximum / np.float32(127.0)).astype(np.float16)
    q = np.clip(np.rint(chosen / scale.astype(np.float32)[..., None]), -127, 127).astype(np.int8)
    for item in range(items):
        base = int(slots[item]) * stride
        got_q = pool[base + heads * dim: base + 2 * heads * dim].view(np.int8)
        np.testing.assert_array_equal(got_q.reshape(heads, dim // 64, 64), q[:, item])
        got_scale = pool[base + token_elements: base + stride].view(np.uint16)
        first = (heads * dim) // 64
        np.testing.assert_array_equal(got_scale[first:first + heads * dim // 64],
                                      scale[:, item].reshape(-1).view(np.uint16))
    back = oracle.q8_unpack(pool, slots, params).astype(np.float32)
    error = np.abs(back - source[:, 2:2 + items, :].astype(np.float32))
    bound = np.repeat(scale.astype(np.float32), 64, axis=-1).reshape(heads, items, dim)
    assert np.all(error <= 0.5 * bound * 1.01 + 1e-3 * np.abs(back))


def _paged_setup(golden_case, query_heads):
    pool = np.zeros(132, dtype=np.uint8)
    pool[64:128] = 2
    pool[128:132] = np.array([0x3c00, 0x3c00], dtype=np.uint16).view(np.uint8)
    params = PagedParams(batches=1, query_heads=query_heads, kv_heads=1, past_length=1,
                         head_dim=64, mask_batches=1, mask_heads=1, token_elements=128,
                         key_offset=0, value_offset=64, group_size=64, token_stride=132,
                         scale=1.0, query_length=1, mask_dtype=1, window=0)
    query = np.zeros((1, query_heads, 1, 64), dtype=np.float16)
    current_key = np.zeros((1, 1, 1, 64), dtype=np.float16)
    current_value = _f16([golden_case["current_value_bits"]] * 64).reshape(1, 1, 1, 64)
    mask = np.array([1, 1], dtype=np.uint8)
    return query, current_key, current_value, pool, np.zeros(1, dtype=np.uint32), mask, params


@pytest.mark.parametrize("name,heads", [("paged_attention_h64", 1), ("paged_attention_gqa3", 3)])
def test_paged_attention_reference_vectors(golden, name, heads):
    base = golden["paged_attention_h64"]
    args = _paged_setup(base, heads)
    out = oracle.paged_attention_q8(*args)
    bits = out.astype(np.float16).view(np.uint16).reshape(-1)
    assert bits.size == 64 * heads
    assert np.all(bits == golden[name]["expected_output_bits"])


def test_dense_attention_reference_vector(golden):
    case = golden["dense_attention_2x2"]
    q = _f16(case["query_bits"]).reshape(1, 1, 2, 2)
    k = _f16(case["key_bits"]).reshape(1, 1, 2, 2)
    v = _f16(case["value_bits"]).reshape(1, 1, 2, 2)
    mask = np.array(case["mask_bool"], dtype=np.float32).reshape(1, 1, 2, 2)
    out = oracle.attention(q, k, v, mask, scale=1.0)
    assert out.astype(np.float16).view(np.uint16).reshape(-1).tolist() == case["expected_output_bits"]


def test_dense_attention_brute_force_and_invariants():
    rng = np.random.default_rng(8)
    b, h, ql, kl, d = 2, 3, 2, 7, 8
    q = rng.standard_normal((b, h, ql, d)).astype(np.float32)
    k = rng.standard_normal((b, h, kl, d)).astype(np.float32)
    v = rng.standard_normal((b, h, kl, d)).astype(np.float32)
    mask = (rng.random((b, 1, ql, kl)) > 0.3).astype(np.float32)
    mask[0, 0, 0, :] = 0  # a fully masked row -> zeros
    scale = 0.37
    out = oracle.attention(q, k, v, mask, scale)
    for bi in range(b):
        for hi in range(h):
            for qi in range(ql):
                keys = [j for j in range(kl) if mask[bi, 0, qi, j] != 0]
                if not keys:
                    assert np.all(out[bi, hi, qi] == 0)
                    continue
                s = [scale * math.fsum(float(q[bi, hi, qi, t]) * float(k[bi, hi, j, t])
                                       for t in range(d)) for j in keys]
                top = max(s)
                w = [math.exp(x - top) for x in s]
                z = math.fsum(w)
                for t in range(d):
                    expected = math.fsum(wi / z * float(v[bi, hi, j, t]) for wi, j in zip(w, keys))
                    assert abs(out[bi, hi, qi, t] - expected) <= 1e-6 * max(1.0, abs(expected))
    # causal flag: key_position <= query_position
    ones = np.ones((1, 1, ql, kl), dtype=np.float32)
    causal = oracle.attention(q, k, v, ones, scale, causal=True)
    np.testing.assert_allclose(causal[:, :, 0], v[:, :, 0], rtol=1e-6)
    # shift invariance of softmax: adding a constant vector c to all keys with q.c fixed
    # -> all-equal scores give the mean of V
    zero_q = np.zeros_like(q)
    mean_out = oracle.attention(zero_q, k, v, ones, scale)
    np.testing.assert_allclose(mean_out[:, :, 0], v.mean(axis=2), rtol=1e-6, atol=1e-7)


def _build_pool(rng, batches, kv_heads, dim, lengths, layers=1, layer=0, capacity_extra=3):
    token_elements, stride = _layout(kv_heads, dim, layers)
    total = int(sum(lengths))
    capacity = total + capacity_extra
    pool = np.zeros(capacity * stride, dtype=np.uint8)
    order = rng.permutation(capacity)[:total].astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    key_offset = layer * 2 * kv_heads * dim
    value_offset = key_offset + kv_heads * dim
    keys, values = [], []
    for bi, length in enumerate(lengths):
        kf = rng.standard_normal((kv_heads, length, dim)).astype(np.float16)
        vf = rng.standard_normal((kv_heads, length, dim)).astype(np.float16)
        seq_slots = order[offsets[bi]:offsets[bi] + length]
        oracle.q8_pack(kf, seq_slots, pool, _pack_params(length, key_offset, kv_heads, dim,
                                                         token_elements, stride))
        oracle.q8_pack(vf, seq_slots, pool, _pack_params(length, value_offset, kv_heads, dim,
                                                         token_elements, stride))
        keys.append(kf)
        values.append(vf)
    return pool, order, offsets, (token_elements, stride, key_offset, value_offset)


def test_paged_equals_dequant_then_dense_attention():
    """The paged oracle must equal: Q8 unpack (fp32 value, not rounded to f16) ->
    GQA expansion -> append the current token -> Cpu.attention."""
    rng = np.random.default_rng(21)
    b, h, kvh, dim = 2, 4, 2, 64
    lengths = [5, 9]
    pool, slots, offsets, (te, stride, ko, vo) = _build_pool(rng, b, kvh, dim, lengths, layers=2,
                                                              layer=1)
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=0, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride, scale=scale,
                         query_length=1, mask_dtype=0, window=0)
    out = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params,
                                    past_lengths=np.array(lengths), slot_offsets=offsets)
    for bi in range(b):
        length = lengths[bi]
        seq_slots = slots[offsets[bi]:offsets[bi] + length]
        dk = np.empty((kvh, length, dim), dtype=np.float32)
        dv = np.empty((kvh, length, dim), dtype=np.float32)
        for t, slot in enumerate(seq_slots):
            token = pool[int(slot) * stride:(int(slot) + 1) * stride]
            scales = token[te:].view(np.float16).astype(np.float32)
            ints = token[:te].view(np.int8).astype(np.float32)
            for head in range(kvh):
                for g in range(dim // 64):
                    sk = scales[ko // 64 + head * (dim // 64) + g]
                    sv = scales[vo // 64 + head * (dim // 64) + g]
                    dk[head, t, g * 64:(g + 1) * 64] = ints[ko + head * dim + g * 64: ko + head * dim + (g + 1) * 64] * sk
                    dv[head, t, g * 64:(g + 1) * 64] = ints[vo + head * dim + g * 64: vo + head * dim + (g + 1) * 64] * sv
        full_k = np.concatenate([dk, ck[bi].astype(np.float32)], axis=1)
        full_v = np.concatenate([dv, cv[bi].astype(np.float32)], axis=1)
        full_k = np.repeat(full_k, h // kvh, axis=0)[None]
        full_v = np.repeat(full_v, h // kvh, axis=0)[None]
        mask = np.ones((1, 1, 1, length + 1), dtype=np.float32)
        dense = oracle.attention(query[bi:bi + 1], full_k, full_v, mask, np.float32(scale))
        # paged output is token-major [b,q,h,D]
        np.testing.assert_allclose(out[bi, 0], dense[0, :, 0], rtol=1e-6, atol=1e-7)


def test_paged_shared_slots_window_and_mask():
    rng = np.random.default_rng(4)
    h, kvh, dim, past = 2, 1, 64, 6
    pool, slots, _, (te, stride, ko, vo) = _build_pool(rng, 1, kvh, dim, [past])
    query = rng.standard_normal((2, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((2, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((2, kvh, 1, dim)).astype(np.float16)

    def run(**kw):
        fields = dict(batches=2, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                      mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                      value_offset=vo, group_size=64, token_stride=stride, scale=0.125,
                      query_length=1, mask_dtype=0, window=0)
        mask = kw.pop("mask", None)
        fields.update(kw)
        return oracle.paged_attention_q8(query, ck, cv, pool, slots, mask, PagedParams(**fields))

    full = run()
    # window 1 -> only the current token -> output = current value
    only_current = run(window=1)
    for bi in range(2):
        for head in range(h):
            np.testing.assert_allclose(only_current[bi, 0, head], cv[bi, 0, 0].astype(np.float32),
                                       rtol=1e-6)
    # a bool mask that hides every past token gives the same
    mask = np.zeros((1, 1, 1, past + 1), dtype=np.uint8)
    mask[..., past] = 1
    np.testing.assert_array_equal(run(mask=mask, mask_batches=1, mask_heads=1, mask_dtype=1),
                                  only_current)
    # f16 additive mask: >= 0 allowed, -inf hidden
    additive = np.full((1, 1, 1, past + 1), -np.inf, dtype=np.float16)
    additive[..., past] = 0
    np.testing.assert_array_equal(run(mask=additive, mask_batches=1, mask_heads=1, mask_dtype=2),
                                  only_current)
    # all-ones mask = no mask; fully hidden -> zeros
    ones = np.ones((1, 1, 1, past + 1), dtype=np.uint8)
    np.testing.assert_array_equal(run(mask=ones, mask_batches=1, mask_heads=1, mask_dtype=1), full)
    assert np.all(run(mask=np.zeros_like(ones), mask_batches=1, mask_heads=1, mask_dtype=1) == 0)
    # window >= key_length changes nothing
    np.testing.assert_array_equal(run(window=past + 1), full)
    # both batches share the slot table in the reference operator
    assert not np.array_equal(full[0], full[1])


def test_rms_norm_reference_vector_and_rotary_and_argmax(golden):
    x = np.array([[1, 0, 0, 0], [0, 1, 0, 0]], dtype=np.float32)
    out = oracle.rms_norm(x, np.ones(4, dtype=np.float16), 0.0)
    assert out.astype(np.float16).view(np.uint16).reshape(-1).tolist() == \
        golden["rms_norm"]["expected_output_bits"]
    rng = np.random.default_rng(1)
    tokens, heads, d = 3, 2, 8
    v = rng.standard_normal((tokens, heads, d)).astype(np.float32)
    angle = rng.standard_normal((tokens, d // 2))
    cos = np.concatenate([np.cos(angle), np.cos(angle)], axis=1)
    sin = np.concatenate([np.sin(angle), np.sin(angle)], axis=1)
    rotated = oracle.rotary_h(v, cos, sin)
    # rotation preserves the norm of every (c, c+h) pair and is the complex product
    z_in = v[..., :d // 2] + 1j * v[..., d // 2:]
    z_out = rotated[..., :d // 2] + 1j * rotated[..., d // 2:]
    expected = z_in * np.exp(1j * angle)[:, None, :]
    np.testing.assert_allclose(z_out, np.transpose(expected, (1, 0, 2)), rtol=1e-5, atol=1e-6)
    assert oracle.argmax(np.array([1.0, 5.0, 5.0, 2.0])) == 1
    assert oracle.argmax(np.array([-1.0])) == 0
