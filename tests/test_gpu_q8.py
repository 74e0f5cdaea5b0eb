"""GPU parity of the Q8 KV cache kernels and paged decode attention against the CPU oracle."""
import math
import struct

import numpy as np
import pytest

import oracle
from oracle import CacheParams, PagedParams
from tests.gpu_util import assert_close_to_oracle, u32s

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def layout(kv_heads, head_dim, layers=1):
    token_elements = 2 * kv_heads * head_dim * layers
    return token_elements, token_elements + 2 * (token_elements // 64)


def cache_params_bytes(items, segment_offset, heads, head_dim, token_elements, stride,
                       source_items, source_offset):
    return u32s(items, segment_offset, heads, head_dim, 64, token_elements, token_elements // 64,
                stride, source_items, source_offset)


def oracle_cache_params(items, segment_offset, heads, head_dim, token_elements, stride,
                        source_items, source_offset):
    return CacheParams(items=items, segment_offset=segment_offset, heads=heads, head_dim=head_dim,
                       group_size=64, token_elements=token_elements,
                       token_groups=token_elements // 64, token_stride=stride,
                       source_items=source_items, source_offset=source_offset)


@pytest.mark.parametrize("name", ["llmopt_cache_pack_attention_q8", "llmopt_cache_pack_attention_q8_simd"])
def test_pack_is_bit_exact(runtime, name):
    rng = np.random.default_rng(3)
    heads, dim, items, source_items, source_offset = 3, 128, 37, 50, 5
    token_elements, stride = layout(heads, dim, layers=2)
    capacity = 64
    source = rng.standard_normal((heads, source_items, dim)).astype(np.float16)
    source[0, source_offset + 1, :64] = 0           # an all-zero group -> scale 1.0
    source[1, source_offset + 2, 64:] = 60000.0     # large magnitudes
    source[2, source_offset + 3, :64] = 6e-8        # tiny (subnormal f16) magnitudes
    slots = rng.permutation(capacity)[:items].astype(np.uint32)
    segment = 2 * heads * dim + heads * dim  # layer 1, V segment
    host_pool = rng.integers(0, 256, size=capacity * stride, dtype=np.uint8)
    expected = host_pool.copy()
    oracle.q8_pack(source, slots, expected,
                   oracle_cache_params(items, segment, heads, dim, token_elements, stride,
                                       source_items, source_offset))
    pool = runtime.buffer_of_bytes(host_pool)
    runtime.dispatch(name, [runtime.buffer_of_bytes(source), runtime.buffer_of_bytes(slots), pool],
                     cache_params_bytes(items, segment, heads, dim, token_elements, stride,
                                        source_items, source_offset),
                     grid=(items * heads * dim // 64 * 32, 1, 1), group=(256, 1, 1))
    got = pool.numpy(np.uint8)
    finite_scale = np.float32(6e-8) / np.float32(127.0)
    assert np.float16(finite_scale) == 0  # documents why the tiny group is excluded below
    # the tiny group divides by a zero scale (x/0): undefined in the reference too; skip its bytes
    tiny_slot = int(slots[3]) * stride
    lo, hi = tiny_slot + segment + 2 * dim, tiny_slot + segment + 2 * dim + 64
    mask = np.ones_like(got, dtype=bool)
    mask[lo:hi] = False
    np.testing.assert_array_equal(got[mask], expected[mask])


@pytest.mark.parametrize("name", ["llmopt_cache_pack_attention_q8", "llmopt_cache_pack_attention_q8_simd"])
def test_pack_rounds_ties_to_even(runtime, name):
    """Every quotient x / scale lands exactly halfway between two integers: a group's largest
    magnitude is 127 * 2^e (scale 2^e exactly) and the others are (n + 0.5) * 2^e, all exact in
    fp16.  rint rounds them to the even neighbour, both signs (lib/metal_cache_source.ml:67-75)."""
    rng = np.random.default_rng(17)
    heads, dim, items = 2, 128, 24
    token_elements, stride = layout(heads, dim)
    source = np.empty((heads, items, dim), dtype=np.float16)
    for head in range(heads):
        for item in range(items):
            for group in range(dim // 64):
                step = np.float32(2.0) ** int(rng.integers(-6, 3))
                n = rng.integers(0, 127, size=64).astype(np.float32)
                sign = rng.choice([-1.0, 1.0], size=64).astype(np.float32)
                values = sign * (n + np.float32(0.5)) * step
                values[int(rng.integers(0, 64))] = np.float32(127.0) * step * rng.choice([-1.0, 1.0])
                source[head, item, group * 64:(group + 1) * 64] = values.astype(np.float16)
    assert np.array_equal(source.astype(np.float32).astype(np.float16), source)
    slots = rng.permutation(items + 3)[:items].astype(np.uint32)
    expected = np.zeros((items + 3) * stride, dtype=np.uint8)
    oracle.q8_pack(source, slots, expected, oracle_cache_params(items, 0, heads, dim, token_elements, stride, items, 0))
    quantised = expected.reshape(items + 3, stride)[slots][:, :heads * dim].view(np.int8)
    assert np.all((quantised % 2 == 0) | (np.abs(quantised) == 127))  # every tie went to the even neighbour
    pool = runtime.create_buffer((items + 3) * stride)
    runtime.dispatch(name, [runtime.buffer_of_bytes(source), runtime.buffer_of_bytes(slots), pool],
                     cache_params_bytes(items, 0, heads, dim, token_elements, stride, items, 0),
                     grid=(items * heads * dim // 64 * 32, 1, 1), group=(256, 1, 1))
    np.testing.assert_array_equal(pool.numpy(np.uint8), expected)


def test_pair_pack_and_unpack_round_trip(runtime, golden):
    cycle = golden["q8_round_trip"]["value_bits_cycle"]
    heads, dim, items = 2, 64, 5
    token_elements, stride = layout(heads, dim)
    values = np.array([cycle[i % 4] for i in range(heads * items * dim)], dtype=np.uint16)
    key = values.view(np.float16).reshape(heads, items, dim)
    value = (-key.astype(np.float32)).astype(np.float16)
    slots = np.array([4, 0, 2, 6, 1], dtype=np.uint32)
    pool = runtime.create_buffer(8 * stride)
    key_offset, value_offset = 0, heads * dim
    runtime.dispatch("llmopt_cache_pack_attention_q8_pair_simd",
                     [runtime.buffer_of_bytes(key), runtime.buffer_of_bytes(value),
                      runtime.buffer_of_bytes(slots), pool],
                     u32s(items, key_offset, value_offset, heads, dim, 64, token_elements,
                          token_elements // 64, stride, items, 0),
                     grid=(items * heads * 32, 1, 1), group=(256, 1, 1))
    expected = np.zeros(8 * stride, dtype=np.uint8)
    for src, offset in ((key, key_offset), (value, value_offset)):
        oracle.q8_pack(src, slots, expected,
                       oracle_cache_params(items, offset, heads, dim, token_elements, stride, items, 0))
    np.testing.assert_array_equal(pool.numpy(np.uint8), expected)
    for name in ("llmopt_cache_unpack_attention_q8", "llmopt_cache_unpack_attention_q8_vec4"):
        for src, offset in ((key, key_offset), (value, value_offset)):
            destination = runtime.create_buffer(heads * items * dim * 2)
            runtime.dispatch(name, [pool, runtime.buffer_of_bytes(slots), destination],
                             cache_params_bytes(items, offset, heads, dim, token_elements, stride, items, 0),
                             grid=(items * heads * dim, 1, 1), group=(256, 1, 1))
            np.testing.assert_array_equal(destination.numpy(np.uint16), src.view(np.uint16).reshape(-1))


def test_unpack_matches_oracle_on_random_pool(runtime):
    rng = np.random.default_rng(12)
    heads, dim, items = 4, 128, 9
    token_elements, stride = layout(heads, dim)
    source = (rng.standard_normal((heads, items, dim)) * 3).astype(np.float16)
    slots = rng.permutation(16)[:items].astype(np.uint32)
    host_pool = np.zeros(16 * stride, dtype=np.uint8)
    params = oracle_cache_params(items, heads * dim, heads, dim, token_elements, stride, items, 0)
    oracle.q8_pack(source, slots, host_pool, params)
    destination = runtime.create_buffer(heads * items * dim * 2)
    runtime.dispatch("llmopt_cache_unpack_attention_q8_vec4",
                     [runtime.buffer_of_bytes(host_pool), runtime.buffer_of_bytes(slots), destination],
                     cache_params_bytes(items, heads * dim, heads, dim, token_elements, stride, items, 0))
    np.testing.assert_array_equal(destination.numpy(np.uint16),
                                  oracle.q8_unpack(host_pool, slots, params).view(np.uint16).reshape(-1))


def paged_params_bytes(p: PagedParams, max_past=None):
    raw = struct.pack("<12IfIII", p.batches, p.query_heads, p.kv_heads, p.past_length, p.head_dim,
                      p.mask_batches, p.mask_heads, p.token_elements, p.key_offset, p.value_offset,
                      p.group_size, p.token_stride, p.scale, p.query_length, p.mask_dtype, p.window)
    assert len(raw) == 64
    if max_past is not None:
        raw += struct.pack("<I", max_past)
    return raw


def build_pool(rng, kv_heads, dim, lengths, layers=1, layer=0, extra=5):
    token_elements, stride = layout(kv_heads, dim, layers)
    total = int(sum(lengths))
    capacity = total + extra
    pool = np.zeros(capacity * stride, dtype=np.uint8)
    order = rng.permutation(capacity)[:total].astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    key_offset = layer * 2 * kv_heads * dim
    value_offset = key_offset + kv_heads * dim
    for index, length in enumerate(lengths):
        seq_slots = order[offsets[index]:offsets[index] + length]
        for offset in (key_offset, value_offset):
            src = rng.standard_normal((kv_heads, length, dim)).astype(np.float16)
            oracle.q8_pack(src, seq_slots, pool,
                           oracle_cache_params(length, offset, kv_heads, dim, token_elements, stride,
                                               length, 0))
    return pool, order, offsets, token_elements, stride, key_offset, value_offset


def run_paged(runtime, name, query, ck, cv, pool, slots, mask, params, lengths=None, offsets=None):
    b, h, q_len, dim = query.shape
    out = runtime.buffer_of_bytes(np.full((b, q_len, h, dim), np.nan, dtype=np.float16))
    b_slots = runtime.buffer_of_bytes(slots if slots.size else np.zeros(1, dtype=np.uint32))
    b_mask = runtime.buffer_of_bytes(mask) if mask is not None else b_slots
    buffers = [runtime.buffer_of_bytes(query), runtime.buffer_of_bytes(ck), runtime.buffer_of_bytes(cv),
               runtime.buffer_of_bytes(pool), b_slots, b_mask, out]
    raw = paged_params_bytes(params)
    if lengths is not None:
        buffers += [runtime.buffer_of_bytes(np.asarray(lengths, dtype=np.uint32)),
                    runtime.buffer_of_bytes(np.asarray(offsets, dtype=np.uint32))]
        raw = paged_params_bytes(params, int(max(lengths)))
    rows = b * h * q_len
    runtime.dispatch(name, buffers, raw, grid=(((rows + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    return out.numpy(np.float16, (b, q_len, h, dim))


@pytest.mark.parametrize("name,heads", [("llmopt_attention_q8_paged_simd_h64", 1),
                                        ("llmopt_attention_q8_paged_simd_h64_gqa3", 3)])
def test_reference_paged_vectors(runtime, golden, name, heads):
    pool = np.zeros(132, dtype=np.uint8)
    pool[64:128] = 2
    pool[128:132] = np.array([0x3c00, 0x3c00], dtype=np.uint16).view(np.uint8)
    params = PagedParams(batches=1, query_heads=heads, kv_heads=1, past_length=1, head_dim=64,
                         mask_batches=1, mask_heads=1, token_elements=128, key_offset=0,
                         value_offset=64, group_size=64, token_stride=132, scale=1.0,
                         query_length=1, mask_dtype=1, window=0)
    query = np.zeros((1, heads, 1, 64), dtype=np.float16)
    ck = np.zeros((1, 1, 1, 64), dtype=np.float16)
    cv = np.full((1, 1, 1, 64), 4.0, dtype=np.float16)
    out = run_paged(runtime, name, query, ck, cv, pool, np.zeros(1, dtype=np.uint32),
                    np.array([1, 1], dtype=np.uint8), params)
    assert np.all(out.view(np.uint16) == golden["paged_attention_h64"]["expected_output_bits"])


SPLIT_CASES = [
    # (batches, query_heads, kv_heads, head_dim, past_length)
    (1, 4, 1, 128, 64), (2, 32, 8, 128, 300), (1, 9, 3, 64, 513), (1, 8, 8, 64, 1000),
    (2, 16, 1, 128, 257), (1, 4, 2, 128, 2048),
]


@pytest.mark.parametrize("b,h,kvh,dim,past", SPLIT_CASES)
def test_decode_attention_shared_slots(runtime, b, h, kvh, dim, past):
    rng = np.random.default_rng(b * 1000 + h * 10 + past)
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [past], layers=2, layer=1)
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=1, mask_dtype=0, window=0)
    name = "llmopt_attention_q8_paged_simd_generic" if dim == 128 else "llmopt_attention_q8_paged_simd_h64"
    out = run_paged(runtime, name, query, ck, cv, pool, slots, None, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params)
    assert_close_to_oracle(out, expected, f"paged b{b} h{h}/{kvh} d{dim} past{past}")


@pytest.mark.parametrize("kvh,dim,layers,layer", [(3, 64, 3, 1), (1, 128, 3, 2), (3, 64, 30, 17)])
def test_decode_attention_slots_not_16_byte_aligned(runtime, kvh, dim, layers, layer):
    """Token strides that are not a multiple of 16 (e.g. 11880 bytes for 30 layers of 3 x 64)."""
    rng = np.random.default_rng(layers * 100 + dim)
    past, group = 700, 3
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [past], layers=layers, layer=layer)
    assert stride % 16 != 0
    h = kvh * group
    query = rng.standard_normal((2, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((2, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((2, kvh, 1, dim)).astype(np.float16)
    params = PagedParams(batches=2, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=1, mask_dtype=0, window=0)
    name = "llmopt_attention_q8_paged_simd_generic" if dim == 128 else "llmopt_attention_q8_paged_simd_h64_gqa3"
    out = run_paged(runtime, name, query, ck, cv, pool, slots, None, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params)
    assert_close_to_oracle(out, expected, f"unaligned stride {stride}")


def test_decode_attention_per_sequence_lengths(runtime):
    """The batched extension: ragged contexts, one slot table per sequence."""
    rng = np.random.default_rng(99)
    b, h, kvh, dim = 5, 32, 8, 128
    lengths = [64, 700, 257, 1, 1500]
    pool, slots, offsets, te, stride, ko, vo = build_pool(rng, kvh, dim, lengths)
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=0, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=1, mask_dtype=0, window=0)
    out = run_paged(runtime, "llmopt_attention_q8_paged_batched", query, ck, cv, pool, slots, None,
                    params, lengths=lengths, offsets=offsets)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params,
                                         past_lengths=np.array(lengths), slot_offsets=offsets)
    assert_close_to_oracle(out, expected, "batched ragged")
    # single-key sanity: sequence 3 has one past token + the current one
    assert np.all(np.isfinite(out[3]))


@pytest.mark.parametrize("b,kvh,group,dim,seed", [(70, 2, 2, 64, 5), (130, 1, 4, 128, 6), (3, 8, 4, 128, 7),
                                                   (5, 4, 4, 256, 8), (70, 1, 2, 256, 9), (2, 6, 1, 256, 10)])
def test_decode_attention_balanced_split_over_many_sequences(runtime, b, kvh, group, dim, seed):
    """Ragged batches, also wider than the 64 sequences one planning pass of a wave covers: every
    sequence gets its own chunk size from the device-side lengths; empty, one-token and
    tile-boundary contexts among them, and one long context that takes most of the chunk slots."""
    rng = np.random.default_rng(seed)
    lengths = [int(v) for v in rng.integers(64, 400, size=b)]
    for index, value in zip(range(0, b, max(1, b // 9)), [0, 1, 15, 16, 17, 63, 65, 127, 129]):
        lengths[index] = value
    lengths[b // 2] = 3000
    h = kvh * group
    pool, slots, offsets, te, stride, ko, vo = build_pool(rng, kvh, dim, lengths)
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=0, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=1, mask_dtype=0, window=0)
    out = run_paged(runtime, "llmopt_attention_q8_paged_batched", query, ck, cv, pool, slots, None,
                    params, lengths=lengths, offsets=offsets)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params,
                                         past_lengths=np.array(lengths), slot_offsets=offsets)
    assert np.all(np.isfinite(out))
    assert_close_to_oracle(out, expected, f"balanced split b{b} kv{kvh} d{dim}")


@pytest.mark.parametrize("b,kvh,group,dim,window,seed", [(9, 3, 3, 64, 200, 1), (70, 2, 4, 128, 65, 2),
                                                         (4, 8, 4, 128, 1024, 3), (3, 1, 1, 64, 4000, 4),
                                                         (8, 2, 8, 256, 333, 5)])
def test_decode_attention_sliding_window_over_ragged_batch(runtime, b, kvh, group, dim, window, seed):
    """A sliding window on the split-over-context kernels: every sequence reads its last window - 1
    cached tokens (the window counts the current token) through a slot table entered `first` entries
    in.  Contexts below, at and above the window, empty ones, and windows that start inside a tile."""
    rng = np.random.default_rng(100 + seed)
    lengths = [int(v) for v in rng.integers(1, 3 * window // 2 + 200, size=b)]
    for index, value in zip(range(b), [2 * window + 37, window - 1, window, window + 1, 0, 1, window - 2]):
        lengths[index] = value
    h = kvh * group
    pool, slots, offsets, te, stride, ko, vo = build_pool(rng, kvh, dim, lengths)
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=0, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=1, mask_dtype=0, window=window)
    out = run_paged(runtime, "llmopt_attention_q8_paged_batched", query, ck, cv, pool, slots, None,
                    params, lengths=lengths, offsets=offsets)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params,
                                         past_lengths=np.array(lengths), slot_offsets=offsets)
    assert np.all(np.isfinite(out))
    assert_close_to_oracle(out, expected, f"window {window} b{b} kv{kvh} d{dim}")
    # the window moves the result: without it the same launch gives something else
    no_window = PagedParams.from_buffer_copy(bytes(params))
    no_window.window = 0
    unwindowed = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, no_window,
                                           past_lengths=np.array(lengths), slot_offsets=offsets)
    assert np.abs(unwindowed[0].astype(np.float64) - expected[0].astype(np.float64)).max() > 1e-3


@pytest.mark.parametrize("name,h,kvh,dim,past,window", [
    ("llmopt_attention_q8_paged_simd_h64_gqa3", 9, 3, 64, 2048, 512),
    ("llmopt_attention_q8_paged_simd_generic", 32, 8, 128, 700, 300),
    ("llmopt_attention_q8_paged_simd_h64", 4, 4, 64, 100, 100),
    ("llmopt_attention_q8_paged_simd_generic", 8, 2, 128, 99, 100),
    ("llmopt_attention_q8_paged_simd_h256", 16, 4, 256, 1024, 0),
    ("llmopt_attention_q8_paged_simd_h256", 8, 1, 256, 777, 512)])
def test_reference_entries_with_sliding_window(runtime, name, h, kvh, dim, past, window):
    """The reference's own entries (one context length for the whole batch) with a window: the
    split-over-context kernels when the windowed context has 64 tokens or more."""
    rng = np.random.default_rng(past + window)
    b = 2
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [past])
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=1, mask_dtype=0, window=window)
    out = run_paged(runtime, name, query, ck, cv, pool, slots, None, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params)
    assert_close_to_oracle(out, expected, f"{name} window {window} of {past}")


ROW_CASES = [
    # (b, h, kvh, dim, past, q_len, window, mask_dtype)
    (1, 2, 1, 64, 10, 1, 0, 0), (2, 4, 2, 128, 33, 1, 8, 0), (1, 3, 1, 64, 20, 3, 0, 1),
    (1, 2, 2, 256, 17, 1, 0, 2), (1, 1, 1, 512, 9, 2, 0, 1), (1, 6, 2, 192, 12, 1, 0, 0),
    (1, 4, 1, 64, 0, 1, 0, 0),
]


@pytest.mark.parametrize("b,h,kvh,dim,past,q_len,window,mask_dtype", ROW_CASES)
def test_row_kernel_features(runtime, b, h, kvh, dim, past, q_len, window, mask_dtype):
    rng = np.random.default_rng(past * 7 + dim)
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [max(past, 1)])
    slots = slots[:past]
    query = rng.standard_normal((b, h, q_len, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    mask = None
    mask_batches = mask_heads = 0
    if mask_dtype == 1:
        mask = (rng.random((1, 1, q_len, past + q_len)) > 0.3).astype(np.uint8)
        mask[..., past] = 1
        mask_batches = mask_heads = 1
    elif mask_dtype == 2:
        allowed = rng.random((b, h, q_len, past + q_len)) > 0.3
        allowed[..., 0] = True
        mask = np.where(allowed, 0.0, -np.inf).astype(np.float16)
        mask_batches, mask_heads = b, h
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=mask_batches, mask_heads=mask_heads, token_elements=te,
                         key_offset=ko, value_offset=vo, group_size=64, token_stride=stride,
                         scale=1.0 / math.sqrt(dim), query_length=q_len, mask_dtype=mask_dtype,
                         window=window)
    out = run_paged(runtime, "llmopt_attention_q8_paged_simd_generic", query, ck, cv, pool, slots,
                    mask, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, mask, params)
    assert_close_to_oracle(out, expected, "row kernel")


GENERAL_CASES = [
    # (b, h, kvh, dim, past, q_len, window, mask_dtype, restride): several 64-key tiles, a tile with no
    # allowed key, a window that starts inside the context, pool rows that are not dword aligned
    (2, 4, 2, 128, 200, 3, 0, 2, 0), (1, 8, 2, 64, 300, 1, 150, 0, 0), (1, 2, 1, 192, 130, 2, 100, 1, 0),
    (1, 4, 4, 64, 257, 1, 0, 1, 2), (2, 2, 1, 128, 70, 2, 0, 0, 6), (1, 2, 1, 512, 65, 1, 0, 2, 0),
]


@pytest.mark.parametrize("b,h,kvh,dim,past,q_len,window,mask_dtype,restride", GENERAL_CASES)
def test_general_kernel_tiles_masks_windows_alignment(runtime, b, h, kvh, dim, past, q_len, window, mask_dtype,
                                                      restride):
    rng = np.random.default_rng(past * 3 + dim + restride)
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [past])
    if restride:  # the same tokens at a stride that is no multiple of four
        rows = pool.reshape(-1, stride)
        wider = np.zeros((rows.shape[0], stride + restride), dtype=np.uint8)
        wider[:, :stride] = rows
        pool, stride = wider.reshape(-1), stride + restride
    query = rng.standard_normal((b, h, q_len, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    mask, mask_batches, mask_heads = None, 0, 0
    if mask_dtype:
        allowed = rng.random((b, h, q_len, past + q_len)) > 0.4
        allowed[..., 64:128] = False      # a whole tile of keys without an allowed one
        allowed[..., past:] = True        # the query tokens themselves stay visible
        mask = allowed.astype(np.uint8) if mask_dtype == 1 else np.where(allowed, 0.0, -np.inf).astype(np.float16)
        mask_batches, mask_heads = b, h
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=mask_batches, mask_heads=mask_heads, token_elements=te, key_offset=ko,
                         value_offset=vo, group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim),
                         query_length=q_len, mask_dtype=mask_dtype, window=window)
    out = run_paged(runtime, "llmopt_attention_q8_paged_simd_generic", query, ck, cv, pool, slots, mask, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, mask, params)
    assert_close_to_oracle(out, expected, "general kernel")


@pytest.mark.parametrize("batches", [16, 1])
def test_decode_attention_full_size_closed_form(runtime, batches):
    """BASELINE's attention configuration (32/8 heads of 128, contexts up to 8192 tokens, scattered
    slots), far beyond what the oracle finishes in seconds.  Every cached key of a (sequence, KV head)
    is the same vector, so all past scores of a row coincide and the output has a closed form:
    (w_past * sum_t V_t + w_cur * v_cur) / (L * w_past + w_cur), evaluated here in float64 from the
    dequantised pool.  Batch 16 takes 128-token chunks, batch 1 the 64-token ones."""
    rng = np.random.default_rng(1234 + batches)
    heads, kv_heads, dim = 32, 8, 128
    lengths = rng.integers(512, 8193, size=batches).astype(np.uint32)
    lengths[0] = 8192
    token_elements, stride = layout(kv_heads, dim)
    total = int(lengths.sum())
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    slots = rng.permutation(total).astype(np.uint32)
    pool = np.zeros((total, stride), dtype=np.uint8)
    key_q = rng.integers(-127, 128, size=(batches, kv_heads * dim), dtype=np.int8)
    key_s = rng.uniform(0.01, 0.03, size=(batches, kv_heads * dim // 64)).astype(np.float16)
    value_q = rng.integers(-127, 128, size=(total, kv_heads * dim), dtype=np.int8)
    value_s = rng.uniform(0.01, 0.03, size=(total, kv_heads * dim // 64)).astype(np.float16)
    sequence_of = np.repeat(np.arange(batches), lengths)
    pool[slots, :kv_heads * dim] = key_q[sequence_of].view(np.uint8)
    pool[slots, kv_heads * dim:token_elements] = value_q.view(np.uint8)
    scales = np.concatenate([key_s[sequence_of], value_s], axis=1)
    pool[slots, token_elements:] = scales.view(np.uint8).reshape(total, -1)
    query = rng.standard_normal((batches, heads, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((batches, kv_heads, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((batches, kv_heads, 1, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = PagedParams(batches=batches, query_heads=heads, kv_heads=kv_heads, past_length=0, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=token_elements, key_offset=0,
                         value_offset=kv_heads * dim, group_size=64, token_stride=stride, scale=scale,
                         query_length=1, mask_dtype=0, window=0)
    out = run_paged(runtime, "llmopt_attention_q8_paged_batched", query, ck, cv, pool.reshape(-1), slots, None,
                    params, lengths=lengths, offsets=offsets)
    value = value_q.astype(np.float64).reshape(total, kv_heads, dim // 64, 64) * \
        value_s.astype(np.float64).reshape(total, kv_heads, dim // 64, 1)
    value = value.reshape(total, kv_heads, dim)
    key = (key_q.astype(np.float64).reshape(batches, kv_heads, dim // 64, 64) *
           key_s.astype(np.float64).reshape(batches, kv_heads, dim // 64, 1)).reshape(batches, kv_heads, dim)
    want = np.empty((batches, 1, heads, dim))
    group = heads // kv_heads
    for b in range(batches):
        rows = slice(int(offsets[b]), int(offsets[b] + lengths[b]))
        value_sum = value[rows].sum(axis=0)  # [kv_heads, dim]
        for h in range(heads):
            kvh = h // group
            q = query[b, h, 0].astype(np.float64)
            s_past = scale * float(q @ key[b, kvh])
            s_cur = scale * float(q @ ck[b, kvh, 0].astype(np.float64))
            top = max(s_past, s_cur)
            w_past, w_cur = math.exp(s_past - top), math.exp(s_cur - top)
            want[b, 0, h] = (w_past * value_sum[kvh] + w_cur * cv[b, kvh, 0].astype(np.float64)) / \
                (int(lengths[b]) * w_past + w_cur)
    assert_close_to_oracle(out, want, f"full-size closed form, batch {batches}")


@pytest.mark.parametrize("decoder,name", [(0, "int8x4_to_h2"), (1, "int8x4_to_h2_biased")])
def test_attention_int8_decoders_are_bit_exact(runtime, decoder, name):
    """The two int8 -> fp16 decoders of the attention kernels over every byte value in every byte
    lane: the integers oracle_q8_unpack produces for the same bytes (scale 1.0)."""
    values = np.arange(256, dtype=np.uint8)
    data = np.stack([np.roll(values, shift) for shift in (0, 1, 2, 3)], axis=1).reshape(-1)  # 1024 bytes
    out = runtime.create_buffer(data.size * 4)
    runtime.dispatch("llmopt_q8_decode_f32", [runtime.buffer_of_bytes(data), out], u32s(data.size, decoder))
    got = out.numpy(np.float32, (data.size,))
    np.testing.assert_array_equal(got, data.view(np.int8).astype(np.float32), err_msg=name)
    # the oracle's unpack of the same bytes as 16 tokens of one 64-wide head with scale 1.0
    tokens, dim = data.size // 64, 64
    pool = np.zeros((tokens, dim + 2), dtype=np.uint8)
    pool[:, :dim] = data.reshape(tokens, dim)
    pool[:, dim:] = np.array([1.0], dtype=np.float16).view(np.uint8)
    params = oracle.CacheParams(items=tokens, segment_offset=0, heads=1, head_dim=dim, group_size=64,
                                token_elements=dim, token_groups=1, token_stride=dim + 2,
                                source_items=tokens, source_offset=0)
    unpacked = oracle.q8_unpack(pool.reshape(-1), np.arange(tokens, dtype=np.uint32), params)
    np.testing.assert_array_equal(got, unpacked.astype(np.float32).reshape(-1), err_msg=name)


@pytest.mark.parametrize("name,b,h,kvh,dim,past,q_len,mask_dtype", [
    ("llmopt_attention_q8_paged_simd_h64_gqa3", 1, 9, 3, 64, 74, 118, 1),   # the reference's suffix prefill
    ("llmopt_attention_q8_paged_simd_generic", 2, 8, 2, 128, 300, 45, 1),
    ("llmopt_attention_q8_paged_simd_generic", 1, 4, 4, 128, 0, 16, 2),    # nothing cached yet
    ("llmopt_attention_q8_paged_simd_h64", 1, 4, 4, 64, 1000, 200, 2),
    ("llmopt_attention_q8_paged_simd_h256", 1, 4, 2, 256, 130, 33, 1),
    ("llmopt_attention_q8_paged_simd_generic", 1, 32, 8, 128, 515, 140, 1),
    # a few new tokens over a long context take the copy as well
    ("llmopt_attention_q8_paged_simd_h64_gqa3", 1, 9, 3, 64, 700, 3, 1),
    ("llmopt_attention_q8_paged_simd_generic", 2, 8, 4, 128, 300, 9, 2),
])
def test_suffix_prefill_over_cached_tokens(runtime, name, b, h, kvh, dim, past, q_len, mask_dtype):
    """Sixteen query tokens or more over a Q8 context, with the mask the reference builds for a suffix
    (causal over the new tokens, every cached token visible; lib/serving_engine.ml:1194-1201) as bytes
    or halves, plus a few holes: the context is copied out as halves once and the dense tile kernel
    runs over it.  Token-major output, GQA, a row whose mask allows nothing."""
    rng = np.random.default_rng(past * 3 + q_len + dim)
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [max(past, 1)])
    slots = slots[:past]
    query = rng.standard_normal((b, h, q_len, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    visible = np.arange(past + q_len)[None, :] <= past + np.arange(q_len)[:, None]
    visible = np.broadcast_to(visible, (b, 1, q_len, past + q_len)).copy()
    visible &= rng.random(visible.shape) > 0.05
    visible[:, :, 2, :] = False
    mask = visible.astype(np.uint8) if mask_dtype == 1 else np.where(visible, 0.0, -np.inf).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=b, mask_heads=1, token_elements=te, key_offset=ko, value_offset=vo,
                         group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim), query_length=q_len,
                         mask_dtype=mask_dtype, window=0)
    out = run_paged(runtime, name, query, ck, cv, pool, slots, mask, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, mask, params)
    assert np.all(out[:, 2].view(np.uint16) == 0)
    assert_close_to_oracle(out, expected, f"suffix prefill {name} {q_len} new after {past}")


@pytest.mark.parametrize("case", range(8))
def test_random_suffix_prefill(runtime, case):
    """Random paged attention with sixteen query tokens or more: head sizes 64 / 128 / 256, any layer of a
    pool of several layers, contexts from nothing to several hundred tokens, masks of either type, shared
    or per head, with random holes."""
    rng = np.random.default_rng(7000 + case)
    dim = int(rng.choice([64, 128, 256]))
    kvh = int(rng.integers(1, 4))
    h = kvh * int(rng.integers(1, 5))
    b = int(rng.integers(1, 3))
    layers = int(rng.integers(1, 4))
    layer = int(rng.integers(0, layers))
    past = int(rng.integers(0, 800)) if case else 0
    q_len = int(rng.integers(16, 200))
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [max(past, 1)], layers=layers, layer=layer)
    slots = slots[:past]
    query = rng.standard_normal((b, h, q_len, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, q_len, dim)).astype(np.float16)
    mask_heads = h if rng.random() < 0.5 else 1
    visible = np.arange(past + q_len)[None, :] <= past + np.arange(q_len)[:, None]
    visible = np.broadcast_to(visible, (b, mask_heads, q_len, past + q_len)).copy()
    visible &= rng.random(visible.shape) > 0.1
    mask_dtype = 1 + case % 2
    mask = visible.astype(np.uint8) if mask_dtype == 1 else np.where(visible, 0.0, -np.inf).astype(np.float16)
    params = PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=b, mask_heads=mask_heads, token_elements=te, key_offset=ko, value_offset=vo,
                         group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim), query_length=q_len,
                         mask_dtype=mask_dtype, window=0)
    out = run_paged(runtime, "llmopt_attention_q8_paged_simd_generic", query, ck, cv, pool, slots, mask, params)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, mask, params)
    assert_close_to_oracle(out, expected, f"random suffix prefill {case}: D={dim} {h}/{kvh} x{b}, {q_len} after {past}, "
                                          f"layer {layer} of {layers}")


def checkpoint_layout(layers, layer_elements):
    elements = layers * layer_elements
    return elements, elements + 2 * (elements // 64)


def quantize_groups(state):
    """The quantiser of lib/metal_cache_source.ml:245-272 on a flat f16 state, group by group."""
    groups = state.astype(np.float32).reshape(-1, 64)
    maximum = np.abs(groups).max(axis=1)
    scale = np.where(maximum == 0, np.float32(1.0), maximum / np.float32(127.0)).astype(np.float16)
    values = np.clip(np.rint(groups / scale.astype(np.float32)[:, None]), -127, 127).astype(np.int8)
    return values.reshape(-1), scale


@pytest.mark.parametrize("name", ["llmopt_cache_pack_checkpoint_q8", "llmopt_cache_pack_checkpoint_q8_simd"])
def test_checkpoint_pack_and_unpack_are_bit_exact(runtime, name):
    """One layer's recurrent state into slot `checkpoint` of a pool of checkpoints and back
    (lib/metal_cache_source.ml:245-343): int8 values and f16 scales against the quantiser's definition,
    the other layers and the other slots untouched, the unpacked halves against int8 x scale."""
    rng = np.random.default_rng(17)
    layers, layer_elements, slots = 3, 5 * 64, 4
    elements, stride = checkpoint_layout(layers, layer_elements)
    state = (rng.standard_normal(layer_elements) * 3).astype(np.float16)
    state[64:128] = 0  # an all-zero group stores scale 1.0
    start = rng.integers(0, 256, size=slots * stride, dtype=np.uint8)
    pool = runtime.buffer_of_bytes(start)
    layer, checkpoint = 1, 2
    params = u32s(checkpoint, layer, layer_elements, 64, elements, elements // 64, stride)
    runtime.dispatch(name, [runtime.buffer_of_bytes(state), pool], params,
                     grid=(layer_elements // 64 * 32, 1, 1), group=(256, 1, 1))
    got = pool.numpy(np.uint8, (slots, stride))
    values, scales = quantize_groups(state)
    expected = start.reshape(slots, stride).copy()
    expected[checkpoint, layer * layer_elements:(layer + 1) * layer_elements] = values.view(np.uint8)
    groups = layer_elements // 64
    expected[checkpoint, elements + 2 * layer * groups:elements + 2 * (layer + 1) * groups] = scales.view(np.uint8)
    np.testing.assert_array_equal(got, expected)
    assert scales[1] == np.float16(1.0)
    want = (values.astype(np.float32).reshape(-1, 64) * scales.astype(np.float32)[:, None]).astype(np.float16)
    for unpack in ("llmopt_cache_unpack_checkpoint_q8", "llmopt_cache_unpack_checkpoint_q8_vec4"):
        destination = runtime.buffer_of_bytes(np.full(layer_elements, np.nan, dtype=np.float16))
        runtime.dispatch(unpack, [pool, destination], params, grid=(layer_elements, 1, 1), group=(256, 1, 1))
        np.testing.assert_array_equal(destination.numpy(np.uint16, (layer_elements,)), want.reshape(-1).view(np.uint16))
    with pytest.raises(Exception, match="pool buffer is too small"):
        runtime.dispatch(name, [runtime.buffer_of_bytes(state), pool],
                         u32s(slots, layer, layer_elements, 64, elements, elements // 64, stride))
    with pytest.raises(Exception, match="layer lies outside"):
        runtime.dispatch(name, [runtime.buffer_of_bytes(state), pool],
                         u32s(0, layers, layer_elements, 64, elements, elements // 64, stride))
