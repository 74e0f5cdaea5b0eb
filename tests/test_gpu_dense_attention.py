"""GPU parity of dense fp16 attention (llmopt_attention_f16 and its per-head-dimension
entries) against the CPU oracle and the reference's own smoke vectors."""
import math
import struct

import numpy as np
import pytest

import oracle
from tests.gpu_util import assert_close_to_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def attention_params(batches, heads, query_length, key_length, head_dim, mask_batches, mask_heads, causal,
                     scale, kv_heads, token_first_output=0, past_length=0, token_first_value=0,
                     mask_dtype=0):
    """Metal_parameters.attention (lib/metal_parameters.ml:95-117): 56 bytes."""
    return struct.pack("<8IfIIIII", batches, heads, query_length, key_length, head_dim, mask_batches,
                       mask_heads, 1 if causal else 0, scale, kv_heads, token_first_output, past_length,
                       token_first_value, mask_dtype)


def run(runtime, name, query, key, value, mask, params, out_shape):
    b_query = runtime.buffer_of_bytes(query)
    buffers = [b_query, runtime.buffer_of_bytes(key), runtime.buffer_of_bytes(value),
               runtime.buffer_of_bytes(mask) if mask is not None else b_query]
    out = runtime.create_buffer(int(np.prod(out_shape)) * 2)
    # poison the output: rows the kernel must zero are then seen to be written
    out.write(np.full(int(np.prod(out_shape)), 0x7e00, dtype=np.uint16))
    rows = query.shape[0] * query.shape[1] * query.shape[2]
    runtime.dispatch(name, buffers + [out], params, grid=(rows, 1, 1), group=(64, 1, 1))
    return out.numpy(np.float16, out_shape)


def expected(query, key, value, allowed, scale):
    """Oracle (Cpu.attention semantics) with GQA expanded and every rule folded into one mask
    [b, h, q, L] of allowed keys."""
    b, h, q, d = query.shape
    kvh = key.shape[1]
    repeat = h // kvh
    key_e = np.repeat(key, repeat, axis=1)
    value_e = np.repeat(value, repeat, axis=1)
    return oracle.attention(query, key_e, value_e, allowed.astype(np.float32), scale, causal=False)


def test_reference_smoke_vector_2x2(runtime):
    """bin/ocaml_metal_primitives_smoke.ml:221-228,382-383: Q = K = I, V = diag(10, 20),
    bool mask [T, F; F, T], scale 1 -> the values themselves."""
    bits = lambda *v: np.array(v, dtype=np.uint16).view(np.float16).reshape(1, 1, 2, 2)
    query = bits(0x3c00, 0, 0, 0x3c00)
    value = bits(0x4900, 0, 0, 0x4d00)
    mask = np.array([1, 0, 0, 1], dtype=np.uint8)
    params = attention_params(1, 1, 2, 2, 2, 1, 1, False, 1.0, 1, mask_dtype=1)
    got = run(runtime, "llmopt_attention_f16", query, query, value, mask, params, (1, 1, 2, 2))
    assert got.view(np.uint16).reshape(-1).tolist() == [0x4900, 0, 0, 0x4d00]


def test_reference_smoke_vector_wide(runtime):
    """bin/native_schedule_fixture.ml:278-294, bin/ocaml_metal_primitives_smoke.ml:229-237,384-386:
    D = 256, two query heads on one KV head, f16 mask [0, -inf; 0, 0], token-major output
    [1, 2, 512]: first token sees key 0 only (1.0), second the mean of 1.0 and 3.0."""
    query = np.zeros((1, 2, 2, 256), dtype=np.float16)
    key = np.zeros((1, 1, 2, 256), dtype=np.float16)
    value = np.empty((1, 1, 2, 256), dtype=np.float16)
    value[0, 0, 0] = 1.0
    value[0, 0, 1] = 3.0
    mask = np.array([0, 0xfc00, 0, 0], dtype=np.uint16)
    params = attention_params(1, 2, 2, 2, 256, 1, 1, False, 1.0, 1, token_first_output=1, mask_dtype=2)
    for name in ("llmopt_attention_f16_simd_h256", "llmopt_attention_f16"):
        got = run(runtime, name, query, key, value, mask, params, (1, 2, 512))
        bits = got.view(np.uint16).reshape(-1)
        assert np.all(bits[:512] == 0x3c00) and np.all(bits[512:] == 0x4000), name


@pytest.mark.parametrize("dim,heads,kv_heads,length", [(64, 9, 3, 200), (128, 8, 2, 150), (64, 2, 2, 33),
                                                      (128, 4, 1, 512)])
def test_causal_prefill_matches_oracle(runtime, dim, heads, kv_heads, length):
    rng = np.random.default_rng(dim + length)
    batches = 2
    query = rng.standard_normal((batches, heads, length, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = attention_params(batches, heads, length, length, dim, 0, 0, True, scale, kv_heads)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value, None, params,
              (batches, heads, length, dim))
    allowed = np.tril(np.ones((length, length), dtype=bool))[None, None]
    want = expected(query, key, value, np.broadcast_to(allowed, (batches, heads, length, length)), scale)
    assert_close_to_oracle(got, want, f"causal prefill D={dim} L={length}")


@pytest.mark.parametrize("dim", [64, 128])
def test_chunked_prefill_with_past_and_token_major_layouts(runtime, dim):
    """A second prefill chunk: 40 new tokens after 100 cached ones, V and the output token-major."""
    rng = np.random.default_rng(11 + dim)
    batches, heads, kv_heads, new, past = 1, 6, 2, 40, 100
    length = past + new
    query = rng.standard_normal((batches, heads, new, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value_token_major = np.ascontiguousarray(value.transpose(0, 2, 1, 3))
    scale = 0.11
    params = attention_params(batches, heads, new, length, dim, 0, 0, True, scale, kv_heads,
                              token_first_output=1, past_length=past, token_first_value=1)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value_token_major, None, params,
              (batches, new, heads, dim))
    allowed = (np.arange(length)[None, :] <= past + np.arange(new)[:, None])[None, None]
    want = expected(query, key, value, np.broadcast_to(allowed, (batches, heads, new, length)), scale)
    assert_close_to_oracle(got.transpose(0, 2, 1, 3), want, f"chunked prefill D={dim}")


@pytest.mark.parametrize("mask_dtype", [1, 2])
@pytest.mark.parametrize("dim", [64, 96])
def test_masks_and_rows_without_keys(runtime, mask_dtype, dim):
    """Random masks (bool / f16), broadcast over heads, one query row with no allowed key -> zeros.
    D = 96 takes the row-serial kernel, D = 64 the matrix-core one."""
    rng = np.random.default_rng(5 + mask_dtype + dim)
    batches, heads, kv_heads, q_len, length = 2, 4, 4, 37, 70
    query = rng.standard_normal((batches, heads, q_len, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    allowed = rng.random((batches, 1, q_len, length)) < 0.6
    allowed[1, 0, 5, :] = False
    if mask_dtype == 1:
        mask = allowed.astype(np.uint8)
    else:
        mask = np.where(allowed, 0.0, -np.inf).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = attention_params(batches, heads, q_len, length, dim, batches, 1, False, scale, kv_heads,
                              mask_dtype=mask_dtype)
    name = f"llmopt_attention_f16_simd_h{dim}" if dim == 64 else "llmopt_attention_f16"
    got = run(runtime, name, query, key, value, mask, params, (batches, heads, q_len, dim))
    want = expected(query, key, value, np.broadcast_to(allowed, (batches, heads, q_len, length)), scale)
    assert np.all(got[1, :, 5, :].view(np.uint16) == 0)
    assert_close_to_oracle(got, want, f"masked attention dtype={mask_dtype} D={dim}")


@pytest.mark.parametrize("dim,q_len,length", [(128, 45, 77), (64, 33, 130), (128, 16, 64), (64, 100, 31)])
def test_ragged_shapes_without_mask_or_causal_limit(runtime, dim, q_len, length):
    """The 32 x 32-tile kernel with a last key tile and a last row tile that are only partly there
    (keys past the end are staged as copies of the last row and must weigh nothing)."""
    rng = np.random.default_rng(dim + q_len + length)
    batches, heads, kv_heads = 2, 4, 2
    query = rng.standard_normal((batches, heads, q_len, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = attention_params(batches, heads, q_len, length, dim, 0, 0, False, scale, kv_heads)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value, None, params,
              (batches, heads, q_len, dim))
    want = expected(query, key, value, np.ones((batches, heads, q_len, length), dtype=bool), scale)
    assert_close_to_oracle(got, want, f"ragged D={dim} q={q_len} L={length}")


def test_single_query_row_and_tiny_shapes(runtime):
    rng = np.random.default_rng(21)
    for dim, q_len, length in ((64, 1, 17), (128, 3, 5), (8, 4, 9)):
        query = rng.standard_normal((1, 2, q_len, dim)).astype(np.float16)
        key = rng.standard_normal((1, 2, length, dim)).astype(np.float16)
        value = rng.standard_normal((1, 2, length, dim)).astype(np.float16)
        params = attention_params(1, 2, q_len, length, dim, 0, 0, False, 0.3, 2)
        got = run(runtime, "llmopt_attention_f16", query, key, value, None, params, (1, 2, q_len, dim))
        want = expected(query, key, value, np.ones((1, 2, q_len, length), dtype=bool), 0.3)
        assert_close_to_oracle(got, want, f"tiny D={dim} q={q_len} L={length}")


@pytest.mark.parametrize("causal", [True, False])
def test_device_filling_launch_against_sampled_rows(runtime, causal):
    """32 heads x 2048 rows: 512 workgroups, as many as the device holds at once.  The kernel maps
    its one-dimensional grid to (row slab, head) itself - every XCD every slab length, the second
    half of each run of workgroups backwards - and every output row must still be the right one:
    all heads, one row out of every 29 (every 128-row slab is hit) against the oracle."""
    rng = np.random.default_rng(123 + causal)
    heads, kv_heads, length, dim = 32, 8, 2048, 64
    query = rng.standard_normal((1, heads, length, dim)).astype(np.float16)
    key = rng.standard_normal((1, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((1, kv_heads, length, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = attention_params(1, heads, length, length, dim, 0, 0, causal, scale, kv_heads)
    print(f"dense attention 32 heads x 2048 rows causal={causal}", flush=True)
    got = run(runtime, "llmopt_attention_f16_simd_h64", query, key, value, None, params, (1, heads, length, dim))
    rows = np.unique(np.concatenate([[0, 31, 32, length - 1], np.arange(5, length, 29)]))
    allowed = np.ones((len(rows), length), dtype=bool)
    if causal:
        allowed = np.arange(length)[None, :] <= rows[:, None]
    want = expected(query[:, :, rows], key, value, np.broadcast_to(allowed[None, None], (1, heads, len(rows), length)),
                    scale)
    assert_close_to_oracle(got[:, :, rows], want, f"sampled rows, causal={causal}")
    assert not np.any(got.view(np.uint16) == 0x7e00)  # every row was written


def test_softmax_shift_invariance_at_full_size(runtime):
    """Prefill 2048 x 2048, D = 128: a property the oracle is too slow for.  With every key equal
    the output is the running mean of V (closed form), whatever the scores are."""
    rng = np.random.default_rng(77)
    heads, kv_heads, length, dim = 4, 1, 2048, 128
    query = rng.standard_normal((1, heads, length, dim)).astype(np.float16)
    key = np.broadcast_to(rng.standard_normal((1, kv_heads, 1, dim)).astype(np.float16),
                          (1, kv_heads, length, dim)).copy()
    value = rng.standard_normal((1, kv_heads, length, dim)).astype(np.float16)
    params = attention_params(1, heads, length, length, dim, 0, 0, True, 1.0 / math.sqrt(dim), kv_heads)
    got = run(runtime, "llmopt_attention_f16_simd_h128", query, key, value, None, params,
              (1, heads, length, dim))
    running_mean = np.cumsum(value[0, 0].astype(np.float64), axis=0) / np.arange(1, length + 1)[:, None]
    want = np.broadcast_to(running_mean[None, None], (1, heads, length, dim))
    assert_close_to_oracle(got, want, "equal keys -> running mean of V")


def test_prefill_then_q8_pack_then_paged_decode(runtime):
    """The step on the other side of the KV cache: prefill attention over fp16 K/V, the same K/V
    quantised into the pool (lib/serving_engine.ml:409-421), then one decode step over the pool.
    The decode row must agree with dense attention over the dequantised cache (oracle) and, to
    quantisation error, with dense attention over the fp16 K/V."""
    from oracle import CacheParams, PagedParams
    rng = np.random.default_rng(31)
    heads, kv_heads, dim, length = 8, 2, 128, 96
    token_elements = 2 * kv_heads * dim
    stride = token_elements + 2 * (token_elements // 64)
    key = rng.standard_normal((1, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((1, kv_heads, length, dim)).astype(np.float16)
    slots = rng.permutation(length).astype(np.uint32)
    pool = runtime.buffer_of_bytes(np.zeros(length * stride, dtype=np.uint8))
    runtime.dispatch("llmopt_cache_pack_attention_q8_pair_simd",
                     [runtime.buffer_of_bytes(key), runtime.buffer_of_bytes(value),
                      runtime.buffer_of_bytes(slots), pool],
                     struct.pack("<11I", length, 0, kv_heads * dim, kv_heads, dim, 64, token_elements,
                                 token_elements // 64, stride, length, 0),
                     grid=(length * kv_heads * 32, 1, 1), group=(256, 1, 1))
    query = rng.standard_normal((1, heads, 1, dim)).astype(np.float16)
    current_key = rng.standard_normal((1, kv_heads, 1, dim)).astype(np.float16)
    current_value = rng.standard_normal((1, kv_heads, 1, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    out = runtime.create_buffer(heads * dim * 2)
    b_slots = runtime.buffer_of_bytes(slots)
    runtime.dispatch("llmopt_attention_q8_paged_simd_generic",
                     [runtime.buffer_of_bytes(query), runtime.buffer_of_bytes(current_key),
                      runtime.buffer_of_bytes(current_value), pool, b_slots, b_slots, out],
                     struct.pack("<12IfIII", 1, heads, kv_heads, length, dim, 0, 0, token_elements, 0,
                                 kv_heads * dim, 64, stride, scale, 1, 0, 0),
                     grid=(256, 1, 1), group=(256, 1, 1))
    decode = out.numpy(np.float16, (1, 1, heads, dim))
    host_pool = pool.numpy(np.uint8, (length * stride,))
    paged = oracle.paged_attention_q8(
        query, current_key, current_value, host_pool, slots, None,
        PagedParams(batches=1, query_heads=heads, kv_heads=kv_heads, past_length=length, head_dim=dim,
                    mask_batches=0, mask_heads=0, token_elements=token_elements, key_offset=0,
                    value_offset=kv_heads * dim, group_size=64, token_stride=stride, scale=scale,
                    query_length=1, mask_dtype=0, window=0))
    assert_close_to_oracle(decode, paged, "decode over the packed prefill cache")
    # dense attention of the same query over [prefill K/V ; current K/V] in fp16
    all_key = np.concatenate([key, current_key], axis=2)
    all_value = np.concatenate([value, current_value], axis=2)
    params = attention_params(1, heads, 1, length + 1, dim, 0, 0, True, scale, kv_heads,
                              token_first_output=1, past_length=length)
    dense = run(runtime, "llmopt_attention_f16_simd_h128", query, all_key, all_value, None, params,
                (1, 1, heads, dim))
    difference = decode.astype(np.float64) - dense.astype(np.float64)
    relative = np.linalg.norm(difference) / np.linalg.norm(dense.astype(np.float64))
    assert relative < 2e-2, f"Q8 cache changes the decode row by {relative:.3e}"


def test_rejects_bad_arguments(runtime):
    query = np.zeros((1, 2, 4, 64), dtype=np.float16)
    key = np.zeros((1, 2, 4, 64), dtype=np.float16)
    good = attention_params(1, 2, 4, 4, 64, 0, 0, False, 1.0, 2)
    with pytest.raises(Exception):
        run(runtime, "llmopt_attention_f16", query, key[:, :, :2], key, None, good, (1, 2, 4, 64))
    with pytest.raises(Exception):
        run(runtime, "llmopt_attention_f16", query, key, key, None, good[:40], (1, 2, 4, 64))
    bad_heads = attention_params(1, 2, 4, 4, 64, 0, 0, False, 1.0, 3)
    with pytest.raises(Exception):
        run(runtime, "llmopt_attention_f16", query, key, key, None, bad_heads, (1, 2, 4, 64))


def check_attention_case(runtime, dim, heads, kv_heads, new, past, mode):
    """Two sequences of `new` query tokens after `past` cached ones against the oracle: causal limits,
    no limit, bool and f16 masks with a row without keys and a row whose first keys are all masked;
    head-major or token-major V and output by the parity of the length."""
    rng = np.random.default_rng(dim + heads + new + past)
    batches, length = 2, past + new
    query = rng.standard_normal((batches, heads, new, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    mask, mask_batches, mask_heads, mask_dtype = None, 0, 0, 0
    if mode == "causal":
        allowed = np.broadcast_to((np.arange(length)[None, :] <= past + np.arange(new)[:, None])[None, None],
                                  (batches, heads, new, length))
    elif mode == "none":
        allowed = np.ones((batches, heads, new, length), dtype=bool)
    else:
        mask_batches, mask_heads = batches, heads
        allowed = rng.random((batches, heads, new, length)) < 0.5
        allowed[:, :, 3, :] = False      # a row without keys
        allowed[:, :, 5, :200] = False   # a row whose first shares are empty
        mask_dtype = 1 if mode == "bool" else 2
        mask = allowed.astype(np.uint8) if mode == "bool" else np.where(allowed, 0.0, -np.inf).astype(np.float16)
    token_major = (new + past) % 2 == 1
    params = attention_params(batches, heads, new, length, dim, mask_batches, mask_heads, mode == "causal", scale,
                              kv_heads, token_first_output=int(token_major), past_length=past if mode == "causal" else 0,
                              token_first_value=int(token_major), mask_dtype=mask_dtype)
    value_in = np.ascontiguousarray(value.transpose(0, 2, 1, 3)) if token_major else value
    out_shape = (batches, new, heads, dim) if token_major else (batches, heads, new, dim)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value_in, mask, params, out_shape)
    if token_major:
        got = got.transpose(0, 2, 1, 3)
    want = expected(query, key, value, allowed, scale)
    if mode in ("bool", "f16"):
        assert np.all(got[:, :, 3, :].view(np.uint16) == 0)
    assert_close_to_oracle(got, want, f"D={dim} {heads}/{kv_heads} {new} new after {past}, {mode}")


@pytest.mark.parametrize("dim,heads,kv_heads,new,past,mode", [
    (64, 9, 3, 700, 0, "causal"), (128, 4, 2, 45, 900, "causal"), (64, 2, 1, 33, 257, "none"),
    (128, 2, 2, 130, 300, "bool"), (64, 3, 3, 64, 1000, "f16"), (128, 1, 1, 1000, 0, "causal"),
])
def test_small_launches_split_the_keys_of_a_slab_over_the_waves(runtime, dim, heads, kv_heads, new, past, mode):
    """Launches with fewer 128-row workgroups than the device has CUs and at least 256 keys: the four
    waves of a workgroup share 32 query rows and take a quarter of every 128-key stage each, and
    their shares (maxima, denominators, weighted sums) are folded through LDS.  Causal limits with
    cached tokens, partial last stages and tiles, rows past the end, both mask types, both layouts."""
    check_attention_case(runtime, dim, heads, kv_heads, new, past, mode)


@pytest.mark.parametrize("heads,kv_heads,new,past,mode", [
    (4, 2, 300, 0, "causal"), (2, 1, 45, 211, "causal"), (2, 2, 33, 100, "none"), (3, 1, 130, 70, "bool"),
    (2, 2, 64, 191, "f16"), (8, 4, 16, 0, "causal"),
])
def test_heads_of_256_on_the_tile_kernel(runtime, heads, kv_heads, new, past, mode):
    """llmopt_attention_f16_simd_h256 with sixteen query rows or more: the 32 x 32 tile kernel with
    eight output blocks per wave and 128 KB of K and V stages per workgroup."""
    check_attention_case(runtime, 256, heads, kv_heads, new, past, mode)


@pytest.mark.parametrize("dim,heads,kv_heads,batches,tokens,past,mask_dtype,window", [
    (128, 16, 4, 3, 700, 0, 2, 0),     # 288 workgroups of 128 rows: the four-wave slabs, f16 causal mask
    (64, 24, 8, 2, 650, 70, 1, 0),     # byte mask of a suffix over cached tokens
    (128, 16, 16, 3, 640, 0, 2, 150),  # sliding window: the first stages of later slabs are forbidden too
    (64, 3, 1, 1, 900, 0, 2, 0),       # few workgroups: 32-row slabs with the keys split over the waves
    (128, 2, 2, 1, 515, 0, 1, 200),    # the same with a window and rows that are not whole runs of four keys
    (256, 2, 1, 2, 300, 33, 2, 64),
])
def test_masks_that_forbid_whole_stages(runtime, dim, heads, kv_heads, batches, tokens, past, mask_dtype, window):
    """The masks the reference's prefill builds (lib/serving_engine.ml:303-321, 1194-1201): causal over
    the new tokens after `past` cached ones, optionally a sliding window, as halves (0 / -inf) or
    bytes, one mask for all batches and heads.  Most stages of keys are forbidden to most slabs of
    rows: the pass over the mask says which, and the attention kernel walks only the others."""
    rng = np.random.default_rng(dim + heads + tokens + past + window)
    length = past + tokens
    query = rng.standard_normal((batches, heads, tokens, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    position = past + np.arange(tokens)[:, None]
    keys = np.arange(length)[None, :]
    visible = keys <= position
    if window:
        visible &= keys > position - window
    allowed = np.broadcast_to(visible[None, None], (batches, heads, tokens, length))
    mask = np.where(visible, 0.0, -np.inf).astype(np.float16) if mask_dtype == 2 else visible.astype(np.uint8)
    params = attention_params(batches, heads, tokens, length, dim, 1, 1, False, scale, kv_heads, mask_dtype=mask_dtype)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value, mask[None, None], params,
              (batches, heads, tokens, dim))
    want = expected(query, key, value, allowed, scale)
    assert_close_to_oracle(got, want, f"mask of whole stages D={dim} {heads}/{kv_heads} x {tokens} after {past}, window {window}")


@pytest.mark.parametrize("dim,heads,kv_heads,batches,tokens,mask_dtype", [
    (128, 16, 4, 3, 700, 1),   # 288 workgroups: two groups of four waves per slab
    (64, 24, 8, 4, 680, 2),    # 576 workgroups: four waves per slab
    (64, 4, 2, 2, 1100, 1),    # 32-row slabs with the keys split over the waves
])
def test_masks_of_every_batch_and_head(runtime, dim, heads, kv_heads, batches, tokens, mask_dtype):
    """A mask of its own for every (batch, head): causal with a sliding window whose width depends on
    the head and a band of forbidden keys that depends on the batch - so the stages a slab has to
    walk differ from one mask row group to the next."""
    rng = np.random.default_rng(dim + heads + tokens)
    query = rng.standard_normal((batches, heads, tokens, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, tokens, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, tokens, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    rows = np.arange(tokens)[:, None]
    keys = np.arange(tokens)[None, :]
    allowed = np.empty((batches, heads, tokens, tokens), dtype=bool)
    for b in range(batches):
        for h in range(heads):
            visible = (keys <= rows) & (keys > rows - (90 + 37 * h))
            visible &= ~((keys >= 100 + 64 * b) & (keys < 230 + 64 * b))
            allowed[b, h] = visible
    mask = np.where(allowed, 0.0, -np.inf).astype(np.float16) if mask_dtype == 2 else allowed.astype(np.uint8)
    params = attention_params(batches, heads, tokens, tokens, dim, batches, heads, False, scale, kv_heads,
                              mask_dtype=mask_dtype)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value, mask, params,
              (batches, heads, tokens, dim))
    want = expected(query, key, value, allowed, scale)
    assert_close_to_oracle(got, want, f"per-head masks D={dim} {heads}/{kv_heads} x {tokens}")


@pytest.mark.parametrize("case", range(10))
def test_random_block_masks(runtime, case):
    """Masks made of random rectangles of allowed keys (so that whole stages, whole tiles, single rows
    and single keys are forbidden in no particular pattern), random geometry: every slab layout, both
    mask types, masks shared or per batch / head, rows of the mask that are and are not whole runs."""
    rng = np.random.default_rng(9000 + case)
    dim = int(rng.choice([64, 128, 256]))
    kv_heads = int(rng.integers(1, 4))
    heads = kv_heads * int(rng.integers(1, 4))
    batches = int(rng.integers(1, 3))
    new = int(rng.integers(16, 700))
    past = int(rng.integers(0, 900))
    if case % 3 == 0:  # enough workgroups of 128 rows for the four- and eight-wave slabs
        heads, kv_heads, batches, new = 16 * int(rng.integers(1, 3)), 8, int(rng.integers(2, 4)), int(rng.integers(500, 800))
        dim = int(rng.choice([64, 128]))
    length = past + new
    if case % 2 == 0:
        length = (length + 7) // 8 * 8
        past = length - new
    query = rng.standard_normal((batches, heads, new, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    mask_batches = batches if rng.random() < 0.5 else 1
    mask_heads = heads if rng.random() < 0.5 else 1
    allowed = np.zeros((mask_batches, mask_heads, new, length), dtype=bool)
    for b in range(mask_batches):
        for h in range(mask_heads):
            for _ in range(int(rng.integers(1, 6))):
                r0, k0 = int(rng.integers(0, new)), int(rng.integers(0, length))
                r1 = min(new, r0 + int(rng.integers(1, new + 1)))
                k1 = min(length, k0 + int(rng.integers(1, length + 1)))
                allowed[b, h, r0:r1, k0:k1] = True
    allowed[:, :, new // 2, :] = False
    mask_dtype = 1 + case % 2
    mask = allowed.astype(np.uint8) if mask_dtype == 1 else np.where(allowed, 0.0, -np.inf).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    params = attention_params(batches, heads, new, length, dim, mask_batches, mask_heads, False, scale, kv_heads,
                              mask_dtype=mask_dtype)
    got = run(runtime, f"llmopt_attention_f16_simd_h{dim}", query, key, value, mask, params, (batches, heads, new, dim))
    want = expected(query, key, value, np.broadcast_to(allowed, (batches, heads, new, length)), scale)
    assert np.all(got[:, :, new // 2].view(np.uint16) == 0)
    assert_close_to_oracle(got, want, f"random block mask {case}: D={dim} {heads}/{kv_heads} x{batches}, {new} after {past}")


@pytest.mark.parametrize("dim,heads,kv_heads,batches,q_len,past,masks", [
    (64, 9, 3, 1, 4, 300, [1, 3, 7, 15, 0, 0, 0, 0]),          # the default chain of four drafts
    (64, 4, 4, 2, 8, 0, [1, 3, 5, 11, 21, 37, 69, 133]),       # a tree; nothing cached
    (128, 8, 2, 1, 6, 1000, [1, 3, 5, 9, 19, 35, 0, 0]),
    (128, 2, 1, 1, 10, 40, [1, 2, 4, 8, 16, 32, 64, 128]),     # query tokens 8 and 9 see the past only
    (256, 2, 2, 1, 3, 500, [1, 1, 5, 0, 0, 0, 0, 0]),
])
def test_speculative_tree_attention(runtime, dim, heads, kv_heads, batches, q_len, past, masks):
    """llmopt_attention_tree_speculative_f16{,_simd_h64}: draft tokens over the cached keys and over each
    other as eight bit masks say (lib/metal_attention_source.ml:361-381); token-major V and output.
    The expected rows are the oracle's dense attention under the mask that function describes."""
    rng = np.random.default_rng(dim + q_len + past)
    length = past + q_len
    query = rng.standard_normal((batches, heads, q_len, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    scale = 1.0 / math.sqrt(dim)
    allowed = np.zeros((q_len, length), dtype=bool)
    allowed[:, :past] = True
    for q in range(min(q_len, 8)):
        for draft in range(q_len):
            allowed[q, past + draft] = bool((masks[q] >> draft) & 1)
    params = struct.pack("<7If8I", batches, heads, q_len, length, dim, kv_heads, past, scale, *masks)
    name = "llmopt_attention_tree_speculative_f16_simd_h64" if dim == 64 else "llmopt_attention_tree_speculative_f16"
    out = runtime.buffer_of_bytes(np.full((batches, q_len, heads, dim), np.nan, dtype=np.float16))
    value_token_major = np.ascontiguousarray(value.transpose(0, 2, 1, 3))
    runtime.dispatch(name, [runtime.buffer_of_bytes(query), runtime.buffer_of_bytes(key),
                            runtime.buffer_of_bytes(value_token_major), out], params,
                     grid=(((batches * heads * q_len + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    got = out.numpy(np.float16, (batches, q_len, heads, dim)).transpose(0, 2, 1, 3)
    want = expected(query, key, value, np.broadcast_to(allowed[None, None], (batches, heads, q_len, length)), scale)
    if past == 40:  # rows without a visible key at all do not occur here; rows 8, 9 see exactly the past
        assert np.all(np.isfinite(got))
    assert_close_to_oracle(got, want, f"tree attention D={dim} {heads}/{kv_heads}, {q_len} drafts after {past}")
