"""Seeded random shapes through the C ABI against the CPU oracle.

The other GPU tests pin the shapes of the benchmark configurations and the edges each kernel's
launcher names.  These draw shapes the launchers were not written around - odd column counts, K of
one group, row counts on both sides of every kernel boundary, ragged contexts at any layer of a
multi-layer pool - so that a wrong bound in a kernel choice or a tile edge shows up as a parity
failure here rather than in a caller.  Sizes keep the oracle at a fraction of a second per case.
"""
import math

import numpy as np
import pytest

import oracle
from oracle import PagedParams
from tests.gpu_util import assert_close_to_oracle, w4_case
from tests.test_gpu_q8 import build_pool, run_paged
from tests.test_gpu_w4a16 import run_linear

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def draw_linear_shapes():
    rng = np.random.default_rng(4242)
    shapes = []
    # decode rows, the row-group kernel (9..32 rows of a small matrix) and the tiled GEMM above them
    for m in [1, 2, 3, 4, 5, 7, 8, 9, 13, 16, 17, 31, 32, 33, 40, 65, 129, 200]:
        for _ in range(2):
            k = 64 * int(rng.integers(1, 40))
            n = int(rng.integers(1, 700)) if rng.random() < 0.5 else 8 * int(rng.integers(1, 200))
            shapes.append((m, n, k))
    # the K values with kernels of their own, at column counts around those kernels' limits
    for k in (4096, 14336):
        for n in (760, 764, 3068, 3072, 3076, 7164, 7172, 9004, 14340):
            shapes.append((int(rng.integers(1, 9)), n, k))
    # keep the oracle quick: thin out the activation rows of the biggest products
    return [(m, n, k) for m, n, k in shapes if m * n * k <= 3.0e8]


LINEAR_SHAPES = draw_linear_shapes()


@pytest.mark.parametrize("m,n,k", LINEAR_SHAPES)
def test_random_linear_shapes(runtime, m, n, k):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    x, packed, scale, bias = w4_case(rng, m, n, k, bias=True)
    epilogue = int(rng.integers(0, 3))  # none, a [1, n] bias, an [m, n] residual
    if epilogue == 0:
        out = run_linear(runtime, x, packed, scale)
        expected = oracle.w4a16_linear(x, packed, scale, None)
    elif epilogue == 1:
        out = run_linear(runtime, x, packed, scale, bias=bias)
        expected = oracle.w4a16_linear(x, packed, scale, bias)
    else:
        residual = rng.standard_normal((m, n)).astype(np.float16)
        out = run_linear(runtime, x, packed, scale, residual=residual)
        expected = oracle.add(oracle.w4a16_linear(x, packed, scale, None), residual.astype(np.float32))
    assert_close_to_oracle(out, expected, f"linear {m}x{n}x{k} epilogue {epilogue}")


def draw_attention_cases():
    rng = np.random.default_rng(777)
    cases = []
    for index in range(28):
        dim = int(rng.choice([64, 128]))
        kv_heads = int(rng.choice([1, 2, 3, 4, 8]))
        group = int(rng.choice([1, 2, 3, 4, 8, 16]))
        batches = int(rng.integers(1, 9))
        layers = int(rng.choice([1, 1, 2, 5]))
        layer = int(rng.integers(0, layers))
        top = int(rng.choice([40, 130, 700, 2300, 5000]))
        lengths = [int(v) for v in rng.integers(0, top + 1, size=batches)]
        lengths[int(rng.integers(0, batches))] = top  # one sequence reaches the top of the range
        if kv_heads * group * dim * sum(lengths) > 6.0e7:  # the oracle's cost
            lengths = [value // 4 for value in lengths]
        cases.append((index, batches, kv_heads, group, dim, layers, layer, lengths))
    return cases


@pytest.mark.parametrize("index,batches,kv_heads,group,dim,layers,layer,lengths", draw_attention_cases())
def test_random_ragged_decode_attention(runtime, index, batches, kv_heads, group, dim, layers, layer, lengths):
    rng = np.random.default_rng(9000 + index)
    heads = kv_heads * group
    pool, slots, offsets, te, stride, ko, vo = build_pool(rng, kv_heads, dim, lengths, layers=layers, layer=layer)
    query = rng.standard_normal((batches, heads, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((batches, kv_heads, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((batches, kv_heads, 1, dim)).astype(np.float16)
    params = PagedParams(batches=batches, query_heads=heads, kv_heads=kv_heads, past_length=0, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko, value_offset=vo,
                         group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim), query_length=1,
                         mask_dtype=0, window=0)
    out = run_paged(runtime, "llmopt_attention_q8_paged_batched", query, ck, cv, pool, slots, None, params,
                    lengths=lengths, offsets=offsets)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params,
                                         past_lengths=np.array(lengths), slot_offsets=offsets)
    assert np.all(np.isfinite(out))
    assert_close_to_oracle(out, expected, f"ragged attention case {index}: {batches} x {heads}/{kv_heads} x {dim}, "
                                          f"layer {layer} of {layers}, contexts {lengths}")


def draw_projection_cases():
    rng = np.random.default_rng(1234)
    cases = []
    for m in [1, 1, 2, 3, 4, 5, 8, 8, 9, 11, 24, 32, 33, 70, 150]:
        k = 64 * int(rng.integers(1, 49))
        sizes = tuple(64 * int(v) for v in rng.integers(1, 13, size=3))
        ffn = 64 * int(rng.integers(1, 33))
        cases.append((m, k, sizes, ffn))
    return cases


@pytest.mark.parametrize("m,k,sizes,ffn", draw_projection_cases())
def test_random_qkv_and_ffn_shapes(runtime, m, k, sizes, ffn):
    """The QKV projection (three matrices, one launch), the dual-SwiGLU projection and the down
    projection with its residual at random widths, plain and normalising entries."""
    import struct
    from tests.gpu_util import linear_grid, u32s
    rng = np.random.default_rng(m * 7919 + k + ffn)
    epsilon = 1e-5
    x = (rng.standard_normal((m, k)) * 2.0).astype(np.float16)
    gain = rng.uniform(0.5, 1.5, size=k).astype(np.float16)
    normalised = oracle.rms_norm(x, gain, epsilon).astype(np.float16)
    mats = [w4_case(rng, 1, width, k)[1:3] for width in sizes]
    weights = []
    for packed, scale in mats:
        weights += [runtime.buffer_of_bytes(packed), runtime.buffer_of_bytes(scale)]
    bx, bg = runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(gain)
    suffix = "" if m == 1 else "_m4"
    blank = lambda width: runtime.buffer_of_bytes(np.full((m, width), np.nan, dtype=np.float16))

    plain = [blank(width) for width in sizes]
    runtime.dispatch("llmopt_w4a16_qkv_linear_f16_g64" + suffix, [bx, *weights, *plain], u32s(m, k, *sizes),
                     grid=(linear_grid(m * sum(sizes)), 1, 1), group=(256, 1, 1))
    normalising = [blank(width) for width in sizes]
    runtime.dispatch("llmopt_rms_w4a16_qkv_linear_f16_g64", [bx, bg, *weights, *normalising],
                     u32s(m, k, *sizes) + struct.pack("<f", epsilon),
                     grid=(linear_grid(m * sum(sizes)), 1, 1), group=(256, 1, 1))
    for (packed, scale), first, second, width in zip(mats, plain, normalising, sizes):
        assert_close_to_oracle(first.numpy(np.float16, (m, width)), oracle.w4a16_linear(x, packed, scale, None),
                               f"qkv {m}x{width}x{k}")
        assert_close_to_oracle(second.numpy(np.float16, (m, width)),
                               oracle.w4a16_linear(normalised, packed, scale, None), f"rms+qkv {m}x{width}x{k}")

    _, gate_w, gate_s, _ = w4_case(rng, 1, ffn, k)
    _, up_w, up_s, _ = w4_case(rng, 1, ffn, k)
    _, down_w, down_s, _ = w4_case(rng, 1, k, ffn)
    ffn_weights = [runtime.buffer_of_bytes(a) for a in (gate_w, gate_s, up_w, up_s)]
    params = u32s(m, ffn, k) + struct.pack("<f", epsilon)
    product = blank(ffn)
    runtime.dispatch("llmopt_rms_w4a16_dual_swiglu_f16_g64", [bx, bg, *ffn_weights, product], params,
                     grid=(linear_grid(m * ffn), 1, 1), group=(256, 1, 1))
    got_product = product.numpy(np.float16, (m, ffn))
    assert_close_to_oracle(got_product,
                           oracle.silu_mul(oracle.w4a16_linear(normalised, gate_w, gate_s, None),
                                           oracle.w4a16_linear(normalised, up_w, up_s, None)),
                           f"rms+dual swiglu {m}x{ffn}x{k}")
    residual = rng.standard_normal((m, k)).astype(np.float16)
    output = blank(k)
    runtime.dispatch("llmopt_w4a16_down_add_f16_g64" + suffix,
                     [product, runtime.buffer_of_bytes(down_w), runtime.buffer_of_bytes(down_s),
                      runtime.buffer_of_bytes(residual), output], params,
                     grid=(linear_grid(m * k), 1, 1), group=(256, 1, 1))
    assert_close_to_oracle(output.numpy(np.float16, (m, k)),
                           oracle.add(oracle.w4a16_linear(got_product, down_w, down_s, None),
                                      residual.astype(np.float32)), f"down+residual {m}x{k}x{ffn}")


def draw_dense_cases():
    rng = np.random.default_rng(31337)
    cases = []
    for index in range(24):
        dim = int(rng.choice([64, 128, 128, 64, 32, 96, 256]))
        kv_heads = int(rng.choice([1, 2, 3]))
        group = int(rng.choice([1, 2, 3, 4]))
        batches = int(rng.integers(1, 4))
        new = int(rng.choice([1, 7, 16, 31, 32, 33, 64, 90, 129, 200]))
        past = int(rng.choice([0, 0, 5, 64, 100, 257]))
        mode = int(rng.integers(0, 4))  # causal, none, bool mask, f16 mask
        layouts = int(rng.integers(0, 4))  # bit 0: token-major output, bit 1: token-major V
        cases.append((index, dim, kv_heads, group, batches, new, past, mode, layouts))
    return cases


@pytest.mark.parametrize("index,dim,kv_heads,group,batches,new,past,mode,layouts", draw_dense_cases())
def test_random_dense_attention(runtime, index, dim, kv_heads, group, batches, new, past, mode, layouts):
    """Dense fp16 attention (prefill, chunked prefill) at random lengths, head sizes on and off the
    matrix-core kernel, causal limits with cached tokens before them, masks of both types and both
    memory layouts of V and of the output."""
    from tests.test_gpu_dense_attention import attention_params, expected, run
    rng = np.random.default_rng(555 + index)
    heads = kv_heads * group
    length = past + new
    query = rng.standard_normal((batches, heads, new, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    scale = float(rng.choice([1.0 / math.sqrt(dim), 0.05, 0.3]))
    token_first_output, token_first_value = layouts & 1, (layouts >> 1) & 1
    mask, mask_batches, mask_heads, mask_dtype = None, 0, 0, 0
    if mode == 0:
        allowed = np.broadcast_to((np.arange(length)[None, :] <= past + np.arange(new)[:, None])[None, None],
                                  (batches, heads, new, length))
    elif mode == 1:
        allowed = np.ones((batches, heads, new, length), dtype=bool)
    else:
        mask_batches, mask_heads = batches, int(rng.choice([1, heads]))
        drawn = rng.random((mask_batches, mask_heads, new, length)) < 0.7
        drawn[..., 0] = True  # every row keeps a key
        mask_dtype = 1 if mode == 2 else 2
        mask = drawn.astype(np.uint8) if mode == 2 else np.where(drawn, 0.0, -np.inf).astype(np.float16)
        allowed = np.broadcast_to(drawn, (batches, heads, new, length))
    params = attention_params(batches, heads, new, length, dim, mask_batches, mask_heads, mode == 0, scale, kv_heads,
                              token_first_output=token_first_output, past_length=past if mode == 0 else 0,
                              token_first_value=token_first_value, mask_dtype=mask_dtype)
    value_in = np.ascontiguousarray(value.transpose(0, 2, 1, 3)) if token_first_value else value
    out_shape = (batches, new, heads, dim) if token_first_output else (batches, heads, new, dim)
    name = f"llmopt_attention_f16_simd_h{dim}" if dim in (64, 128, 256) and rng.random() < 0.5 else "llmopt_attention_f16"
    got = run(runtime, name, query, key, value_in, mask, params, out_shape)
    if token_first_output:
        got = got.transpose(0, 2, 1, 3)
    want = expected(query, key, value, allowed, scale)
    assert_close_to_oracle(got, want, f"dense case {index}: D={dim} {heads}/{kv_heads} heads, {new} new after {past}, "
                                      f"mode {mode}, layouts {layouts}, {name}")
