"""The reference's dispatch_* operators over the HIP backend (lib/metal_dispatch_linear.mli,
lib/metal_dispatch_attention.mli): kernel choice, error behaviour and results against the oracle."""
import math

import numpy as np
import pytest

import oracle
from oracle import PagedParams
from llmopt_amd import ops
from llmopt_amd.ops import BOOL, F16, F32, I32, U8, Value
from tests.gpu_util import assert_close_to_oracle, w4_case
from tests.test_gpu_q8 import build_pool

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


@pytest.fixture()
def operators(runtime):
    instance = ops.Operators(runtime)
    yield instance
    instance.close()


def w4_values(runtime, packed, scale):
    return [Value(runtime.buffer_of_bytes(packed), U8, packed.shape),
            Value(runtime.buffer_of_bytes(scale), F16, scale.shape)]


@pytest.mark.parametrize("m,expected_kernel", [(1, "llmopt_w4a16_linear_f16_g64"), (5, "llmopt_w4a16_linear_f16_g64_m4")])
def test_dispatch_w4a16_linear(runtime, operators, m, expected_kernel):
    rng = np.random.default_rng(m)
    n, k = 1536, 576
    x, packed, scale, bias = w4_case(rng, m, n, k, bias=True)
    out = Value(runtime.buffer_of_bytes(np.full((m, n), np.nan, np.float16)), F16, (m, n))
    base = [Value(runtime.buffer_of_bytes(x), F16, (m, k))] + w4_values(runtime, packed, scale)
    assert operators.w4a16_linear(m=m, n=n, k=k, has_bias=False, values=base, output=out) == [expected_kernel]
    assert_close_to_oracle(out.buffer.numpy(np.float16, (m, n)), oracle.w4a16_linear(x, packed, scale, None), "linear")
    # a [1, n] bias broadcasts over rows (stride 0) ...
    with_bias = base + [Value(runtime.buffer_of_bytes(bias), F16, (1, n))]
    operators.w4a16_linear(m=m, n=n, k=k, has_bias=True, values=with_bias, output=out)
    assert_close_to_oracle(out.buffer.numpy(np.float16, (m, n)), oracle.w4a16_linear(x, packed, scale, bias), "bias")
    # ... an [m, n] one is a residual (row stride n, lib/metal_dispatch_linear.ml:957-963)
    residual = rng.standard_normal((m, n)).astype(np.float16)
    with_residual = base + [Value(runtime.buffer_of_bytes(residual), F16, (m, n))]
    operators.w4a16_linear(m=m, n=n, k=k, has_bias=True, values=with_residual, output=out)
    expected = oracle.add(oracle.w4a16_linear(x, packed, scale, None), residual.astype(np.float32))
    if m > 1:
        assert_close_to_oracle(out.buffer.numpy(np.float16, (m, n)), expected, "residual")


def test_dispatch_w4a16_linear_rejects_inconsistent_bias(runtime, operators):
    a = Value(runtime.create_buffer(64), F16, (1, 8))
    with pytest.raises(ops.LlmoptError, match="W4A16 schedule command has inconsistent bias inputs"):
        operators.w4a16_linear(m=1, n=64, k=64, has_bias=True, values=[a, a, a], output=a)
    with pytest.raises(ops.LlmoptError, match="inconsistent bias inputs"):
        operators.w4a16_linear(m=1, n=64, k=64, has_bias=False, values=[a, a, a, a], output=a)


def test_dispatch_w4a16_qkv_linear_command(runtime, operators):
    rng = np.random.default_rng(2)
    m, k, n_q, n_k, n_v = 1, 576, 576, 192, 192
    x = rng.standard_normal((m, k)).astype(np.float16)
    weights = [w4_case(rng, m, n, k)[1:3] for n in (n_q, n_k, n_v)]
    values = [Value(runtime.buffer_of_bytes(x), F16, (m, k))]
    for packed, scale in weights:
        values += w4_values(runtime, packed, scale)
    outs = [Value(runtime.create_buffer(m * n * 2), F16, (m, n)) for n in (n_q, n_k, n_v)]
    kernels = operators.w4a16_qkv_linear_command(m=m, k=k, n_q=n_q, n_k=n_k, n_v=n_v, extra_outputs=outs[1:],
                                                 values=values, output=outs[0])
    assert kernels == ["llmopt_w4a16_qkv_linear_f16_g64"]
    for out, (packed, scale), n in zip(outs, weights, (n_q, n_k, n_v)):
        assert_close_to_oracle(out.buffer.numpy(np.float16, (m, n)), oracle.w4a16_linear(x, packed, scale, None), "qkv")
    with pytest.raises(ops.LlmoptError, match="requires 2 extra outputs"):
        operators.w4a16_qkv_linear_command(m=m, k=k, n_q=n_q, n_k=n_k, n_v=n_v, extra_outputs=outs[1:2],
                                           values=values, output=outs[0])
    with pytest.raises(ops.LlmoptError, match="W4A16 QKV linear command has inconsistent inputs"):
        operators.w4a16_qkv_linear_command(m=m, k=k, n_q=n_q, n_k=n_k, n_v=n_v, extra_outputs=outs[1:],
                                           values=values[:5], output=outs[0])


@pytest.mark.parametrize("m,dtype", [(1, np.float16), (3, np.float32)])
def test_dispatch_w4a16_swiglu_ffn_command(runtime, operators, m, dtype):
    rng = np.random.default_rng(4 + m)
    n, k = 1536, 576
    x, gate_w, gate_s, _ = w4_case(rng, m, n, k)
    x = x.astype(dtype)
    _, up_w, up_s, _ = w4_case(rng, m, n, k)
    _, down_w, down_s, _ = w4_case(rng, m, k, n)
    residual = rng.standard_normal((m, k)).astype(np.float16)
    norm = rng.uniform(0.5, 1.5, k).astype(np.float16)
    b = runtime.buffer_of_bytes
    values = [Value(b(x), F16 if dtype == np.float16 else F32, (m, k)), Value(b(residual), F16, (m, k)),
              *w4_values(runtime, gate_w, gate_s), *w4_values(runtime, up_w, up_s),
              *w4_values(runtime, down_w, down_s), Value(b(norm), F16, (k,))]
    out = Value(b(np.full((m, k), np.nan, np.float16)), F16, (m, k))
    batch = runtime.begin_batch()
    operators.set_batch(batch)
    kernels = operators.w4a16_swiglu_ffn_command(m=m, n=n, k=k, epsilon=1e-5, values=values, output=out)
    operators.set_batch(None)
    suffix = "" if m == 1 else "_m4"
    assert kernels == ["llmopt_w4a16_swiglu_rms_f16_g64" if dtype == np.float16 else "llmopt_w4a16_swiglu_rms_f32_g64",
                       "llmopt_w4a16_dual_swiglu_f16_g64" + suffix, "llmopt_w4a16_down_add_f16_g64" + suffix]
    batch.commit()
    normalized = oracle.rms_norm(x, norm, 1e-5).astype(np.float16)
    product = oracle.silu_mul(oracle.w4a16_linear(normalized, gate_w, gate_s, None),
                              oracle.w4a16_linear(normalized, up_w, up_s, None)).astype(np.float16)
    expected = oracle.add(oracle.w4a16_linear(product, down_w, down_s, None), residual.astype(np.float32))
    assert_close_to_oracle(out.buffer.numpy(np.float16, (m, k)), expected, "swiglu ffn")
    # the macro-op's limits (lib/metal_dispatch_linear.ml:283-309)
    bad = list(values)
    bad[8] = Value(values[8].buffer, F16, (k + 64,))
    with pytest.raises(ops.LlmoptError, match="W4A16 SwiGLU input metadata is inconsistent"):
        operators.w4a16_swiglu_ffn_command(m=m, n=n, k=k, epsilon=1e-5, values=bad, output=out)
    with pytest.raises(ops.LlmoptError, match="metadata is inconsistent"):
        operators.w4a16_swiglu_ffn_command(m=m, n=n, k=k, epsilon=0.0, values=values, output=out)
    with pytest.raises(ops.LlmoptError, match="W4A16 SwiGLU command has inconsistent inputs"):
        operators.w4a16_swiglu_ffn_command(m=m, n=n, k=k, epsilon=1e-5, values=values[:8], output=out)


def test_dispatch_w4a16_lm_head_argmax_command(runtime, operators):
    rng = np.random.default_rng(8)
    m, n, k = 2, 4000, 576
    x, packed, scale, _ = w4_case(rng, m, n, k)
    norm = rng.uniform(0.5, 1.5, k).astype(np.float16)
    b = runtime.buffer_of_bytes
    values = [Value(b(x), F16, (m, k)), Value(b(norm), F16, (k,)), *w4_values(runtime, packed, scale)]
    tokens = Value(b(np.zeros(m, np.uint32)), I32, (m,))
    logits = Value(b(np.full((m, n), np.nan, np.float16)), F16, (m, n))
    kernels = operators.w4a16_lm_head_argmax_command(m=m, n=n, k=k, epsilon=1e-5, extra_outputs=[logits],
                                                     values=values, output=tokens)
    assert kernels == ["llmopt_w4a16_lm_head_argmax_stage1_extra_f16", "llmopt_w4a16_lm_head_reduce"]
    expected = oracle.w4a16_linear(oracle.rms_norm(x, norm, 1e-5), packed, scale, None)
    assert_close_to_oracle(logits.buffer.numpy(np.float16, (m, n)), expected, "lm head logits")
    got = tokens.buffer.numpy(np.uint32, (m,))
    rms = float(np.sqrt(np.mean(expected.astype(np.float64) ** 2)))
    for row in range(m):
        assert expected[row, got[row]] >= expected[row].max() - 2e-2 * rms
    assert operators.w4a16_lm_head_argmax_command(m=m, n=n, k=k, epsilon=1e-5, extra_outputs=[], values=values,
                                                  output=tokens) == ["llmopt_w4a16_lm_head_argmax_stage1_f16",
                                                                     "llmopt_w4a16_lm_head_reduce"]
    with pytest.raises(ops.LlmoptError, match="at most one extra output"):
        operators.w4a16_lm_head_argmax_command(m=m, n=n, k=k, epsilon=1e-5, extra_outputs=[logits, logits],
                                               values=values, output=tokens)
    with pytest.raises(ops.LlmoptError, match="W4A16 LM-head argmax input metadata is inconsistent"):
        operators.w4a16_lm_head_argmax_command(m=m, n=n, k=4096, epsilon=1e-5, extra_outputs=[], values=values,
                                               output=tokens)


@pytest.mark.parametrize("heads,kvh,dim,kernel", [(9, 3, 64, "llmopt_attention_q8_paged_simd_h64_gqa3"),
                                                  (32, 8, 128, "llmopt_attention_q8_paged_simd_generic")])
def test_dispatch_paged_attention_q8(runtime, operators, heads, kvh, dim, kernel):
    rng = np.random.default_rng(heads)
    batches, past = 2, 333
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [past], layers=2, layer=1)
    query = rng.standard_normal((batches, heads, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((batches, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((batches, kvh, 1, dim)).astype(np.float16)
    b = runtime.buffer_of_bytes
    out = Value(b(np.full((batches, 1, heads, dim), np.nan, np.float16)), F16, (batches, 1, heads, dim))
    config = {"token_elements": te, "key_offset": ko, "value_offset": vo, "group_size": 64, "token_stride": stride,
              "scale": 1.0 / math.sqrt(dim), "window": None}
    arguments = dict(config=config, query=Value(b(query), F16, query.shape),
                     current_key=Value(b(ck), F16, ck.shape), current_value=Value(b(cv), F16, cv.shape),
                     pool=Value(b(pool), U8, pool.shape), slots=Value(b(slots), I32, slots.shape), mask_values=[],
                     output=out)
    assert operators.paged_attention_q8(**arguments) == [kernel]
    params = PagedParams(batches=batches, query_heads=heads, kv_heads=kvh, past_length=past, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko, value_offset=vo,
                         group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim), query_length=1,
                         mask_dtype=0, window=0)
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, params)
    assert_close_to_oracle(out.buffer.numpy(np.float16, expected.shape), expected, "paged attention")
    # a boolean mask over [past + 1] keys
    mask = (rng.random((1, 1, 1, past + 1)) > 0.3).astype(np.uint8)
    mask[..., -1] = 1
    arguments["mask_values"] = [Value(b(mask), BOOL, mask.shape)]
    operators.paged_attention_q8(**arguments)
    params.mask_batches, params.mask_heads, params.mask_dtype = 1, 1, 1
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, mask, params)
    assert_close_to_oracle(out.buffer.numpy(np.float16, expected.shape), expected, "masked paged attention")
    # error behaviour (lib/metal_dispatch_attention.ml:107-150)
    arguments["mask_values"] = [arguments["mask_values"][0]] * 2
    with pytest.raises(ops.LlmoptError, match="at most one mask value"):
        operators.paged_attention_q8(**arguments)
    arguments["mask_values"] = []
    arguments["query"] = Value(arguments["query"].buffer, F16, (batches, heads, dim))
    with pytest.raises(ops.LlmoptError, match=r"query must have shape \[b,h,q,d\]"):
        operators.paged_attention_q8(**arguments)


@pytest.mark.parametrize("dim,kernel", [(64, "llmopt_attention_f16_simd_h64"), (128, "llmopt_attention_f16_simd_h128"),
                                        (20, "llmopt_attention_f16")])
def test_dispatch_attention(runtime, operators, dim, kernel):
    """dispatch_attention: layouts read off the value shapes, past_length = L - q, kernel by head
    dimension (lib/metal_dispatch_attention.ml:6-102, lib/metal_dispatch_common.ml:166-189)."""
    rng = np.random.default_rng(dim)
    batches, heads, kv_heads, q_len, length = 1, 4, 2, 24, 40
    query = rng.standard_normal((batches, heads, q_len, dim)).astype(np.float16)
    key = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value = rng.standard_normal((batches, kv_heads, length, dim)).astype(np.float16)
    value_tm = np.ascontiguousarray(value.transpose(0, 2, 1, 3))
    out = runtime.create_buffer(batches * q_len * heads * dim * 2)
    scale = 1.0 / math.sqrt(dim)
    kernels = operators.attention(
        scale=scale, causal=True,
        query=Value(runtime.buffer_of_bytes(query), F16, query.shape),
        key=Value(runtime.buffer_of_bytes(key), F16, key.shape),
        value=Value(runtime.buffer_of_bytes(value_tm), F16, value_tm.shape), mask=None,
        output=Value(out, F16, (batches, q_len, heads * dim)))
    assert kernels == [kernel]
    got = out.numpy(np.float16, (batches, q_len, heads, dim)).transpose(0, 2, 1, 3)
    allowed = (np.arange(length)[None, :] <= (length - q_len) + np.arange(q_len)[:, None])[None, None]
    want = oracle.attention(query, np.repeat(key, 2, axis=1), np.repeat(value, 2, axis=1),
                            np.broadcast_to(allowed, (batches, heads, q_len, length)).astype(np.float32), scale)
    assert_close_to_oracle(got, want, f"dispatch_attention D={dim}")


def test_dispatch_attention_errors(runtime, operators):
    buffer = runtime.create_buffer(4096)
    q = Value(buffer, F16, (1, 2, 4, 64))
    with pytest.raises(ops.LlmoptError, match="attention query must have rank four"):
        operators.attention(scale=1.0, causal=False, query=Value(buffer, F16, (2, 4, 64)), key=q, value=q,
                            mask=None, output=q)
    with pytest.raises(ops.LlmoptError, match="attention key must have rank four"):
        operators.attention(scale=1.0, causal=False, query=q, key=Value(buffer, F16, (2, 4, 64)), value=q,
                            mask=None, output=q)
    with pytest.raises(ops.LlmoptError, match="attention value must match key in head-major or token-major layout"):
        operators.attention(scale=1.0, causal=False, query=q, key=q, value=Value(buffer, F16, (1, 2, 3, 64)),
                            mask=None, output=q)
    with pytest.raises(ops.LlmoptError, match="attention mask must have rank four"):
        operators.attention(scale=1.0, causal=False, query=q, key=q, value=q,
                            mask=Value(buffer, BOOL, (4, 4)), output=q)
    with pytest.raises(ops.LlmoptError, match="attention mask dtype"):
        operators.attention(scale=1.0, causal=False, query=q, key=q, value=q,
                            mask=Value(buffer, F32, (1, 1, 4, 4)), output=q)
