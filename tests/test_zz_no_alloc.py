"""llmopt_hip_attention_q8_paged_no_alloc (the entry point that allocates nothing) against the
dispatch entry it is a variant of, through the C ABI: same kernels, same chunk layout, so the
outputs must agree bit for bit - on two calls in a row, the second with a smaller input, so that
what the first call left in the shared static scratch is there when the second runs."""
import math

import numpy as np
import pytest

import oracle
from oracle import PagedParams
from tests.gpu_util import assert_close_to_oracle
from tests.test_gpu_q8 import build_pool, paged_params_bytes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    rt.set_stream(0)  # the default stream: the entry point under test is given the same one
    yield rt
    rt.close()


def case(runtime, seed, batches, heads, kv_heads, dim, past):
    rng = np.random.default_rng(seed)
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kv_heads, dim, [past])
    query = rng.standard_normal((batches, heads, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((batches, kv_heads, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((batches, kv_heads, 1, dim)).astype(np.float16)
    params = PagedParams(batches=batches, query_heads=heads, kv_heads=kv_heads, past_length=past, head_dim=dim,
                         mask_batches=0, mask_heads=0, token_elements=te, key_offset=ko, value_offset=vo,
                         group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim), query_length=1,
                         mask_dtype=0, window=0)
    b = runtime.buffer_of_bytes
    buffers = dict(query=b(query), ck=b(ck), cv=b(cv), pool=b(pool), slots=b(slots))
    return dict(params=params, raw=paged_params_bytes(params), host=(query, ck, cv, pool, slots), shape=(batches, 1, heads, dim),
                **buffers)


def run_no_alloc(runtime, c):
    from llmopt_amd.native import attention_q8_paged_no_alloc
    out = runtime.buffer_of_bytes(np.full(c["shape"], np.nan, dtype=np.float16))
    attention_q8_paged_no_alloc(c["raw"], c["query"], c["ck"], c["cv"], c["pool"], c["slots"], out, stream=0)
    return out


def run_dispatch(runtime, c):
    out = runtime.buffer_of_bytes(np.full(c["shape"], np.nan, dtype=np.float16))
    rows = c["shape"][0] * c["shape"][2]
    runtime.dispatch("llmopt_attention_q8_paged_simd_generic",
                     [c["query"], c["ck"], c["cv"], c["pool"], c["slots"], c["slots"], out], c["raw"],
                     grid=(((rows + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    return out.numpy(np.float16, c["shape"])


def test_two_calls_in_a_row_match_the_dispatch_entry(runtime):
    big = case(runtime, 5, batches=4, heads=32, kv_heads=8, dim=128, past=1500)
    small = case(runtime, 6, batches=1, heads=9, kv_heads=3, dim=64, past=513)
    # both calls are queued before either result is looked at
    out_big = run_no_alloc(runtime, big)
    out_small = run_no_alloc(runtime, small)
    got_big = out_big.numpy(np.float16, big["shape"])
    got_small = out_small.numpy(np.float16, small["shape"])
    for got, c, label in ((got_big, big, "first call"), (got_small, small, "second, smaller call")):
        want = run_dispatch(runtime, c)
        assert not np.isnan(got.astype(np.float32)).any(), label
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16), err_msg=label)
    query, ck, cv, pool, slots = small["host"]
    expected = oracle.paged_attention_q8(query, ck, cv, pool, slots, None, small["params"])
    assert_close_to_oracle(got_small, expected, "second, smaller call against the oracle")


def test_short_context_takes_no_scratch(runtime):
    c = case(runtime, 7, batches=2, heads=4, kv_heads=2, dim=128, past=33)
    got = run_no_alloc(runtime, c).numpy(np.float16, c["shape"])
    np.testing.assert_array_equal(got.view(np.uint16), run_dispatch(runtime, c).view(np.uint16))


def test_rejects_what_the_static_scratch_cannot_hold(runtime):
    from llmopt_amd.native import LlmoptError, NO_ALLOC_SCRATCH_BYTES, attention_q8_paged_no_alloc
    te, stride = 2 * 8 * 128, 2 * 8 * 128 + 2 * (2 * 8 * 128 // 64)
    past, batches = 8192, 300
    params = PagedParams(batches=batches, query_heads=32, kv_heads=8, past_length=past, head_dim=128, mask_batches=0,
                         mask_heads=0, token_elements=te, key_offset=0, value_offset=8 * 128, group_size=64,
                         token_stride=stride, scale=1.0, query_length=1, mask_dtype=0, window=0)
    tiny = runtime.create_buffer(16)
    pool = runtime.create_buffer(stride)
    slots = runtime.create_buffer(past * 4)
    with pytest.raises(LlmoptError) as error:
        attention_q8_paged_no_alloc(paged_params_bytes(params), tiny, tiny, tiny, pool, slots, tiny)
    assert error.value.code == -2
    assert "exceed the static scratch of %d bytes" % NO_ALLOC_SCRATCH_BYTES in str(error.value)
