"""End-to-end parity of one decode step (embedding -> layers -> LM-head argmax)
built by llmopt_amd.decode_step against the same chain composed from the CPU
oracle, with every kernel boundary rounded to half as the kernels store it."""
import numpy as np
import pytest

from oracle.chain import decode_chain as oracle_step
from tests.gpu_util import assert_close_to_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def ragged_lengths(batch, seed):
    """Context lengths of a batch: short and long ones side by side, 1 .. 300 tokens."""
    rng = np.random.default_rng(seed)
    lengths = rng.integers(1, 301, size=batch)
    lengths[0], lengths[-1] = 300, 1
    return [int(v) for v in lengths]


# Batch 1-2 run the register-activation GEMV, 3-8 the matrix-core GEMV (normalising its rows
# itself), 9-32 its row-grouped form: batch 8 and 32 are the sizes the decode-step benchmark times.
@pytest.mark.parametrize("batch,lengths", [(1, [37]), (1, [77]), (2, [130, 9]), (3, [0, 70, 12]), (3, [64, 5, 300]), (8, ragged_lengths(8, 5)),
                                           (32, ragged_lengths(32, 6))])
@pytest.mark.parametrize("launches", [6, 5, 4, 3], ids=["six_launches_a_layer", "five_launches_a_layer", "four_launches_a_layer",
                                                        "three_launches_a_layer"])
def test_decode_step_matches_oracle_chain(runtime, batch, lengths, launches):
    from llmopt_amd.decode_step import DecodeConfig, DecodeStep, random_weights
    if launches == 3 and max(lengths) < 64:
        pytest.skip("the projecting attention takes contexts of 64 tokens and more")
    rng = np.random.default_rng(17 + batch)
    config = DecodeConfig(layers=2, vocabulary=1000)
    weights = random_weights(config, rng)
    total = sum(lengths)
    capacity = total + batch + 3
    order = rng.permutation(capacity).astype(np.uint32)
    slots, new_slots = order[:total], order[total:total + batch]
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    stride, elements = config.token_stride, config.token_elements
    pool = np.zeros((capacity, stride), dtype=np.uint8)
    pool[:, :elements] = np.clip(np.rint(rng.standard_normal((capacity, elements)) * 38), -127, 127) \
        .astype(np.int8).view(np.uint8)
    pool[:, elements:] = rng.uniform(0.02, 0.035, (capacity, elements // 64)).astype(np.float16) \
        .view(np.uint8).reshape(capacity, -1)
    pool = pool.reshape(-1)
    positions = lengths
    tokens = rng.integers(0, config.vocabulary, batch)

    device_pool = runtime.buffer_of_bytes(pool)
    step = DecodeStep(runtime, config, weights, batch, device_pool, runtime.buffer_of_bytes(slots), offsets,
                      lengths, new_slots, positions, fused=launches < 5, projecting=launches == 3, fused_qkv=launches == 5)
    assert len(step.dispatches) == {6: 14, 5: 12, 4: 11, 3: 10}[launches]  # (the last layer of a fused step: five)
    got_tokens = step.run(tokens)
    got_hidden = step.work["x"][0].numpy(np.float16, (batch, config.hidden))

    hidden, logits, expected_pool = oracle_step(config, weights, pool, slots, offsets, lengths, new_slots,
                                                positions, tokens)
    # Every kernel is held to rel-L2 1e-3 on its own in the other test files.  Here 19 kernels
    # are chained and each stores half: a one-ulp difference in an intermediate (2^-11 relative)
    # is carried by the residual stream, so the chain is held to 4e-3.
    assert_close_to_oracle(got_hidden, hidden, "hidden state after the last layer", rel_l2_tol=4e-3)
    rms = float(np.sqrt(np.mean(logits.astype(np.float64) ** 2)))
    for b in range(batch):
        assert float(logits[b, got_tokens[b]]) >= float(logits[b].max()) - 2e-2 * rms
    # the new token's K/V landed in its slot: int8 values within one quantum; scales within two ulps
    # (a key that differs from the oracle's in its last half bit just above a power of two is one ulp
    # of 2^-10 relative, and max|x| / 127 sits near the top of its binade, where that is two ulps)
    got_pool = device_pool.numpy(np.uint8, (capacity, stride))
    want_pool = expected_pool.reshape(capacity, stride)
    for b in range(batch):
        got_q = got_pool[new_slots[b], :elements].view(np.int8).astype(np.int32)
        want_q = want_pool[new_slots[b], :elements].view(np.int8).astype(np.int32)
        assert np.abs(got_q - want_q).max() <= 1
        got_s = got_pool[new_slots[b], elements:].copy().view(np.uint16)
        want_s = want_pool[new_slots[b], elements:].copy().view(np.uint16)
        first = config.layer_elements // 64  # scale groups of the first layer
        assert np.abs(got_s[:first].astype(np.int32) - want_s[:first].astype(np.int32)).max() <= 2
        # a later layer's keys and values carry what the chain before them is allowed: their largest (the scale
        # is it / 127) within the hidden state's own 4e-3
        later_got, later_want = got_s[first:].view(np.float16).astype(np.float64), want_s[first:].view(np.float16).astype(np.float64)
        assert np.all(np.abs(later_got - later_want) <= 4e-3 * later_want)
    untouched = np.setdiff1d(np.arange(capacity), new_slots)
    np.testing.assert_array_equal(got_pool[untouched], want_pool[untouched])


@pytest.mark.parametrize("shape", [dict(hidden=256, q_heads=4, kv_heads=2, mlp=512), dict(hidden=1024, q_heads=16, kv_heads=4, mlp=2048),
                                   dict(hidden=128, q_heads=2, kv_heads=2, mlp=1536), dict(hidden=704, q_heads=8, kv_heads=1, mlp=960)],
                         ids=["256x512", "1024x2048", "128x1536", "704x960"])
@pytest.mark.parametrize("launches", [6, 5, 4, 3])
def test_decode_step_of_other_models_matches_oracle_chain(runtime, shape, launches):
    """The three launch forms on models other than the benchmark's: other widths, head counts and group
    sizes (one KV head for eight query heads; as many KV heads as query heads), an FFN too wide for
    slices of 32 columns (2048 / 32 = 64 partial sums) and one where they apply at every batch here."""
    from llmopt_amd.decode_step import DecodeConfig, DecodeStep, random_weights
    config = DecodeConfig(layers=2, vocabulary=512, **shape)
    batch, lengths = 3, [90, 7, 140]
    rng = np.random.default_rng(config.hidden + launches)
    weights = random_weights(config, rng)
    total = sum(lengths)
    capacity = total + batch + 2
    order = rng.permutation(capacity).astype(np.uint32)
    slots, new_slots = order[:total], order[total:total + batch]
    offsets = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.uint32)
    stride, elements = config.token_stride, config.token_elements
    pool = np.zeros((capacity, stride), dtype=np.uint8)
    pool[:, :elements] = np.clip(np.rint(rng.standard_normal((capacity, elements)) * 38), -127, 127) \
        .astype(np.int8).view(np.uint8)
    pool[:, elements:] = rng.uniform(0.02, 0.035, (capacity, elements // 64)).astype(np.float16) \
        .view(np.uint8).reshape(capacity, -1)
    pool = pool.reshape(-1)
    tokens = rng.integers(0, config.vocabulary, batch)
    device_pool = runtime.buffer_of_bytes(pool)
    step = DecodeStep(runtime, config, weights, batch, device_pool, runtime.buffer_of_bytes(slots), offsets, lengths,
                      new_slots, lengths, fused=launches < 5, projecting=launches == 3, fused_qkv=launches == 5)
    assert len(step.dispatches) == {6: 14, 5: 12, 4: 11, 3: 10}[launches]
    got_tokens = step.run(tokens)
    got_hidden = step.work["x"][0].numpy(np.float16, (batch, config.hidden))
    hidden, logits, expected_pool = oracle_step(config, weights, pool, slots, offsets, lengths, new_slots, lengths, tokens)
    assert_close_to_oracle(got_hidden, hidden, "hidden state after the last layer", rel_l2_tol=4e-3)
    rms = float(np.sqrt(np.mean(logits.astype(np.float64) ** 2)))
    for b in range(batch):
        assert float(logits[b, got_tokens[b]]) >= float(logits[b].max()) - 2e-2 * rms
    got_pool = device_pool.numpy(np.uint8, (capacity, stride))
    want_pool = expected_pool.reshape(capacity, stride)
    difference = got_pool[new_slots, :elements].view(np.int8).astype(np.int32) - \
        want_pool[new_slots, :elements].view(np.int8).astype(np.int32)
    assert np.abs(difference).max() <= 1
    untouched = np.setdiff1d(np.arange(capacity), new_slots)
    np.testing.assert_array_equal(got_pool[untouched], want_pool[untouched])


@pytest.mark.parametrize("batch", [4, 8])
def test_batched_decode_continues_from_prefilled_sequences(runtime, batch):
    """Every sequence of a batch is prefilled by its own PrefillStep into one shared pool; one
    DecodeStep over all of them then continues, against the oracle's decode chain over the pool
    bytes the prefills left."""
    from llmopt_amd.decode_step import DecodeConfig, DecodeStep, random_weights
    from llmopt_amd.prefill_step import PrefillStep
    rng = np.random.default_rng(300 + batch)
    config = DecodeConfig(layers=2, vocabulary=1000)
    weights = random_weights(config, rng)
    lengths = [int(v) for v in rng.integers(2, 90, size=batch)]
    capacity = sum(lengths) + batch + 2
    order = rng.permutation(capacity).astype(np.uint32)
    # a sequence's slot-table entries: its prompt's slots, then the slot its first decoded token takes
    offsets = np.concatenate([[0], np.cumsum([n + 1 for n in lengths])[:-1]]).astype(np.uint32)
    stride = config.token_stride
    device_pool = runtime.buffer_of_bytes(rng.integers(0, 256, size=capacity * stride, dtype=np.uint8))
    device_slots = runtime.buffer_of_bytes(order)
    first_tokens, device_weights = [], None
    for b in range(batch):
        table = device_slots.view(int(offsets[b]) * 4, (lengths[b] + 1) * 4)
        step = PrefillStep(runtime, config, weights, lengths[b], device_pool, table, device_weights=device_weights)
        device_weights = step.device
        first_tokens.append(step.run(rng.integers(0, config.vocabulary, lengths[b])))
    new_slots = order[offsets + np.asarray(lengths, dtype=np.uint32)]
    pool_after_prefill = device_pool.numpy(np.uint8, (capacity * stride,)).copy()
    decode = DecodeStep(runtime, config, weights, batch, device_pool, device_slots, offsets, lengths, new_slots,
                        lengths)
    got_tokens = decode.run(first_tokens)
    hidden, logits, _ = oracle_step(config, weights, pool_after_prefill, order, offsets, lengths, new_slots, lengths,
                                    first_tokens)
    # real keys and values in the pool: the attention output is as large as the residual stream, so
    # the per-kernel half roundings are not diluted as with the synthetic pool above (the same bound
    # as the single-sequence continuation in tests/test_gpu_prefill_step.py)
    assert_close_to_oracle(decode.work["x"][0].numpy(np.float16, (batch, config.hidden)), hidden,
                           "batched decode step after the prefills", rel_l2_tol=2e-2)
    rms = float(np.sqrt(np.mean(logits.astype(np.float64) ** 2)))
    for b in range(batch):
        assert float(logits[b, got_tokens[b]]) >= float(logits[b].max()) - 2e-2 * rms
