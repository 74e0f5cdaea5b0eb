"""Retained decode plans (llmopt_hip_prebaked_*) and the ring worker over one: several consecutive
tokens through the frozen dispatch array against the same steps launched eagerly, and against the
CPU oracle chain."""
import numpy as np
import pytest

from tests.gpu_util import assert_close_to_oracle
from oracle.chain import decode_chain as oracle_step

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def make_case(rng, config, lengths, room):
    """A pool with every sequence's context, and a slot table with `room` free slots behind each
    sequence's own (the slots its next tokens will take)."""
    batch = len(lengths)
    spans = [length + room for length in lengths]
    capacity = sum(spans) + 3
    order = rng.permutation(capacity).astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(spans)[:-1]]).astype(np.uint32)
    slots = order[:sum(spans)]
    stride, elements = config.token_stride, config.token_elements
    pool = np.zeros((capacity, stride), dtype=np.uint8)
    pool[:, :elements] = np.clip(np.rint(rng.standard_normal((capacity, elements)) * 38), -127, 127) \
        .astype(np.int8).view(np.uint8)
    pool[:, elements:] = rng.uniform(0.02, 0.035, (capacity, elements // 64)).astype(np.float16) \
        .view(np.uint8).reshape(capacity, -1)
    new_slots = slots[offsets + np.asarray(lengths, dtype=np.uint32)]
    return pool.reshape(-1), slots, offsets, new_slots, capacity, batch


def build_step(runtime, config, weights, case, lengths, room, **kwargs):
    from llmopt_amd.decode_step import DecodeStep
    pool, slots, offsets, new_slots, capacity, batch = case
    device_pool = runtime.buffer_of_bytes(pool)
    step = DecodeStep(runtime, config, weights, batch, device_pool, runtime.buffer_of_bytes(slots), offsets, lengths,
                      new_slots, lengths, max_context=max(lengths) + room, slots_host=slots, **kwargs)
    return step, device_pool


def test_prebaked_plan_advances_a_batch_like_eager_steps(runtime):
    """The decode step's own dispatch list (batched extension entries: lengths, slots and rotary
    rows in device buffers) frozen into a plan: five tokens through llmopt_hip_prebaked_execute
    leave the same tokens, hidden states and pool bytes as five eager steps - bit for bit, the
    kernels and their launch geometry being the same."""
    from llmopt_amd.decode_step import DecodeConfig, random_weights
    from llmopt_amd.native import Prebaked
    rng = np.random.default_rng(91)
    config = DecodeConfig(layers=2, vocabulary=1000)
    weights = random_weights(config, rng)
    lengths, room, steps = [64, 5, 300], 8, 5
    case = make_case(rng, config, lengths, room)
    eager, eager_pool = build_step(runtime, config, weights, case, lengths, room)
    frozen, frozen_pool = build_step(runtime, config, weights, case, lengths, room)
    plan = Prebaked(runtime, frozen.dispatches, frozen.tokens, frozen.token_ids)
    assert plan.single_submission
    tokens = rng.integers(0, config.vocabulary, len(lengths))
    plan_tokens = tokens.copy()
    for index in range(steps):
        print(f"prebaked batch step {index}", flush=True)
        want = eager.run(tokens)
        frozen.tokens.write(np.asarray(plan_tokens, dtype=np.int64))
        first = plan.execute(int(plan_tokens[0]), int(frozen.host_lengths[0]))
        got = frozen.token_ids.numpy(np.uint32, (len(lengths),))
        assert first == int(got[0])
        np.testing.assert_array_equal(got, want, err_msg=f"tokens of step {index}")
        np.testing.assert_array_equal(frozen.work["x"][0].numpy(np.uint16), eager.work["x"][0].numpy(np.uint16),
                                      err_msg=f"hidden state of step {index}")
        np.testing.assert_array_equal(frozen_pool.numpy(np.uint8), eager_pool.numpy(np.uint8),
                                      err_msg=f"pool after step {index}")
        tokens, plan_tokens = want.astype(np.int64), got.astype(np.int64)
        eager.advance()
        frozen.advance()
    # the new tokens did land: every step changed exactly one slot per sequence
    changed = np.flatnonzero((frozen_pool.numpy(np.uint8).reshape(case[4], -1) !=
                              case[0].reshape(case[4], -1)).any(axis=1))
    assert len(changed) == steps * len(lengths)


@pytest.mark.parametrize("first_past", [37, 0])
def test_prebaked_plan_patches_the_reference_attention_entries(runtime, first_past):
    """One sequence through the reference's own kernel names: the plan owns the context length
    (llmopt_hip_prebaked_execute's past_tokens, the reference's patch of parameter byte 12).  Four
    consecutive tokens against the CPU oracle chain and against eager launches with the byte patched
    by the host (those size the attention launch for the context, the plan for the slot table's
    capacity: same results up to the order of float32 sums)."""
    from llmopt_amd.decode_step import DecodeConfig, random_weights
    from llmopt_amd.native import Prebaked
    rng = np.random.default_rng(17 + first_past)
    config = DecodeConfig(layers=2, vocabulary=1000)
    weights = random_weights(config, rng)
    lengths, room, steps = [first_past], 70, 4
    case = make_case(rng, config, lengths, room)
    eager, eager_pool = build_step(runtime, config, weights, case, lengths, room, reference_entries=True)
    frozen, frozen_pool = build_step(runtime, config, weights, case, lengths, room, reference_entries=True)
    plan = Prebaked(runtime, frozen.dispatches, frozen.tokens, frozen.token_ids)
    assert plan.single_submission
    pool_host, slots, offsets, _, capacity, _ = case
    oracle_pool = pool_host.copy()
    token = int(rng.integers(0, config.vocabulary))
    for index in range(steps):
        past = first_past + index
        print(f"prebaked reference-entry step {index} past {past}", flush=True)
        want_token = int(eager.run([token])[0])
        got_token = plan.execute(token, past)
        got_hidden = frozen.work["x"][0].numpy(np.float16, (1, config.hidden))
        hidden, logits, oracle_pool = oracle_step(config, weights, oracle_pool, slots, offsets, [past],
                                                  [int(slots[past])], [past], [token])
        assert_close_to_oracle(got_hidden, hidden, f"hidden state of step {index}", rel_l2_tol=4e-3)
        assert_close_to_oracle(got_hidden, eager.work["x"][0].numpy(np.float16, (1, config.hidden)),
                               f"plan against eager, step {index}", rel_l2_tol=2e-3)
        rms = float(np.sqrt(np.mean(logits.astype(np.float64) ** 2)))
        assert float(logits[0, got_token]) >= float(logits[0].max()) - 2e-2 * rms
        assert got_token == want_token
        stride, elements = config.token_stride, config.token_elements
        got_slot = frozen_pool.numpy(np.uint8).reshape(capacity, stride)[int(slots[past])]
        want_slot = oracle_pool.reshape(capacity, stride)[int(slots[past])]
        assert np.abs(got_slot[:elements].view(np.int8).astype(np.int32) -
                      want_slot[:elements].view(np.int8).astype(np.int32)).max() <= 1
        # the oracle continues from the GPU's own cache contents, so that one quantum of difference
        # in a stored key does not grow into a different continuation
        oracle_pool = frozen_pool.numpy(np.uint8)
        frozen_pool.copy_to(eager_pool)
        token = got_token
        eager.advance()
        frozen.advance()
    with pytest.raises(Exception) as error:
        plan.execute(token, first_past + room + 1000)
    assert "context tokens" in str(error.value)


def markov_plan(runtime, rng, vocabulary=512, hidden=576):
    """token -> embedding row -> LM-head argmax: a plan whose output token is a function of its input."""
    from llmopt_amd.decode_step import random_w4, u32s
    import struct
    embedding = (rng.standard_normal((vocabulary, hidden)) * 0.5).astype(np.float16)
    norm = rng.uniform(0.5, 1.5, hidden).astype(np.float16)
    head_w, head_s = random_w4(rng, vocabulary, hidden)
    b = runtime.buffer_of_bytes
    tokens, token_ids = b(np.zeros(1, dtype=np.int64)), b(np.zeros(1, dtype=np.uint32))
    x = runtime.create_buffer(hidden * 2)
    dispatches = [
        ("llmopt_embedding_f16", [tokens, b(embedding), x], u32s(1, vocabulary, hidden), (((hidden + 255) // 256) * 256, 1, 1),
         (256, 1, 1)),
        ("llmopt_w4a16_lm_head_argmax_f16", [x, b(norm), b(head_w), b(head_s), token_ids],
         u32s(1, vocabulary, hidden) + struct.pack("<f", 1e-5), (256, 1, 1), (256, 1, 1)),
    ]
    return dispatches, tokens, token_ids


@pytest.mark.parametrize("depth", ["1", "2"])
def test_ring_worker_runs_chained_steps_of_a_plan(runtime, depth, monkeypatch):
    from llmopt_amd.native import Prebaked, Ring
    monkeypatch.setenv("LLMOPT_QUEUE_DEPTH", depth)
    rng = np.random.default_rng(5)
    dispatches, tokens, token_ids = markov_plan(runtime, rng)
    # what the chain must produce: the same plan, one token at a time
    plan = Prebaked(runtime, dispatches, tokens, token_ids)
    expected, token = [], 5
    for _ in range(12):
        token = plan.execute(token, 0)
        expected.append(token)
    assert len(set(expected)) > 3  # not a fixed point: the chain really feeds tokens back
    del plan
    ring = Ring()
    ring.start_worker(runtime, dispatches, tokens, token_ids)
    assert ring.submit(100, 5, 0)
    for request in range(1, 12):
        assert ring.submit(100 + request, -1, request)  # chained: input = the previous output, on the GPU
    done = [ring.wait_completion() for _ in range(12)]
    assert [d[0] for d in done] == [100 + r for r in range(12)]
    assert [d[1] for d in done] == expected
    assert all(d[2] == 0 for d in done)
    # an explicit token restarts the chain
    ring.submit(7, 5, 0)
    assert ring.wait_completion() == (7, expected[0], 0)
    ring.destroy()


def test_profile_breakdown_replay_prints_gpu_time_by_kernel(runtime, monkeypatch, capfd):
    """LLMOPT_PROFILE_BREAKDOWN (native/ocaml_metal_stubs.m:2270-2347): the records run one at a
    time, the step's result is unchanged, and the table of GPU time by kernel name goes to stderr."""
    from llmopt_amd.native import Prebaked
    rng = np.random.default_rng(5)
    dispatches, tokens, token_ids = markov_plan(runtime, rng)
    plan = Prebaked(runtime, dispatches, tokens, token_ids)
    want = plan.execute(5, 3)
    capfd.readouterr()
    monkeypatch.setenv("LLMOPT_PROFILE_BREAKDOWN", "1")
    got = plan.execute(5, 3)
    report = capfd.readouterr().err
    assert got == want
    assert "DECODE KERNEL BREAKDOWN (past_tokens=3)" in report
    rows = {line.split("|")[0].strip(): line for line in report.splitlines() if "|" in line}
    assert set(rows) >= {"llmopt_embedding_f16", "llmopt_w4a16_lm_head_argmax_f16", "TOTAL DISPATCHES"}
    assert rows["llmopt_embedding_f16"].split("|")[1].strip() == "1"
    assert float(rows["TOTAL DISPATCHES"].split("|")[2]) > 0.0


def test_nan_check_replay_names_the_first_record_that_produces_a_nan(runtime, monkeypatch, capfd):
    """LLMOPT_DEBUG_NAN_CHECK (native/ocaml_metal_stubs.m:2136-2268).  The embedding table holds a
    NaN in row 7 only: token 5 passes, token 7 is reported at record 0, buffer 2 (the row it wrote;
    the table itself held its NaN before and is not blamed).  A step with no context is only
    checked under LLMOPT_CHECK_PREFILL, as in the reference."""
    from llmopt_amd.native import Prebaked
    rng = np.random.default_rng(5)
    dispatches, tokens, token_ids = markov_plan(runtime, rng)
    table = dispatches[0][1][1]
    poisoned = table.numpy(np.uint16).copy().reshape(512, 576)
    poisoned[7, 100] = 0x7E00
    table.write(poisoned)
    plan = Prebaked(runtime, dispatches, tokens, token_ids)
    monkeypatch.setenv("LLMOPT_DEBUG_NAN_CHECK", "1")
    plan.execute(5, 3)
    assert "Starting check across 2 records (past_tokens=3)" in capfd.readouterr().err
    with pytest.raises(Exception) as error:
        plan.execute(7, 3)
    assert "record 0 'llmopt_embedding_f16' produced the first NaN, in buffer 2" in str(error.value)
    report = capfd.readouterr().err
    assert "FIRST NaN PRODUCED AT RECORD 0" in report and "kernel: 'llmopt_embedding_f16'" in report
    # past_tokens = 0: not checked, the step runs as usual (the NaN row flows into the argmax)
    plan.execute(7, 0)
    assert "DEBUG_NAN_CHECK" not in capfd.readouterr().err
    monkeypatch.setenv("LLMOPT_CHECK_PREFILL", "1")
    plan.execute(5, 0)  # a clean row again (a buffer that held a NaN before a record is not blamed on it)
    with pytest.raises(Exception):
        plan.execute(7, 0)


def test_plan_writes_the_checkpoint_slot_of_each_step(runtime):
    """llmopt_hip_prebaked_execute's checkpoint argument: the llmopt_cache_pack_checkpoint_q8_simd
    records of a plan write the slot the step names (native/ocaml_metal_stubs.m:2186-2188 rewrites
    byte 0 of their parameter block), the other checkpoint entry keeps the slot it was created with."""
    from llmopt_amd.native import Prebaked
    from tests.gpu_util import u32s
    rng = np.random.default_rng(23)
    layers, layer_elements, slots = 2, 4 * 64, 5
    elements = layers * layer_elements
    stride = elements + 2 * (elements // 64)
    state = (rng.standard_normal(layer_elements) * 2).astype(np.float16)
    start = np.zeros(slots * stride, dtype=np.uint8)
    pool = runtime.buffer_of_bytes(start)
    source = runtime.buffer_of_bytes(state)
    token = runtime.buffer_of_bytes(np.zeros(1, dtype=np.int64))
    output = runtime.buffer_of_bytes(np.zeros(1, dtype=np.int32))
    params = lambda slot, layer: u32s(slot, layer, layer_elements, 64, elements, elements // 64, stride)
    grid = (layer_elements // 64 * 32, 1, 1)
    plan = Prebaked(runtime, [("llmopt_cache_pack_checkpoint_q8_simd", [source, pool], params(0, 0), grid, (256, 1, 1)),
                              ("llmopt_cache_pack_checkpoint_q8", [source, pool], params(4, 1), grid, (256, 1, 1))],
                    token, output)
    assert plan.single_submission
    for slot in (3, 1):
        plan.execute(0, 0, checkpoint=slot)
    got = pool.numpy(np.uint8, (slots, stride))
    written = got[:, :layer_elements].any(axis=1)
    np.testing.assert_array_equal(written, [False, True, False, True, False])   # layer 0: the slots of the two steps
    np.testing.assert_array_equal(got[3, :layer_elements], got[1, :layer_elements])
    assert got[4, layer_elements:elements].any() and not got[:4, layer_elements:elements].any()  # layer 1: slot 4 only
    # a slot the pool has no room for: refused on the host, nothing queued (the launch itself, reading
    # the slot from device memory, could only clamp it)
    from llmopt_amd.native import LlmoptError
    with pytest.raises(LlmoptError, match=r"checkpoints 0\.\.4, step asks for 5") as error:
        plan.execute(0, 0, checkpoint=slots)
    assert error.value.code == -2
    np.testing.assert_array_equal(pool.numpy(np.uint8, (slots, stride)), got)
    del plan


def test_plan_is_captured_again_after_the_kernel_workspace_moved(runtime):
    """A plan's graph holds the address of the context's kernel workspace (the attention launches'
    partial results).  An eager launch that needs more grows the workspace - the old block is freed -
    and the next step of the plan must capture its records again: tokens, hidden state and pool equal
    to eager steps bit for bit, before and after."""
    import math
    import struct
    from llmopt_amd.decode_step import DecodeConfig, random_weights
    from llmopt_amd.native import Prebaked, Runtime
    own = Runtime()  # a context of its own: what other tests left in the shared one's workspace is not known
    try:
        rng = np.random.default_rng(77)
        config = DecodeConfig(layers=2, vocabulary=1000)
        weights = random_weights(config, rng)
        lengths, room = [120, 70], 6
        case = make_case(rng, config, lengths, room)
        eager, eager_pool = build_step(own, config, weights, case, lengths, room)
        frozen, frozen_pool = build_step(own, config, weights, case, lengths, room)
        plan = Prebaked(own, frozen.dispatches, frozen.tokens, frozen.token_ids)
        assert plan.single_submission
        tokens = rng.integers(0, config.vocabulary, len(lengths))

        def both_step(label):
            nonlocal tokens
            want = eager.run(tokens)
            frozen.tokens.write(np.asarray(tokens, dtype=np.int64))
            plan.execute(int(tokens[0]), int(frozen.host_lengths[0]))
            np.testing.assert_array_equal(frozen.token_ids.numpy(np.uint32, (len(lengths),)), want, err_msg=label)
            np.testing.assert_array_equal(frozen.work["x"][0].numpy(np.uint16), eager.work["x"][0].numpy(np.uint16),
                                          err_msg=label)
            np.testing.assert_array_equal(frozen_pool.numpy(np.uint8), eager_pool.numpy(np.uint8), err_msg=label)
            tokens = want.astype(np.int64)
            eager.advance()
            frozen.advance()

        both_step("before the workspace moved")
        # 64 sequences of 8 KV heads of 128: about 18 MB of partial results, many times what the two
        # short sequences of the plan asked for
        batch, q_heads, kv_heads, dim, context = 64, 32, 8, 128, 80
        elements = 2 * kv_heads * dim
        stride = elements + 2 * (elements // 64)
        big_pool = own.buffer_of_bytes(rng.integers(0, 256, size=context * stride, dtype=np.uint8))
        big_slots = own.buffer_of_bytes(np.tile(np.arange(context, dtype=np.uint32), batch))
        rows = lambda heads: own.buffer_of_bytes(rng.standard_normal(batch * heads * dim).astype(np.float16))
        out = own.create_buffer(batch * q_heads * dim * 2)
        own.dispatch("llmopt_attention_q8_paged_batched",
                     [rows(q_heads), rows(kv_heads), rows(kv_heads), big_pool, big_slots, big_slots, out,
                      own.buffer_of_bytes(np.full(batch, context, dtype=np.uint32)),
                      own.buffer_of_bytes(np.arange(batch, dtype=np.uint32) * context)],
                     struct.pack("<12IfIII", batch, q_heads, kv_heads, 0, dim, 0, 0, elements, 0, kv_heads * dim, 64, stride,
                                 1.0 / math.sqrt(dim), 1, 0, 0) + struct.pack("<I", context),
                     grid=(256, 1, 1), group=(256, 1, 1))
        own.synchronize()
        for index in range(2):
            both_step(f"step {index} after the workspace moved")
        del plan
    finally:
        own.close()


def test_plan_with_a_masked_attention_is_launched_from_the_host(runtime):
    """A masked paged attention cannot read its context length from device memory (the mask's row
    length follows it): such a plan is not one graph but the records launched one by one, the length
    patched into parameter byte 12 on the host - as the reference does for every plan.  Two steps at
    different context lengths against the oracle."""
    import math
    import oracle
    from oracle import PagedParams
    from llmopt_amd.native import Prebaked
    from tests.test_gpu_q8 import build_pool, paged_params_bytes
    rng = np.random.default_rng(5)
    b, h, kvh, dim, capacity = 1, 4, 2, 64, 90
    pool, slots, _, te, stride, ko, vo = build_pool(rng, kvh, dim, [capacity])
    query = rng.standard_normal((b, h, 1, dim)).astype(np.float16)
    ck = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    cv = rng.standard_normal((b, kvh, 1, dim)).astype(np.float16)
    params = lambda past: PagedParams(batches=b, query_heads=h, kv_heads=kvh, past_length=past, head_dim=dim,
                                      mask_batches=1, mask_heads=1, token_elements=te, key_offset=ko, value_offset=vo,
                                      group_size=64, token_stride=stride, scale=1.0 / math.sqrt(dim), query_length=1,
                                      mask_dtype=1, window=0)
    mask_buffer = runtime.create_buffer(capacity + 1)
    out = runtime.buffer_of_bytes(np.full((b, 1, h, dim), np.nan, dtype=np.float16))
    slot_buffer = runtime.buffer_of_bytes(slots)
    token = runtime.buffer_of_bytes(np.zeros(1, dtype=np.int64))
    output = runtime.buffer_of_bytes(np.zeros(1, dtype=np.int32))
    plan = Prebaked(runtime, [("llmopt_attention_q8_paged_simd_generic",
                               [runtime.buffer_of_bytes(query), runtime.buffer_of_bytes(ck), runtime.buffer_of_bytes(cv),
                                runtime.buffer_of_bytes(pool), slot_buffer, mask_buffer, out],
                               paged_params_bytes(params(0)), (256, 1, 1), (256, 1, 1))], token, output)
    assert not plan.single_submission
    for past in (70, 33):
        mask = (rng.random((1, 1, 1, past + 1)) > 0.3).astype(np.uint8)
        mask[..., past] = 1
        mask_buffer.write(np.concatenate([mask.reshape(-1), np.zeros(capacity - past, dtype=np.uint8)]))
        plan.execute(0, past)
        expected = oracle.paged_attention_q8(query, ck, cv, pool, slots[:past], mask, params(past))
        assert_close_to_oracle(out.numpy(np.float16, (b, 1, h, dim)), expected, f"masked plan at {past} tokens")
    del plan
