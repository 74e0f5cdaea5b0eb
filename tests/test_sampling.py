"""Host-side token selection (lib/sampling.ml, native/ocaml_metal_stubs.m:2565-2765): the library's
`llmopt_hip_f16_argmax` / `llmopt_hip_sample_f16` behind `llmopt_amd.sampling`, against the
reference's own sampling test, closed forms and the Python restatement in oracle/.  No GPU."""
import math
import struct

import numpy as np
import pytest

from llmopt_amd import sampling
from llmopt_amd.sampling import Float16Logits, Greedy, Params, SamplingError, sample
from oracle import sampling_oracle


def f16_bytes(values) -> bytes:
    return np.asarray(values, dtype=np.float16).tobytes()


def reference_logits() -> bytes:
    """test/test_generation.ml:462-470: 64 logits, token 10 = 0x4900, token 20 = 0x4880, others 1.0."""
    bits = [0x4900 if i == 10 else 0x4880 if i == 20 else 0x3C00 for i in range(64)]
    return struct.pack("<64H", *bits)


def test_reference_sampling_vectors():
    logits = reference_logits()
    assert sample(Params.greedy(), 64, logits) == 10
    assert sample(Params.greedy(), 64, logits, suppress_token_ids=[10]) == 20
    assert Greedy.f16_all_rows(64, logits, suppress_token_ids=[10]) == [20]
    assert Float16Logits.top(1, 64, logits, suppress_token_ids=[10]) == [(20, 9.0)]
    custom = Params.create(temperature=0.7, top_k=40, top_p=0.9, min_p=0.05, seed=42)
    assert (custom.temperature, custom.top_k, custom.top_p, custom.min_p, custom.seed) == (0.7, 40, 0.9, 0.05, 42)
    assert not custom.is_greedy() and Params.greedy().is_greedy()
    first, second = sample(custom, 64, logits), sample(custom, 64, logits)
    assert first == second and first in (10, 20)
    assert first == sampling_oracle.sample_f16(logits, 0.7, 40, 0.9, 0.05, 42)


def test_params_create_clamps_like_the_reference():
    params = Params.create(temperature=-1.0, top_k=-5, top_p=1.5, min_p=-0.2, seed=7)
    assert (params.temperature, params.top_k, params.top_p, params.min_p, params.seed) == (0.0, 0, 1.0, 0.0, 7)
    assert Params.create().is_greedy()  # temperature 0
    assert Params.create(temperature=0.8, top_k=1).is_greedy()
    assert not Params.create(temperature=0.8).is_greedy()


def test_error_strings():
    row = f16_bytes([1.0, 2.0, 3.0])
    with pytest.raises(SamplingError, match="float16 logits vocabulary must be positive"):
        Float16Logits.last_row(0, row)
    with pytest.raises(SamplingError, match=r"float16 logits contain 6 bytes; expected complete 8-byte rows"):
        Float16Logits.last_row(4, row)
    with pytest.raises(SamplingError, match=r"float16 logits contain 0 bytes; expected complete 6-byte rows"):
        Float16Logits.last_row(3, b"")
    with pytest.raises(SamplingError, match=r"suppressed token id 3 is outside vocabulary \[0,3\)"):
        sample(Params.greedy(), 3, row, suppress_token_ids=[3])
    with pytest.raises(SamplingError, match="cannot suppress the complete sampling vocabulary"):
        sample(Params.greedy(), 3, row, suppress_token_ids=[0, 1, 2, 1])
    with pytest.raises(SamplingError, match="float16 logits top count must be positive"):
        Float16Logits.top(0, 3, row)
    with pytest.raises(SamplingError, match="float16 logits contain NaN at token 1"):
        Float16Logits.top(2, 3, f16_bytes([1.0, float("nan"), 0.0]))
    with pytest.raises(SamplingError, match="on-device greedy token must contain 4 bytes; got 8"):
        Greedy.on_device(b"\0" * 8)
    with pytest.raises(SamplingError, match="on-device greedy token rows contain 6 bytes; expected a positive multiple of 4"):
        Greedy.on_device_last(b"\0" * 6)
    with pytest.raises(SamplingError, match="on-device greedy token rows contain 0 bytes"):
        Greedy.on_device_all(b"")


def test_on_device_tokens_and_rows():
    data = struct.pack("<3I", 5, 0xFFFFFFFF, 49151)
    assert Greedy.on_device(data[:4]) == 5
    assert Greedy.on_device_last(data) == 49151
    assert Greedy.on_device_all(data) == [5, 0xFFFFFFFF, 49151]
    rows = f16_bytes([[0.0, 3.0, 3.0], [9.0, -1.0, 2.0]])
    assert Float16Logits.last_row(3, rows) == f16_bytes([9.0, -1.0, 2.0])
    assert Greedy.f16_all_rows(3, rows) == [1, 0]  # a tie goes to the lowest index
    assert Float16Logits.top(3, 3, rows[:6]) == [(1, 3.0), (2, 3.0), (0, 0.0)]
    assert sampling.float16(0x3C00) == 1.0 and sampling.float16(0xFC00) == -math.inf
    assert sampling.float16(0x0001) == 2.0 ** -24 and math.isnan(sampling.float16(0x7E00))


@pytest.mark.parametrize("seed", range(6))
def test_greedy_paths_are_the_first_maximum(seed):
    rng = np.random.default_rng(seed)
    vocabulary = int(rng.integers(1, 3000))
    values = np.round(rng.standard_normal(vocabulary) * 3).astype(np.float16)  # many ties
    if seed == 3:
        values[0] = np.float16("nan")  # a leading NaN is never displaced: index 0 (reference: `ptr[i] > max_val`)
    data = values.tobytes()
    if seed == 3:
        expected = 0
    else:
        expected = int(np.argmax(values.astype(np.float32)))
    assert Greedy.f16_last_row(vocabulary, data) == expected == sampling_oracle.argmax_f16(data)
    assert sample(Params.create(temperature=0.9, top_k=1, seed=5), vocabulary, data) == expected
    assert sample(Params.create(temperature=0.00005, top_k=50, seed=5), vocabulary, data) == expected


def test_generator_known_answers():
    state = [1, 2]
    assert sampling_oracle.xoroshiro128plus(state) == 3
    assert state == [0x1030003, 0x6000000000]
    assert sampling_oracle.xoroshiro128plus(state) == 0x6001030003
    assert sampling_oracle.seed_state(0x9E3779B97F4A7C15 ^ 0) != [0, 0]
    # the first draw is (seed ^ 0x9E37...) + rotl(seed, 31): small seeds all start near 0.618 (the
    # constant over 2^64), seeds spread over 62 bits are uniform
    assert all(abs(float(sampling_oracle.uniform01(sampling_oracle.seed_state(seed))) - 0.6180340) < 1e-5
               for seed in range(1, 50))
    rng = np.random.default_rng(3)
    draws = [float(sampling_oracle.uniform01(sampling_oracle.seed_state(int(seed))))
             for seed in rng.integers(1, 2 ** 62, size=4000)]
    assert 0.0 <= min(draws) and max(draws) <= 1.0
    assert abs(np.mean(draws) - 0.5) < 0.03


CASES = [
    # (vocabulary, temperature, top_k, top_p, min_p)
    (1, 0.7, 0, 1.0, 0.0), (5, 1.0, 0, 1.0, 0.0), (64, 0.7, 40, 0.9, 0.05), (300, 1.3, 2, 1.0, 0.0),
    (1000, 0.5, 256, 0.95, 0.0), (5000, 2.0, 1000, 0.5, 0.01), (777, 0.8, 64, 1.0, 0.3), (4096, 1.0, 0, 0.8, 0.0),
    (50, 10.0, 100, 0.999, 0.0), (2048, 0.3, 8, 0.0, 1.0),
]


@pytest.mark.parametrize("vocabulary,temperature,top_k,top_p,min_p", CASES)
def test_library_matches_the_restatement(vocabulary, temperature, top_k, top_p, min_p):
    """Same token as the Python restatement for 40 seeds per case; coarse logits make ties, which the
    heap must break the reference's way."""
    rng = np.random.default_rng(vocabulary * 7 + top_k)
    for trial in range(40):
        scale = [0.25, 1.0, 4.0][trial % 3]
        values = (np.round(rng.standard_normal(vocabulary) * 2 / scale) * scale).astype(np.float16)
        if trial % 5 == 4:
            values[rng.integers(0, vocabulary)] = np.float16("-inf")
        data = values.tobytes()
        seed = int(rng.integers(1, 2 ** 62))
        params = Params.create(temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p, seed=seed)
        expected = sampling_oracle.sample_f16(data, params.temperature, params.top_k, params.top_p, params.min_p, seed)
        assert sample(params, vocabulary, data) == expected, (trial, seed)


def test_two_candidates_follow_their_softmax_probabilities():
    values = np.full(500, -20.0, dtype=np.float16)
    values[123], values[321] = 2.0, 1.0
    data = values.tobytes()
    seeds = np.random.default_rng(5).integers(1, 2 ** 62, size=4000)
    draws = [sample(Params.create(temperature=1.0, top_k=2, seed=int(seed)), 500, data) for seed in seeds]
    assert set(draws) == {123, 321}
    expected = 1.0 / (1.0 + math.exp(-1.0))  # P(token 123)
    share = draws.count(123) / len(draws)
    assert abs(share - expected) < 4 * math.sqrt(expected * (1 - expected) / len(draws))


def test_filters_reduce_to_the_best_tokens():
    rng = np.random.default_rng(11)
    values = np.round(rng.standard_normal(900) * 2).astype(np.float16)
    best = np.flatnonzero(values == values.max())
    data = values.tobytes()
    for seed in (int(v) for v in np.random.default_rng(6).integers(1, 2 ** 62, size=60)):
        # top_p below the best token's probability keeps the head of the list only
        assert sample(Params.create(temperature=1.0, top_k=50, top_p=1e-4, seed=seed), 900, data) in best
        # min_p = 1: only tokens as probable as the best one survive
        assert sample(Params.create(temperature=1.0, top_k=50, min_p=1.0, seed=seed), 900, data) in best
    # seed 0 draws from the clock: any kept candidate, i.e. a token at least as good as the 40th best
    # (which of the tokens tied at that value are kept is the heap's business)
    drawn = sample(Params.create(temperature=1.0, top_k=40, seed=0), 900, data)
    assert values[drawn] >= np.sort(values.astype(np.float32))[-40]
