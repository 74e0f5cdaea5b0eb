"""CPU restatement of the reference's host-side sampler (test infrastructure only: tests import
this, the shipped library never does).

Follows caml_llmopt_f16_argmax and caml_llmopt_sample_f16_native
(native/ocaml_metal_stubs.m:2565-2765) step by step in numpy float32 scalars:
greedy shortcut (:2645-2656), bounded min-heap top-k (:2581-2612, :2658-2691),
exp((logit - best) / temperature) weights (:2693-2704), min-p (:2706-2726), top-p (:2728-2745),
xoroshiro128+ draw (:2614-2627, :2747-2763).

Pinned by tests/test_sampling.py: the reference's own sampling test (test/test_generation.ml:462-500:
64 logits with token 10 at 10.0 and token 20 at 9.0 - greedy 10, with 10 suppressed 20, seeded
stochastic choice repeatable and in {10, 20}); top_k = 1 and temperature <= 1e-4 reduce to the first
maximum; two candidates drawn over many seeds follow their softmax probabilities; top_p below the
best probability and min_p = 1 leave only the best (tied) tokens; the generator's first outputs from state (1, 2) against values worked out by
hand (3, then 0x6001030003), which fixes its rotations and shift.
"""
from __future__ import annotations

import numpy as np

MASK = (1 << 64) - 1
F32 = np.float32


def f16_row(data: bytes) -> np.ndarray:
    return np.frombuffer(data, dtype="<f2")


def argmax_f16(data: bytes) -> int:
    """First maximum in IEEE comparison order; a NaN never replaces the running best."""
    values = f16_row(data).astype(np.float32)
    best = 0
    for index in range(1, len(values)):
        if values[index] > values[best]:
            best = index
    return best


def xoroshiro128plus(state: list[int]) -> int:
    s0, s1 = state
    result = (s0 + s1) & MASK
    s1 ^= s0
    state[0] = (((s0 << 24) | (s0 >> 40)) & MASK) ^ s1 ^ ((s1 << 16) & MASK)
    state[1] = ((s1 << 37) | (s1 >> 27)) & MASK
    return result


def seed_state(seed: int) -> list[int]:
    seed &= MASK
    state = [seed ^ 0x9E3779B97F4A7C15, ((seed << 31) | (seed >> 33)) & MASK]
    if state == [0, 0]:
        state = [1, 2]
    return state


def uniform01(state: list[int]) -> np.float32:
    return F32(F32(xoroshiro128plus(state) >> 11) * F32(1.0 / 9007199254740992.0))


def _sift_down(heap: list, size: int, index: int) -> None:
    while True:
        smallest = index
        left, right = 2 * index + 1, 2 * index + 2
        if left < size and heap[left][1] < heap[smallest][1]:
            smallest = left
        if right < size and heap[right][1] < heap[smallest][1]:
            smallest = right
        if smallest == index:
            return
        heap[index], heap[smallest] = heap[smallest], heap[index]
        index = smallest


def _sift_up(heap: list, index: int) -> None:
    while index > 0:
        parent = (index - 1) // 2
        if heap[index][1] < heap[parent][1]:
            heap[index], heap[parent] = heap[parent], heap[index]
            index = parent
        else:
            return


def ranked_candidates(values: np.ndarray, top_k: int) -> list[tuple[int, np.float32]]:
    keep = 64
    if 0 < top_k <= 256:
        keep = top_k
    elif top_k > 256:
        keep = 256
    heap: list = []
    for token, value in enumerate(values):
        if len(heap) < keep:
            heap.append((token, value))
            _sift_up(heap, len(heap) - 1)
        elif value > heap[0][1]:
            heap[0] = (token, value)
            _sift_down(heap, keep, 0)
    ordered = [None] * len(heap)
    size = len(heap)
    for index in range(len(ordered) - 1, -1, -1):
        ordered[index] = heap[0]
        heap[0] = heap[size - 1]
        size -= 1
        _sift_down(heap, size, 0)
    return ordered


def sample_f16(data: bytes, temperature: float, top_k: int, top_p: float, min_p: float, seed: int) -> int:
    values = f16_row(data).astype(np.float32)
    if len(values) == 0:
        return 0
    temp, nucleus, floor_ratio = F32(temperature), F32(top_p), F32(min_p)
    if temp <= F32(0.0001) or top_k == 1:
        return argmax_f16(data)
    ranked = ranked_candidates(values, top_k)
    best = ranked[0][1]
    inverse = F32(F32(1.0) / temp)
    weights = []
    total = F32(0.0)
    with np.errstate(over="ignore", invalid="ignore"):
        for _, logit in ranked:
            weight = F32(np.exp(F32(F32(logit - best) * inverse)))
            weights.append(weight)
            total = F32(total + weight)
        live = len(ranked)
        if floor_ratio > 0 and total > 0:
            threshold = F32(F32(weights[0] / total) * floor_ratio)
            kept_total, kept = F32(0.0), 0
            for weight in weights:
                if F32(weight / total) >= threshold:
                    kept_total = F32(kept_total + weight)
                    kept += 1
                else:
                    break
            if kept > 0:
                live, total = kept, kept_total
        if 0 < nucleus < 1 and total > 0:
            cumulative, kept_total, cut = F32(0.0), F32(0.0), live
            for index in range(live):
                cumulative = F32(cumulative + F32(weights[index] / total))
                kept_total = F32(kept_total + weights[index])
                if cumulative >= nucleus:
                    cut = index + 1
                    break
            live, total = cut, kept_total
        if seed == 0:
            raise ValueError("seed 0 draws from the clock: not reproducible")
        state = seed_state(seed)
        target = F32(uniform01(state) * total)
        reached = F32(0.0)
        for index in range(live):
            reached = F32(reached + weights[index])
            if reached >= target:
                return int(ranked[index][0])
    return int(ranked[0][0])
