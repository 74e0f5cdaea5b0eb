"""The ring queue (submission / completion queues with one worker thread) over a host step
function: ordering, chaining, capacity, polling and failure status - no GPU involved.
Mirrors how lib/metal_native.ml:404-437 drives caml_llmopt_ring_*."""
import os
import threading
import time

import pytest

from llmopt_amd.native import LlmoptError, Ring


def drain(ring, count):
    return [ring.wait_completion() for _ in range(count)]


@pytest.mark.parametrize("depth", ["1", "2"])
def test_completions_come_back_in_submission_order(depth, monkeypatch):
    monkeypatch.setenv("LLMOPT_QUEUE_DEPTH", depth)
    seen = []

    def step(token, past_tokens):
        seen.append((token, past_tokens, threading.get_ident()))
        return token * 3 + past_tokens

    ring = Ring()
    ring.start_worker_with(step)
    for request in range(40):
        assert ring.submit(request_id=1000 + request, token=request, past_tokens=7 + request)
    done = drain(ring, 40)
    assert [d[0] for d in done] == [1000 + r for r in range(40)]
    assert [d[1] for d in done] == [r * 3 + 7 + r for r in range(40)]
    assert all(d[2] == 0 for d in done)
    assert [s[:2] for s in seen] == [(r, 7 + r) for r in range(40)]
    assert len({s[2] for s in seen}) == 1 and seen[0][2] != threading.get_ident()  # one worker thread, not ours
    assert ring.poll_completion() is None
    ring.destroy()


def test_negative_token_chains_the_previous_result():
    ring = Ring()
    ring.start_worker_with(lambda token, past: token + 1)
    ring.submit(1, 10, 0)
    for request in range(2, 6):
        ring.submit(request, -1, request)
    assert [d[1] for d in drain(ring, 5)] == [11, 12, 13, 14, 15]
    ring.destroy()


def test_queue_holds_256_submissions():
    ring = Ring()  # no worker: nothing is taken out
    for request in range(256):
        assert ring.submit(request, request, 0)
    assert not ring.submit(256, 256, 0)
    assert ring.poll_completion() is None
    ring.start_worker_with(lambda token, past: token)
    assert [d[0] for d in drain(ring, 256)] == list(range(256))
    assert ring.submit(256, 5, 0)
    assert ring.wait_completion() == (256, 5, 0)
    ring.destroy()


def test_poll_does_not_block_and_sees_a_finished_step():
    release = threading.Event()

    def step(token, past):
        release.wait(5)
        return 42

    ring = Ring()
    ring.start_worker_with(step)
    ring.submit(9, 0, 0)
    assert ring.poll_completion() is None  # the step is still running
    release.set()
    deadline = time.time() + 5
    found = None
    while found is None and time.time() < deadline:
        found = ring.poll_completion()
    assert found == (9, 42, 0)
    ring.destroy()


def test_failed_step_reports_status_one_and_the_queue_goes_on():
    def step(token, past):
        if token == 2:
            raise RuntimeError("step failed")
        return token

    ring = Ring()
    ring.start_worker_with(step)
    for request in range(4):
        ring.submit(request, request, 0)
    assert [(d[0], d[2]) for d in drain(ring, 4)] == [(0, 0), (1, 0), (2, 1), (3, 0)]
    ring.destroy()


def test_stop_flag_ends_the_worker():
    ring = Ring()
    ring.start_worker_with(lambda token, past: token)
    ring.submit(1, 1, 0)
    assert ring.wait_completion() == (1, 1, 0)
    ring.submit(2, 0, 0, flags=2)  # the worker leaves without a completion
    time.sleep(0.05)
    ring.submit(3, 3, 0)           # nobody takes it
    time.sleep(0.05)
    assert ring.poll_completion() is None
    ring.destroy()


def test_worker_cannot_start_twice():
    ring = Ring()
    ring.start_worker_with(lambda token, past: token)
    with pytest.raises(LlmoptError):
        ring.start_worker_with(lambda token, past: token)
    ring.destroy()
