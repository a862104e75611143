"""Queue discipline of BatchedComputeKernel (reference: compute/kernel.hh:56-170): every pushed
state comes out exactly once, in push order, processed by the model with the contexts of its
rows, and the eventfd counts the finished states.  Host only: the model is a stand-in that
advances tokens."""
import time

import numpy as np
import pytest

from glinthawk_amd import wire
from glinthawk_amd._lib import GlintError
from glinthawk_amd.kernel import ComputeKernel

DIM, KV = wire.HostState.DIM, wire.HostState.KV_DIM


def make_state(rng, state_id, batch, ctx_pool):
    p = wire.new_prompts(batch)
    p["active"] = rng.integers(0, 4, batch) > 0
    p["context_id"] = rng.choice(ctx_pool, batch, replace=False)
    p["token"] = rng.integers(0, 32000, batch)
    p["token_pos"] = rng.integers(0, 10, batch)
    p["kv_tier"] = 0
    meta = dict(id=state_id, dtype=0, next_layer=0, next_stage=0)
    acts = rng.standard_normal((batch, DIM)).astype(np.float16)
    return wire.pack_state(meta, p, activations=acts), p, acts


def drain(kernel, n, timeout_s=30.0):
    out, events = [], 0
    deadline = time.time() + timeout_s
    while len(out) < n and time.time() < deadline:
        kernel.wait(0.2)
        events += kernel.read_event()
        while True:
            raw = kernel.pop()
            if raw is None:
                break
            out.append(raw)
    events += kernel.read_event()
    return out, events


def test_exactly_once_in_order_with_the_right_rows():
    rng = np.random.default_rng(90)
    kernel = ComputeKernel(echo=True, concurrency=8, max_contexts=12)
    assert kernel.pop() is None and kernel.read_event() == 0 and not kernel.wait(0.01)
    ctx_pool = np.arange(100, 112)
    sent = []
    n = 300
    for i in range(n):
        raw, p, acts = make_state(rng, i, int(rng.integers(1, 9)), ctx_pool)
        sent.append((p, acts))
        kernel.push(raw)
        if i % 37 == 0:
            time.sleep(0.002)                     # let the queues run empty now and then
    out, events = drain(kernel, n)
    assert len(out) == n and events == n
    assert kernel.pop() is None
    used = set()
    for i, raw in enumerate(out):
        m, p, acts, q, kv = wire.unpack_state(raw, DIM, KV)
        want_p, want_acts = sent[i]
        assert int(m["id"]) == i                                          # push order
        active = want_p["active"].astype(bool)
        used |= set(int(c) for c in want_p["context_id"][active])
        assert np.array_equal(p["token"], want_p["token"] + active)       # the model saw exactly the active rows
        assert np.array_equal(p["token_pos"], want_p["token_pos"] + active)
        for name in ("active", "context_id", "prompt_id", "temperature", "finished", "kv_tier"):
            assert np.array_equal(p[name], want_p[name])
        assert np.array_equal(acts, want_acts)
    counts = kernel.slot_counts()
    assert counts["allocated"] == len(used) and counts["free"] == 12 - len(used)
    kernel.close()


def test_refuses_what_it_cannot_run():
    kernel = ComputeKernel(echo=True, concurrency=4, max_contexts=4)
    raw, _, _ = make_state(np.random.default_rng(91), 1, 3, np.arange(5, 9))
    with pytest.raises(GlintError, match="too small"):
        kernel.push(raw[:40])
    with pytest.raises(GlintError, match="more data"):
        kernel.push(raw + b"!")
    big, _, _ = make_state(np.random.default_rng(92), 2, 5, np.arange(5, 12))
    with pytest.raises(GlintError, match="concurrency limit"):
        kernel.push(big)
    empty = wire.pack_state(dict(dtype=0), wire.new_prompts(0))
    with pytest.raises(GlintError, match="concurrency limit"):
        kernel.push(empty)
    kernel.push(raw)                                                    # still alive
    out, events = drain(kernel, 1)
    assert len(out) == 1 and events == 1
    kernel.close()


def test_shutdown_with_work_in_flight_returns():
    rng = np.random.default_rng(93)
    for _ in range(5):
        kernel = ComputeKernel(echo=True, concurrency=8, max_contexts=8)
        for i in range(50):
            kernel.push(make_state(rng, i, 4, np.arange(1, 9))[0])
        t0 = time.time()
        kernel.close()
        assert time.time() - t0 < 5.0
