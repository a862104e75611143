"""Benchmark configurations 3 and 5 at their own shapes, one hosted layer each, through the C++ stage
driver and against the oracle's fp32 CPU path:

  config 3  Llama2-13B shape (dim 5120, 40 heads, MHA), 8 prompts x 2048 tokens through the batched
            prefill (tile GEMMs on 16384 rows, causal MFMA attention over up to 2048 keys), then
            decode steps on the caches the prefill left
  config 5  Llama2-70B GQA shape, 256 context slots with lengths U[16, 4096): decode of all slots,
            then 10 % of them restart in place with a batched 128-token prefill; sticky slot
            indices, and the rows a restarted slot held before are never read again

A layer's output row for (context, token) depends on that token's input row and on the cache rows
before it, so single rows are checked: the rows [0, t) of the context come back from the GPU, the
oracle runs the layer for the one token at position t on them and must reproduce both the output row
and the cache row t that the GPU wrote.  Cache rows are additionally checked on their own for a
larger random sample (a row is a function of its input row alone)."""
import numpy as np
import pytest

import oracle as O
from glinthawk_amd import _lib, ops, stage as S
from helpers import assert_close, errors

pytestmark = pytest.mark.gpu

L = None


def lib():
    global L
    if L is None:
        L = _lib.lib()
    return L


def d2h(ptr, shape, dtype=np.float16):
    out = np.empty(shape, dtype=dtype)
    _lib.check(lib().gh_memcpy(out.ctypes.data, ptr, out.nbytes, _lib.GH_D2H, 0, None), "gh_memcpy")
    return out


def h2d(ptr, arr):
    a = np.ascontiguousarray(arr)
    _lib.check(lib().gh_memcpy(ptr, a.ctypes.data, a.nbytes, _lib.GH_H2D, 0, None), "gh_memcpy")


class Weights:
    """One layer's weights, drawn once on the host (a 4M-value N(0,1) block tiled at random offsets: fast to
    make and still without structure at the scale of a row), as fp16 for the stage and fp32 for the oracle."""

    def __init__(self, cfg, seed):
        rng = np.random.default_rng(seed)
        block = rng.standard_normal(1 << 22).astype(np.float32)

        def tiled(shape, scale, shift=0.0):
            n = int(np.prod(shape))
            reps = (n + block.size - 1) // block.size + 1
            off = int(rng.integers(0, block.size))
            return (np.tile(block, reps)[off:off + n] * np.float32(scale) + np.float32(shift)).astype(np.float16).reshape(shape)

        s_in = 1.0 / np.sqrt(cfg.dim)
        self.w16 = {
            "rms_att_weight": tiled((cfg.dim,), 0.1, 1.0), "wq": tiled((cfg.dim, cfg.dim), s_in),
            "wkv": tiled((2 * cfg.kv_dim, cfg.dim), s_in), "wo": tiled((cfg.dim, cfg.dim), s_in),
            "rms_ffn_weight": tiled((cfg.dim,), 0.1, 1.0), "w1": tiled((cfg.hidden_dim, cfg.dim), s_in),
            "w2": tiled((cfg.dim, cfg.hidden_dim), 1.0 / np.sqrt(cfg.hidden_dim)), "w3": tiled((cfg.hidden_dim, cfg.dim), s_in),
        }
        self.w32 = {k: v.astype(np.float32) for k, v in self.w16.items()}
        re, im = O.rope_tables(cfg.seq_len, cfg.head_size)
        self.re16, self.im16 = re.astype(np.float16), im.astype(np.float16)
        self.re32, self.im32 = self.re16.astype(np.float32), self.im16.astype(np.float32)

    def load(self, st, layer):
        for name, arr in self.w16.items():
            st.set_layer_tensor(layer, name, arr)
        st.set_base_tensor("freq_cis_real", self.re16)
        st.set_base_tensor("freq_cis_imag", self.im16)


def oracle_rows(cfg, w, x_rows, caches, positions):
    """The oracle's layer for a handful of independent (context, position) rows.  `caches[k]` holds the rows
    [0, positions[k]] of that context as the GPU left them (fp32 copies); the oracle overwrites row positions[k]
    with its own K/V.  Returns (output rows, the cache rows the oracle appended)."""
    x = np.ascontiguousarray(x_rows, dtype=np.float32)
    O.layer_forward(cfg, w.w32, w.re32, w.im32, x, caches, positions)
    return x, [caches[k][positions[k]].copy() for k in range(len(positions))]


def oracle_kv_rows(cfg, w, x_rows, positions):
    """[rope(K) | V] of single tokens: rmsnorm -> wkv -> RoPE on the K half (models/llama2/model.hh:326-364)."""
    x = np.ascontiguousarray(x_rows, dtype=np.float32)
    xb = O.rmsnorm(x, w.w32["rms_att_weight"])
    kv = O.matmul(xb, w.w32["wkv"])
    q = np.zeros((len(positions), cfg.dim), np.float32)
    O.apply_rope(cfg, positions, w.re32, w.im32, q, [kv[k] for k in range(len(positions))])
    return kv


@pytest.mark.timeout(900)
def test_config3_llama13b_prefill_8x2048_then_decode(product_route):
    cfg = O.Config(dim=5120, n_layers=40, n_heads=40, n_kv_heads=40, hidden_dim=13824, seq_len=4096, attention_rounds=2)
    layer, batch, T = 12, 8, 2048
    ops.init(0)
    w = Weights(cfg, seed=31)
    st = S.Stage("llama2-13b-4k", "f16", layer, 1, batch, batch)
    w.load(st, layer)
    rng = np.random.default_rng(32)
    x = ops.pinned_empty((batch * T, cfg.dim), np.float16)
    x[:] = rng.standard_normal((batch * T, cfg.dim)).astype(np.float16)
    y = ops.pinned_empty((batch * T, cfg.dim), np.float16)
    y[:] = 0
    ids = [900 + i for i in range(batch)]
    res = st.prefill(ids, [0] * batch, T, layer, activations=x, out=y)
    assert res is not None and res[0] is y
    out = y.reshape(batch, T, cfg.dim)
    xin = x.reshape(batch, T, cfg.dim)
    assert np.isfinite(out.astype(np.float32)).all()

    row_elems = 2 * cfg.kv_dim
    # the prompt rows of every context, as the prefill wrote them (the oracle needs room up to the decode positions)
    n_keep = T + 8
    caches = [np.zeros((n_keep, row_elems), np.float32) for _ in range(batch)]
    for i in range(batch):
        caches[i][:T] = d2h(st.context_layer_ptr(i, layer), (T, row_elems)).astype(np.float32)

    # (a) cache rows on their own: 192 random (context, token) pairs plus the corners
    pairs = [(0, 0), (0, 1), (batch - 1, T - 1), (3, 63), (3, 64), (3, 65), (5, 1023), (5, 1024)]
    pairs += [(int(rng.integers(0, batch)), int(rng.integers(0, T))) for _ in range(192)]
    want_kv = oracle_kv_rows(cfg, w, np.stack([xin[i, t] for i, t in pairs]), [t for _, t in pairs])
    got_kv = np.stack([caches[i][t] for i, t in pairs])
    assert_close(got_kv, want_kv, what="13B prefill: cache rows [rope(K) | V]")
    for k in range(0, len(pairs), 25):           # and row by row, so that one bad row cannot hide in the mean
        a, r = errors(got_kv[k], want_kv[k])
        assert a <= 2e-2 and r <= 2e-3, (pairs[k], a, r)

    # (b) whole-layer output rows: 64 (context, token) pairs, one per context at a time
    tokens = [0, 1, 15, 16, 63, 64, 65, 127, 128, 255, 256, 1023, 1024, 2046, 2047]
    sample = [(i, t) for i in range(batch) for t in tokens[i::2]]                       # every context, every listed token once or more
    sample += [(int(rng.integers(0, batch)), int(rng.integers(0, T))) for _ in range(64 - len(sample))]
    worst = 0.0
    pending = list(dict.fromkeys(sample))
    while pending:
        group, seen = [], set()                  # at most one row per context at a time: the oracle writes into the context's rows
        for i, t in pending:
            if i not in seen and len(group) < batch:
                group.append((i, t))
                seen.add(i)
        pending = [p for p in pending if p not in group]
        saved = [caches[i][t].copy() for i, t in group]
        want, appended = oracle_rows(cfg, w, np.stack([xin[i, t] for i, t in group]), [caches[i] for i, _ in group], [t for _, t in group])
        for k, (i, t) in enumerate(group):
            a, r = errors(out[i, t].astype(np.float32), want[k])
            worst = max(worst, r)
            assert a <= 2e-2 and r <= 1e-3, f"13B prefill: output row of context {i}, token {t}: max_abs {a:.2e}, mean_rel {r:.2e}"
            a, r = errors(saved[k], appended[k])
            assert a <= 2e-2 and r <= 2e-3, f"13B prefill: cache row of context {i}, token {t}: max_abs {a:.2e}, mean_rel {r:.2e}"
            caches[i][t] = saved[k]              # later rows are checked against what the GPU holds
    assert worst > 0.0
    product_route.check()                        # the prefill's plain products ran where the route says

    # (c) decode steps on the caches the prefill left (MHA: the dot2/DPP kernel over 2049.. keys)
    for step in range(3):
        pos = T + step
        xd = rng.standard_normal((batch, cfg.dim)).astype(np.float16)
        st.new_state(batch, next_layer=layer)
        for i in range(batch):
            st.set_prompt(i, ids[i], 1, pos)
        st.activations(allocate=True)[:] = xd.reshape(-1)
        assert st.forward()
        got = st.activations().reshape(batch, cfg.dim).astype(np.float32)
        want, appended = oracle_rows(cfg, w, xd, caches, [pos] * batch)
        assert_close(got, want, what=f"13B decode step {step} after the prefill")
        for i in (0, batch - 1):
            row = d2h(st.context_layer_ptr(i, layer) + pos * row_elems * 2, (row_elems,)).astype(np.float32)
            a, r = errors(row, appended[i])
            assert a <= 2e-2 and r <= 2e-3, (i, a, r)
            caches[i][pos] = row
    st.close()


def test_prefill_cache_rows_equal_the_token_by_token_path_13b_shape():
    """The rows a batched prefill appends against those of the reference's way (one token per forward) on one
    short prompt at the 13B shape.  The two run different GEMM kernels (tile against weight-streaming), whose
    fp32 sums differ in order, so a few elements of a row differ in the last place (for an element near zero
    that is many units of its own last place, hence the absolute bound)."""
    cfg = O.Config(dim=5120, n_layers=40, n_heads=40, n_kv_heads=40, hidden_dim=13824, seq_len=4096, attention_rounds=2)
    layer, batch, T = 12, 3, 48
    ops.init(0)
    w = Weights(cfg, seed=33)
    a = S.Stage("llama2-13b-4k", "f16", layer, 1, batch, batch)
    b = S.Stage("llama2-13b-4k", "f16", layer, 1, batch, batch)
    for st in (a, b):
        w.load(st, layer)
    rng = np.random.default_rng(34)
    x = rng.standard_normal((batch, T, cfg.dim)).astype(np.float16)
    ids = [50, 51, 52]
    res = a.prefill(ids, [0] * batch, T, layer, activations=x.reshape(batch * T, cfg.dim))
    assert res is not None
    out_a = res[0].reshape(batch, T, cfg.dim).astype(np.float32)
    out_b = np.zeros_like(out_a)
    for pos in range(T):
        b.new_state(batch, next_layer=layer)
        for i in range(batch):
            b.set_prompt(i, ids[i], 1, pos)
        b.activations(allocate=True)[:] = x[:, pos].reshape(-1)
        assert b.forward()
        out_b[:, pos] = b.activations().reshape(batch, cfg.dim).astype(np.float32)
    row_elems = 2 * cfg.kv_dim
    from helpers import half_ulp_diff
    for i in range(batch):
        ra = d2h(a.context_layer_ptr(i, layer), (T, row_elems))
        rb = d2h(b.context_layer_ptr(i, layer), (T, row_elems))
        _, frac = half_ulp_diff(ra, rb)
        assert frac < 0.01, (i, frac)                                              # measured: 0.15 % of the elements differ at all
        np.testing.assert_allclose(ra.astype(np.float32), rb.astype(np.float32), rtol=1e-3, atol=1e-3)
    np.testing.assert_allclose(out_a, out_b, rtol=6e-3, atol=6e-3)
    a.close()
    b.close()


NAN16 = np.uint16(0x7E00)


@pytest.mark.timeout(900)
def test_config5_churn_256_slots_batched_refill():
    cfg = O.Config(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096)
    layer, slots, refill, steps = 40, 256, 128, 5
    ops.init(0)
    w = Weights(cfg, seed=51)
    st = S.Stage("llama2-70b-4k", "f16", layer, 1, slots, slots)
    w.load(st, layer)
    rng = np.random.default_rng(52)
    pos = rng.integers(16, 4096, slots)
    pos[:4] = [16, 4094, 2047, 300]                                   # the extremes are always there
    ids = [1000 + i for i in range(slots)]
    st.new_state(slots, next_layer=layer)
    for i in range(slots):
        st.set_prompt(i, ids[i], 1, int(pos[i]))
    assert st.acquire_contexts()
    slot_of = [st.context_slot(i) for i in range(slots)]
    assert sorted(slot_of) == list(range(slots))
    row_elems = 2 * cfg.kv_dim
    layer_ptr = [st.context_layer_ptr(i, layer) for i in range(slots)]
    poison = np.full((cfg.seq_len, row_elems), NAN16, dtype=np.uint16)
    for i in range(slots):
        # rows [0, pos) hold N(0,1) values, everything from the current position on is NaN: a kernel that reads a
        # row it must not read shows up as NaN in its output
        _lib.check(lib().gh_fill_normal(layer_ptr[i], int(pos[i]) * row_elems, 0.0, 1.0, 7000 + i, _lib.GH_F16, None))
        h2d(layer_ptr[i] + int(pos[i]) * row_elems * 2, poison[int(pos[i]):])
    ops.sync()
    prompt = ops.pinned_empty((slots * refill, cfg.dim), np.float16)
    restarted_total = 0

    for step in range(steps):
        # ---- decode of all 256 slots at their ragged positions
        xd = rng.standard_normal((slots, cfg.dim)).astype(np.float16)
        st.new_state(slots, next_layer=layer)
        for i in range(slots):
            st.set_prompt(i, ids[i], 1, int(pos[i]))
        st.activations(allocate=True)[:] = xd.reshape(-1)
        assert st.forward()
        assert [st.context_slot(i) for i in range(slots)] == slot_of                     # sticky: nobody moved
        assert [st.context_layer_ptr(i, layer) for i in range(slots)] == layer_ptr
        got = st.activations().reshape(slots, cfg.dim).astype(np.float32)
        assert np.isfinite(got).all(), f"step {step}: a row beyond some slot's position was read"
        # sampled slots against the oracle: the shortest, the longest, a just-restarted one (from step 1 on), random ones
        sample = {int(np.argmin(pos)), int(np.argmax(pos)), int(rng.integers(0, slots)), int(rng.integers(0, slots))}
        if step > 0:
            sample.add(int(last_gone[0]))
        sample = sorted(sample)
        caches = []
        for i in sample:
            c = np.zeros((int(pos[i]) + 1, row_elems), np.float32)
            c[:] = d2h(layer_ptr[i], (int(pos[i]) + 1, row_elems)).astype(np.float32)
            caches.append(c)
        gpu_rows = [c[int(pos[i])].copy() for c, i in zip(caches, sample)]
        want, appended = oracle_rows(cfg, w, xd[sample], caches, [int(pos[i]) for i in sample])
        for k, i in enumerate(sample):
            a, r = errors(got[i], want[k])
            assert a <= 2e-2 and r <= 1e-3, f"step {step}, slot {i} at position {pos[i]}: max_abs {a:.2e}, mean_rel {r:.2e}"
            a, r = errors(gpu_rows[k], appended[k])
            assert a <= 2e-2 and r <= 2e-3, f"step {step}, slot {i}: appended row max_abs {a:.2e}, mean_rel {r:.2e}"
        pos = pos + 1

        # ---- 10 % of the slots finish and restart in place with a batched 128-token prefill
        done = (rng.random(slots) < 0.10) | (pos >= cfg.seq_len - 1)
        gone = np.nonzero(done)[0]
        assert len(gone) > 0
        restarted_total += len(gone)
        for i in gone:
            h2d(layer_ptr[i], poison)                                                    # everything the slot held is now poison
        n = len(gone) * refill
        prompt[:n] = rng.standard_normal((n, cfg.dim)).astype(np.float16)
        res = st.prefill([ids[i] for i in gone], [0] * len(gone), refill, layer, activations=prompt[:n])
        assert res is not None
        out = res[0].reshape(len(gone), refill, cfg.dim).astype(np.float32)
        assert np.isfinite(out).all(), f"step {step}: the refill read rows of the evicted contexts"
        assert [st.context_slot(k) for k in range(len(gone))] == [slot_of[i] for i in gone]     # same slots as before
        pin = prompt[:n].reshape(len(gone), refill, cfg.dim)
        # sampled (slot, token) rows of the refill against the oracle
        picks = [(0, 0), (len(gone) - 1, refill - 1), (len(gone) // 2, 63), (len(gone) // 2, 64)]      # each on its own copy of the rows
        caches = []
        for k, t in picks:
            c = np.zeros((t + 1, row_elems), np.float32)
            c[:] = d2h(layer_ptr[gone[k]], (t + 1, row_elems)).astype(np.float32)
            caches.append(c)
        want, _ = oracle_rows(cfg, w, np.stack([pin[k, t] for k, t in picks]), caches, [t for _, t in picks])
        for j, (k, t) in enumerate(picks):
            a, r = errors(out[k, t], want[j])
            assert a <= 2e-2 and r <= 1e-3, f"step {step}: refill of slot {gone[k]}, token {t}: max_abs {a:.2e}, mean_rel {r:.2e}"
        for i in gone:                                                                   # rows beyond the new prompt stay poison
            tail = d2h(layer_ptr[i] + refill * row_elems * 2, (2, row_elems), np.uint16)
            assert (tail == NAN16).all()
        pos[gone] = refill
        last_gone = gone
    assert restarted_total >= steps * 10
    assert st.slot_counts() == dict(free=0, allocated=slots, total=slots)
    st.close()
