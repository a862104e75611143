"""The C++ stage driver on the GPU against the oracle's layer-by-layer fp32 CPU path: full decode
steps (embedding -> layers -> classifier -> argmax), the stage-at-a-time entry points, fused vs
unfused attention, slot reuse and paged contexts."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from glinthawk_amd import _lib, stage as S
from helpers import assert_close, assert_half_parity, errors

pytestmark = pytest.mark.gpu

SHAPES = {
    "test-tiny": O.Config(dim=32, n_layers=2, n_heads=4, n_kv_heads=2, hidden_dim=48, seq_len=16),
    "test-mha": O.Config(dim=512, n_layers=2, n_heads=4, n_kv_heads=4, hidden_dim=768, seq_len=192, attention_rounds=2),
    "test-gqa4": O.Config(dim=1024, n_layers=3, n_heads=8, n_kv_heads=2, hidden_dim=1536, seq_len=320),
    "stories15m": O.Config(dim=288, n_layers=6, n_heads=6, n_kv_heads=6, hidden_dim=768, seq_len=256, attention_rounds=2),
}
WCLS = {"test-tiny": True, "test-mha": False, "test-gqa4": True, "stories15m": False}


def d2h(ptr, shape, dtype):
    out = np.empty(shape, dtype=dtype)
    _lib.check(_lib.lib().gh_memcpy(out.ctypes.data, ptr, out.nbytes, _lib.GH_D2H, 0, None), "gh_memcpy")
    return out


def make_weights(cfg, np_dt, seed, wcls):
    """Weights scaled so that activations and logits stay O(1); values are exactly representable in
    the storage type, the oracle gets the same values as fp32."""
    r = np.random.default_rng(seed)
    s = 1.0 / np.sqrt(cfg.dim)
    layers = []
    for _ in range(cfg.n_layers):
        layers.append({
            "rms_att_weight": (1 + 0.1 * r.standard_normal(cfg.dim)).astype(np_dt),
            "wq": (s * r.standard_normal((cfg.dim, cfg.dim))).astype(np_dt),
            "wkv": (s * r.standard_normal((2 * cfg.kv_dim, cfg.dim))).astype(np_dt),
            "wo": (s * r.standard_normal((cfg.dim, cfg.dim))).astype(np_dt),
            "rms_ffn_weight": (1 + 0.1 * r.standard_normal(cfg.dim)).astype(np_dt),
            "w1": (s * r.standard_normal((cfg.hidden_dim, cfg.dim))).astype(np_dt),
            "w2": (r.standard_normal((cfg.dim, cfg.hidden_dim)) / np.sqrt(cfg.hidden_dim)).astype(np_dt),
            "w3": (s * r.standard_normal((cfg.hidden_dim, cfg.dim))).astype(np_dt),
        })
    base = {
        # std 1/sqrt(dim): with a shared classifier the logits (unit-rms activations . table rows) stay O(1)
        "token_embedding_table": (s * r.standard_normal((cfg.vocab_size, cfg.dim))).astype(np_dt),
        "rms_final_weight": (1 + 0.1 * r.standard_normal(cfg.dim)).astype(np_dt),
    }
    base["wcls"] = (s * r.standard_normal((cfg.vocab_size, cfg.dim))).astype(np_dt) if wcls else base["token_embedding_table"]
    re, im = O.rope_tables(cfg.seq_len, cfg.head_size)
    base["freq_cis_real"], base["freq_cis_imag"] = re.astype(np_dt), im.astype(np_dt)
    return layers, base


def load_weights(st, cfg, layers, base, wcls, layer_range=None, with_embedding=True, with_cls=True):
    for l in (layer_range or range(cfg.n_layers)):
        for name in S.LAYER_TENSORS:
            st.set_layer_tensor(l, name, layers[l][name])
    st.set_base_tensor("freq_cis_real", base["freq_cis_real"])
    st.set_base_tensor("freq_cis_imag", base["freq_cis_imag"])
    if with_embedding:
        st.set_base_tensor("token_embedding_table", base["token_embedding_table"])
    if with_cls:
        st.set_base_tensor("rms_final_weight", base["rms_final_weight"])
        if wcls:
            st.set_base_tensor("wcls", base["wcls"])


class OracleModel:
    """The reference's CPU path, layer by layer, with its own KV cache per context id: fp32 storage (the
    parity target), or fp16 storage with every op output rounded where the reference's fp16 build rounds it."""

    def __init__(self, cfg, layers, base, storage=np.float32):
        self.cfg = cfg
        self.storage = storage
        self.layers = [{k: np.ascontiguousarray(v, dtype=storage) for k, v in lw.items()} for lw in layers]
        self.base = {k: np.ascontiguousarray(v, dtype=storage) for k, v in base.items()}
        self.cache = {}

    def ctx(self, cid):
        if cid not in self.cache:
            self.cache[cid] = np.zeros((self.cfg.n_layers, self.cfg.seq_len, 2 * self.cfg.kv_dim), self.storage)
        return self.cache[cid]

    def run_layers(self, x, cids, pos, layer_range):
        for l in layer_range:
            rows = [None if c is None else self.ctx(c)[l] for c in cids]
            O.layer_forward(self.cfg, self.layers[l], self.base["freq_cis_real"], self.base["freq_cis_imag"], x, rows, pos)
        return x

    def step(self, tokens, cids, pos):
        x = np.ascontiguousarray(self.base["token_embedding_table"][tokens])
        self.run_layers(x, cids, pos, range(self.cfg.n_layers))
        return O.classify(self.cfg, self.base["rms_final_weight"], self.base["wcls"], x)


@pytest.mark.parametrize("name,dtype", [("test-tiny", "f32"), ("test-tiny", "f16"), ("test-mha", "f16"), ("test-gqa4", "f16"),
                                        ("stories15m", "f32")])
@pytest.mark.parametrize("fused", [True, False])
def test_full_model_decode_matches_oracle(name, dtype, fused):
    cfg = SHAPES[name]
    np_dt = np.float16 if dtype == "f16" else np.float32
    layers, base = make_weights(cfg, np_dt, seed=5, wcls=WCLS[name])
    batch = 4
    st = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, fused=fused, with_cls=True)
    load_weights(st, cfg, layers, base, WCLS[name])
    ref = OracleModel(cfg, layers, base)
    ref16 = OracleModel(cfg, layers, base, np.float16) if dtype == "f16" else None

    rng = np.random.default_rng(6)
    tokens = rng.integers(0, cfg.vocab_size, batch).tolist()
    steps = min(12, cfg.seq_len)
    st.new_state(batch)
    for i in range(batch):
        st.set_prompt(i, 100 + i, tokens[i], 0, 0.0, 1, 0)
    margin_ok = 0
    for step in range(steps):
        pos = [step] * batch
        want = ref.step(tokens, [100 + i for i in range(batch)], pos)
        assert st.forward()
        got = d2h(st.scratch_ptr("logits"), (batch, cfg.vocab_size), np_dt).astype(np.float32)
        if dtype == "f32":
            # fp32 storage: the north-star tolerance (2e-2 max-abs, 1e-3 mean-relative) and element-wise
            np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-4)
            assert_close(got, want, mean_rel=1e-3, what=f"{name} logits step {step}")
        else:
            # fp16 storage: held to the CPU path with the same storage type; the distance to fp32 is the storage's
            want16 = ref16.step(tokens, [100 + i for i in range(batch)], pos)
            # the smallest shape runs kernels that add in the oracle's order: there the unfused path, which rounds
            # where the reference rounds, reproduces the fp16 oracle almost bit for bit (measured 2e-5)
            assert_half_parity(got, want16, want, what=f"{name} {'fused' if fused else 'unfused'} logits step {step}",
                               tol16=1e-4 if (name == "test-tiny" and not fused) else None)
        rows = [st.row(i) for i in range(batch)]
        for i in range(batch):
            assert rows[i]["token_pos"] == step + 1
            top2 = np.sort(want[i])[-2:]
            if top2[1] - top2[0] > 5e-2:         # clear winner on the CPU: the GPU must pick the same token
                assert rows[i]["token"] == int(np.argmax(want[i]))
                margin_ok += 1
        tokens = [rows[i]["token"] for i in range(batch)]     # teacher forcing from the GPU's choice
        sinfo = st.state()
        assert sinfo["next_layer"] == 0 and sinfo["next_stage"] == S.STAGE_PRE and not sinfo["has_activations"]
    assert margin_ok > steps      # the argmax comparison was not vacuous
    st.close()


def test_stage_at_a_time_equals_forward():
    name, dtype = "test-gqa4", "f16"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=7, wcls=True)
    batch = 3
    a = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True)
    b = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True)
    for st in (a, b):
        load_weights(st, cfg, layers, base, True)
        st.new_state(batch)
        for i in range(batch):
            st.set_prompt(i, i, 11 + i, 0)
    for step in range(5):
        assert a.forward()
        for l in range(cfg.n_layers):
            assert b.forward(S.FWD_PRE)
            sb = b.state()
            assert sb["next_stage"] == S.STAGE_ATT and sb["has_queries"] and sb["has_kvs"]
            assert b.forward(S.FWD_ATT)
            assert b.state()["next_stage"] == S.STAGE_POST
            assert b.forward(S.FWD_POST)
        assert b.state()["next_stage"] == S.STAGE_CLS
        assert b.forward(S.FWD_CLS)
        la = d2h(a.scratch_ptr("logits"), (batch, cfg.vocab_size), np.float16)
        lb = d2h(b.scratch_ptr("logits"), (batch, cfg.vocab_size), np.float16)
        # forward() fuses the projections with their follow-up ops, the staged path issues them one by
        # one and round-trips through host buffers: same arithmetic, possibly different K splits and
        # rmsnorm reduction order, so agreement is to fp16 rounding, not bit for bit
        np.testing.assert_allclose(la.astype(np.float32), lb.astype(np.float32), rtol=4e-3, atol=4e-3)
        ta, tb = [a.row(i)["token"] for i in range(batch)], [b.row(i)["token"] for i in range(batch)]
        for i in range(batch):
            if ta[i] != tb[i]:                 # only a near-tie may flip
                assert abs(float(la[i, ta[i]]) - float(la[i, tb[i]])) < 8e-3
                b.set_prompt(i, i, ta[i], step + 1)
    a.close()
    b.close()


def test_middle_stage_activations_in_and_out():
    # layers 1..2 of a 3-layer model, no embedding, no classifier: activations arrive and leave through the host buffer
    name, dtype = "test-gqa4", "f16"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=8, wcls=True)
    batch = 5
    st = S.Stage(name, dtype, 1, 2, batch, batch, with_cls=False)
    load_weights(st, cfg, layers, base, True, layer_range=[1, 2], with_embedding=False, with_cls=False)
    ref = OracleModel(cfg, layers, base)
    rng = np.random.default_rng(9)
    cids = [7, 8, 9, 10, 11]
    for step in range(6):
        x = rng.standard_normal((batch, cfg.dim)).astype(np.float16)
        st.new_state(batch, next_layer=1)
        for i in range(batch):
            st.set_prompt(i, cids[i], 1, step)
        st.activations(allocate=True)[:] = x.reshape(-1)
        assert st.forward()
        got = st.activations().reshape(batch, cfg.dim).astype(np.float32)
        want = ref.run_layers(x.astype(np.float32), cids, [step] * batch, [1, 2])
        assert_close(got, want, what=f"middle stage step {step}")
        s = st.state()
        assert s["next_stage"] == S.STAGE_CLS and s["has_activations"]      # layer 2 was the last layer
    st.close()


def test_inactive_rows_and_slot_reuse():
    name, dtype = "test-mha", "f16"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=10, wcls=False)
    batch = 4
    st = S.Stage(name, dtype, 0, cfg.n_layers, batch, 3, with_cls=True)       # only 3 slots for 4 rows
    load_weights(st, cfg, layers, base, False)
    ref = OracleModel(cfg, layers, base)
    st.new_state(batch)
    for i in range(batch):
        st.set_prompt(i, 50 + i, 5 + i, 0)
    assert not st.forward()                        # 4 unseen ids, 3 slots: refused, nothing allocated
    assert st.slot_counts() == dict(free=3, allocated=0, total=3)
    st.discard(2)                                  # row 2 inactive -> shared empty context
    tokens = [5, 6, 0, 8]
    for step in range(3):
        assert st.forward()
        assert [st.context_slot(i) for i in range(batch)] == [0, 1, -1, 2]
        want = ref.step(tokens, [50, 51, None, 53], [step] * batch)
        got = d2h(st.scratch_ptr("logits"), (batch, cfg.vocab_size), np.float16).astype(np.float32)
        assert_close(got[[0, 1, 3]], want[[0, 1, 3]], what="active rows")
        assert st.row(2)["token_pos"] == 0 and not st.row(2)["active"]
        tokens = [st.row(i)["token"] for i in range(batch)]
    # row 0 finishes and is refilled under the same context id at position 0: same slot, old rows ignored
    st.set_prompt(0, 50, 9, 0)
    ref.cache.pop(50)
    tokens[0] = 9
    assert st.forward()
    assert st.context_slot(0) == 0
    want = ref.step(tokens, [50, 51, None, 53], [0, 3, 0, 3])
    got = d2h(st.scratch_ptr("logits"), (batch, cfg.vocab_size), np.float16).astype(np.float32)
    assert_close(got[[0, 1, 3]], want[[0, 1, 3]], what="after slot restart")
    st.close()


def test_finish_rule_sets_flag():
    name = "test-tiny"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float32, seed=11, wcls=True)
    st = S.Stage(name, "f32", 0, cfg.n_layers, 2, 2, with_cls=True)
    load_weights(st, cfg, layers, base, True)
    st.new_state(2)
    st.set_prompt(0, 1, 3, 0, 0.0, 2, 3)           # prompt 2 + completion 3 -> finished when token_pos reaches 5
    st.set_prompt(1, 2, 4, cfg.seq_len - 2, 0.0, 1, 0)
    for step in range(5):
        assert st.forward()
        r0, r1 = st.row(0), st.row(1)
        assert r0["finished"] == O.check_finished(r0["token"], r0["token_pos"], 2, 3, cfg.seq_len)
        if step == 0:
            assert not r1["finished"] or r1["token"] == 2
        if step == 1:
            assert r1["finished"]                  # token_pos == seq_len
            st.discard(1)
    assert st.row(0)["finished"]
    st.close()


def test_paged_contexts_equal_static_and_follow_block_rule():
    # one layer of the 70B-4K shape: 16 MiB span per context, 2 MiB = 512 rows per block
    name, dtype = "llama2-70b-4k", "f16"
    cfg70 = O.Config(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096)
    batch = 2
    outs = []
    for paged in (False, True):
        st = S.Stage(name, dtype, 3, 1, batch, batch, paged=paged, seed=3, weight_std=0.02)
        rng = np.random.default_rng(12)
        got = []
        for pos in (0, 1, 2, 511, 512, 513, 1500, 0, 1):     # includes block boundaries, a jump and a restart
            x = rng.standard_normal((batch, cfg70.dim)).astype(np.float16)
            st.new_state(batch, next_layer=3)
            st.set_prompt(0, 1, 1, pos)
            st.set_prompt(1, 2, 1, min(pos, 2))
            st.activations(allocate=True)[:] = x.reshape(-1)
            assert st.forward()
            got.append(st.activations().copy())
            if paged:
                allocated = np.zeros(80, np.uint64)
                O.dynctx_prepare(cfg70, 2, allocated, 3, pos, False, commit_all=True)
                info = st.paging_info(0, 3)
                assert info["allocated_bytes"] >= int(allocated[3])
                if pos == 513:
                    assert info["allocated_bytes"] == 2 * 2 ** 21
                if pos == 1500:
                    assert info["allocated_bytes"] == 3 * 2 ** 21
        if paged:
            info = st.paging_info(0, 3)
            assert info["clears"] == 2 and info["allocated_bytes"] == 2 ** 21      # restart dropped every page
        outs.append(got)
        st.close()
    # positions 0, 1, 2 and the restart see only rows written in this run: identical bits in both modes
    for k in (0, 1, 2, 7, 8):
        assert np.array_equal(outs[0][k], outs[1][k])


def test_set_prompts_equals_row_by_row():
    name = "test-tiny"
    cfg = SHAPES[name]
    a = S.Stage(name, "f32", 0, cfg.n_layers, 5, 5, with_cls=True)
    b = S.Stage(name, "f32", 0, cfg.n_layers, 5, 5, with_cls=True)
    ids, tokens, pos = [40, 41, 42, 43, 44], [3, 1, 4, 1, 5], [0, 7, 2, 9, 1]
    a.new_state(5)
    b.new_state(5)
    for i in range(5):
        a.set_prompt(i, ids[i], tokens[i], pos[i], 0.5, 3, 2)
    b.set_prompts(ids, tokens, pos, 0.5, 3, 2)
    assert [a.row(i) for i in range(5)] == [b.row(i) for i in range(5)]
    assert a.get_state_bytes() == b.get_state_bytes()
    with pytest.raises(ValueError):
        b.set_prompts(ids, tokens[:4], pos)
    a.close()
    b.close()


def test_device_span_timing_counts_steps_and_leaves_results_alone():
    # the span timer records two events per forward(): same outputs with it on, one span per step, a read resets it
    import time
    name, dtype = "test-gqa4", "f16"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=8, wcls=True)
    batch = 5
    rng = np.random.default_rng(10)
    xs = [rng.standard_normal((batch, cfg.dim)).astype(np.float16) for _ in range(4)]

    def run(timed):
        st = S.Stage(name, dtype, 1, 2, batch, batch, with_cls=False)
        load_weights(st, cfg, layers, base, True, layer_range=[1, 2], with_embedding=False, with_cls=False)
        st.time_device_spans(timed)
        outs, wall = [], 0.0
        for step, x in enumerate(xs):
            st.new_state(batch, next_layer=1)
            for i in range(batch):
                st.set_prompt(i, 20 + i, 1, step)
            st.activations(allocate=True)[:] = x.reshape(-1)
            t0 = time.perf_counter()
            assert st.forward()
            wall += time.perf_counter() - t0
            outs.append(st.activations().copy())
        spans = st.device_spans()
        again = st.device_spans()
        st.close()
        return outs, spans, again, wall * 1e3

    plain, spans_off, _, _ = run(False)
    timed, spans_on, again, wall_ms = run(True)
    assert spans_off == (0.0, 0)
    assert spans_on[1] == len(xs) and again == (0.0, 0)
    assert 0.0 < spans_on[0] <= wall_ms, (spans_on, wall_ms)
    for a, b in zip(plain, timed):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("balanced", [True, False], ids=["equal-runs", "per-context"])
@pytest.mark.parametrize("name,first,n_hosted", [("test-gqa4", 1, 2), ("test-mha", 1, 1)])
def test_decode_attention_over_equal_runs_of_keys_in_a_stage(name, first, n_hosted, balanced):
    # contexts of very different lengths and an inactive row; cache rows written straight into the slots.  Both attention
    # routes of the fused path against the oracle on the same rows, for grouped and for one-to-one query heads.
    dtype = "f16"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=12, wcls=WCLS[name])
    top = cfg.seq_len - 1
    pos = [0, 5, top, 64, 100, top - 64, top - 63, top - 19, 17]
    batch = len(pos)
    cids = [40 + i for i in range(batch)]
    hosted = list(range(first, first + n_hosted))
    st = S.Stage(name, dtype, first, n_hosted, batch, batch, with_cls=False, balanced=balanced)
    load_weights(st, cfg, layers, base, WCLS[name], layer_range=hosted, with_embedding=False, with_cls=False)
    ref = OracleModel(cfg, layers, base)
    rng = np.random.default_rng(13)
    st.new_state(batch, next_layer=first)
    for i in range(batch):
        st.set_prompt(i, cids[i], 1, pos[i])
    st.discard(4)
    assert st.acquire_contexts()
    for i in range(batch):
        if i == 4:
            continue
        for l in hosted:
            rows = rng.standard_normal((cfg.seq_len, 2 * cfg.kv_dim)).astype(np.float16)
            _lib.check(_lib.lib().gh_memcpy(st.context_layer_ptr(i, l), rows.ctypes.data, rows.nbytes, _lib.GH_H2D, 0, None), "gh_memcpy")
            ref.ctx(cids[i])[l][:] = rows.astype(np.float32)
    x = rng.standard_normal((batch, cfg.dim)).astype(np.float16)
    st.activations(allocate=True)[:] = x.reshape(-1)
    assert st.forward()
    got = st.activations().reshape(batch, cfg.dim).astype(np.float32)
    want = ref.run_layers(x.astype(np.float32), [None if i == 4 else c for i, c in enumerate(cids)], pos, hosted)
    live = [i for i in range(batch) if i != 4]
    assert_close(got[live], want[live], what="stage step over ragged contexts")
    # the appended rows are where the oracle put them
    for i in (2, 7):
        row = d2h(st.context_layer_ptr(i, hosted[-1]) + pos[i] * 2 * cfg.kv_dim * 2, (2 * cfg.kv_dim,), np.float16).astype(np.float32)
        assert_close(row[None], ref.ctx(cids[i])[hosted[-1]][pos[i]][None], what="appended row")
    st.close()
