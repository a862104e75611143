"""Parity runs shaped like the benchmark configurations, through the C++ stage driver:
  config 1  stories15M shape, fp32, batch 4, greedy decode of 256 positions from 8 prompt tokens
  config 2  Llama2-7B shape (two of its layers), fp16, batch 32, contexts pre-filled to 1024 rows
  config 5  slot churn with ragged lengths, evictions and refills (reduced shape, full bookkeeping)
Each is compared with the oracle's fp32 CPU path fed the same seeded inputs."""
import numpy as np
import pytest

import oracle as O
from glinthawk_amd import _lib, stage as S
from helpers import assert_close, assert_half_parity, errors
from test_gpu_stage import SHAPES, OracleModel, d2h, load_weights, make_weights

pytestmark = pytest.mark.gpu


def h2d(ptr, arr):
    a = np.ascontiguousarray(arr)
    _lib.check(_lib.lib().gh_memcpy(ptr, a.ctypes.data, a.nbytes, _lib.GH_H2D, 0, None), "gh_memcpy")


def test_config1_stories15m_greedy_256():
    name = "stories15m"
    cfg = SHAPES[name]
    rng = np.random.default_rng(1)
    # the configuration's own initialisation: every weight N(0, 0.02), fp32
    layers = []
    for _ in range(cfg.n_layers):
        layers.append({
            "rms_att_weight": (0.02 * rng.standard_normal(cfg.dim)).astype(np.float32),
            "wq": (0.02 * rng.standard_normal((cfg.dim, cfg.dim))).astype(np.float32),
            "wkv": (0.02 * rng.standard_normal((2 * cfg.kv_dim, cfg.dim))).astype(np.float32),
            "wo": (0.02 * rng.standard_normal((cfg.dim, cfg.dim))).astype(np.float32),
            "rms_ffn_weight": (0.02 * rng.standard_normal(cfg.dim)).astype(np.float32),
            "w1": (0.02 * rng.standard_normal((cfg.hidden_dim, cfg.dim))).astype(np.float32),
            "w2": (0.02 * rng.standard_normal((cfg.dim, cfg.hidden_dim))).astype(np.float32),
            "w3": (0.02 * rng.standard_normal((cfg.hidden_dim, cfg.dim))).astype(np.float32),
        })
    base = {
        "token_embedding_table": (0.02 * rng.standard_normal((cfg.vocab_size, cfg.dim))).astype(np.float32),
        "rms_final_weight": (0.02 * rng.standard_normal(cfg.dim)).astype(np.float32),
    }
    base["wcls"] = base["token_embedding_table"]
    base["freq_cis_real"], base["freq_cis_imag"] = O.rope_tables(cfg.seq_len, cfg.head_size)

    batch, n_prompt = 4, 8
    st = S.Stage(name, "f32", 0, cfg.n_layers, batch, batch, with_cls=True)
    load_weights(st, cfg, layers, base, False)
    ref = OracleModel(cfg, layers, base)
    prompts = rng.integers(0, cfg.vocab_size, (batch, n_prompt))
    st.new_state(batch)
    for i in range(batch):
        st.set_prompt(i, i, int(prompts[i, 0]), 0, 0.0, n_prompt, cfg.seq_len)
    tokens = prompts[:, 0].tolist()
    agree = clear = 0
    worst = 0.0
    for pos in range(cfg.seq_len):
        want = ref.step(tokens, list(range(batch)), [pos] * batch)
        assert st.forward()
        got = d2h(st.scratch_ptr("logits"), (batch, cfg.vocab_size), np.float32)
        a, r = errors(got, want)
        worst = max(worst, r)
        assert a <= 2e-2 and r <= 1e-3, f"position {pos}: max_abs {a:.2e} mean_rel {r:.2e}"
        nxt = []
        for i in range(batch):
            row = st.row(i)
            assert row["token_pos"] == pos + 1
            top2 = np.sort(want[i])[-2:]
            if top2[1] - top2[0] > 1e-4:           # logits here are ~1e-3 in size; the margin is scaled to that
                clear += 1
                agree += int(row["token"] == int(np.argmax(want[i])))
            # prompt tokens are forced while inside the prompt (frontend/infer.cc:124-125), then greedy
            t = int(prompts[i, pos + 1]) if pos + 1 < n_prompt else row["token"]
            nxt.append(t)
            if pos + 1 < n_prompt:
                st.set_prompt(i, i, t, pos + 1, 0.0, n_prompt, cfg.seq_len)
        tokens = nxt
    assert all(st.row(i)["finished"] for i in range(batch))          # token_pos reached seq_len
    assert clear > 200 and agree == clear, (agree, clear)
    st.close()


def test_config2_llama7b_shape_two_layers():
    cfg = O.Config(dim=4096, n_layers=32, n_heads=32, n_kv_heads=32, hidden_dim=11008, seq_len=2048, attention_rounds=2)
    batch, prefill = 32, 1024
    first, hosted = 8, 2
    rng = np.random.default_rng(2)
    st = S.Stage("llama2-7b", "f16", first, hosted, batch, batch, seed=3, weight_std=0.02)
    # weights as the configuration says (N(0, 0.02)) except the two norm gains, which are kept near 1
    # so that activations do not collapse to ~1e-3 and the comparison stays meaningful
    layers = {}
    for l in range(first, first + hosted):
        lw = {
            "rms_att_weight": (1 + 0.02 * rng.standard_normal(cfg.dim)).astype(np.float16),
            "wq": (0.02 * rng.standard_normal((cfg.dim, cfg.dim))).astype(np.float16),
            "wkv": (0.02 * rng.standard_normal((2 * cfg.kv_dim, cfg.dim))).astype(np.float16),
            "wo": (0.02 * rng.standard_normal((cfg.dim, cfg.dim))).astype(np.float16),
            "rms_ffn_weight": (1 + 0.02 * rng.standard_normal(cfg.dim)).astype(np.float16),
            "w1": (0.02 * rng.standard_normal((cfg.hidden_dim, cfg.dim))).astype(np.float16),
            "w2": (0.02 * rng.standard_normal((cfg.dim, cfg.hidden_dim))).astype(np.float16),
            "w3": (0.02 * rng.standard_normal((cfg.hidden_dim, cfg.dim))).astype(np.float16),
        }
        layers[l] = lw
        for k, v in lw.items():
            st.set_layer_tensor(l, k, v)
    re, im = O.rope_tables(cfg.seq_len, cfg.head_size)
    st.set_base_tensor("freq_cis_real", re.astype(np.float16))
    st.set_base_tensor("freq_cis_imag", im.astype(np.float16))

    st.new_state(batch, next_layer=first)
    for i in range(batch):
        st.set_prompt(i, i, 1, prefill)
    assert st.acquire_contexts()
    # pre-fill every context with N(0,1) rows; the oracle gets the same values as fp32
    kv_host, kv_half = {}, {}
    for l in range(first, first + hosted):
        kv = rng.standard_normal((batch, cfg.seq_len, 2 * cfg.kv_dim)).astype(np.float16)
        kv[:, prefill + 8:] = 0
        kv_host[l] = kv.astype(np.float32)
        kv_half[l] = kv.copy()
        for i in range(batch):
            h2d(st.context_layer_ptr(i, l), kv[i])
    w32 = {l: {k: v.astype(np.float32) for k, v in lw.items()} for l, lw in layers.items()}
    re16, im16 = re.astype(np.float16).astype(np.float32), im.astype(np.float16).astype(np.float32)

    for step in range(3):
        pos = prefill + step
        x = rng.standard_normal((batch, cfg.dim)).astype(np.float16)
        st.new_state(batch, next_layer=first)
        for i in range(batch):
            st.set_prompt(i, i, 1, pos)
        st.activations(allocate=True)[:] = x.reshape(-1)
        assert st.forward()
        got = st.activations().reshape(batch, cfg.dim).astype(np.float32)
        want = x.astype(np.float32)
        want16 = x.copy()
        for l in range(first, first + hosted):
            O.layer_forward(cfg, w32[l], re16, im16, want, [kv_host[l][i] for i in range(batch)], [pos] * batch)
            O.layer_forward(cfg, layers[l], re.astype(np.float16), im.astype(np.float16), want16, [kv_half[l][i] for i in range(batch)], [pos] * batch)
        # stage output = residual stream after two layers, against the CPU path in both storage types
        assert_half_parity(got, want16, want, what=f"7B-shape stage output step {step}")
    st.close()


def test_config5_slot_churn_reduced_shape():
    """256-slot churn of configuration 5 at a reduced shape (GQA 4, head 128, 3 layers, 320
    positions, 16 slots): ragged lengths, 10 % of the slots finish per step and are refilled under
    the same context id with a fresh prompt that is fed token by token from position 0."""
    name, dtype = "test-gqa4", "f16"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=21, wcls=True)
    n_slots = 16
    st = S.Stage(name, dtype, 0, cfg.n_layers, n_slots, n_slots, with_cls=True)
    load_weights(st, cfg, layers, base, True)
    ref = OracleModel(cfg, layers, base)
    ref16 = OracleModel(cfg, layers, base, np.float16)
    rng = np.random.default_rng(22)

    # ragged start: every slot is first driven to a random length with random tokens (prefill, token by token)
    target = rng.integers(2, 40, n_slots)
    st.new_state(n_slots)
    pos = np.zeros(n_slots, int)
    tokens = rng.integers(0, cfg.vocab_size, n_slots).tolist()
    for i in range(n_slots):
        st.set_prompt(i, 500 + i, tokens[i], 0, 0.0, int(target[i]), 0)
    restarts = 0
    for step in range(70):
        cids = [500 + i for i in range(n_slots)]
        want = ref.step(tokens, cids, pos.tolist())
        want16 = ref16.step(tokens, cids, pos.tolist())
        assert st.forward()
        assert [st.context_slot(i) for i in range(n_slots)] == list(range(n_slots))     # sticky slots, never re-assigned
        got = d2h(st.scratch_ptr("logits"), (n_slots, cfg.vocab_size), np.float16).astype(np.float32)
        assert_half_parity(got, want16, want, what=f"churn (reduced shape) logits step {step}")
        evict = rng.random(n_slots) < 0.10
        for i in range(n_slots):
            row = st.row(i)
            pos[i] += 1
            assert row["token_pos"] == pos[i]
            if evict[i] or pos[i] >= cfg.seq_len - 1:
                # finished: the slot is refilled in place, position 0 (the old rows are simply overwritten)
                restarts += 1
                pos[i] = 0
                tokens[i] = int(rng.integers(0, cfg.vocab_size))
                target[i] = int(rng.integers(2, 40))
                ref.cache.pop(500 + i, None)
                ref16.cache.pop(500 + i, None)
                st.set_prompt(i, 500 + i, tokens[i], 0, 0.0, int(target[i]), 0)
            elif pos[i] < target[i]:
                tokens[i] = int(rng.integers(0, cfg.vocab_size))         # still inside its prompt: forced token
                st.set_prompt(i, 500 + i, tokens[i], int(pos[i]), 0.0, int(target[i]), 0)
            else:
                tokens[i] = row["token"]
    assert restarts > 40
    assert st.slot_counts() == dict(free=0, allocated=n_slots, total=n_slots)
    st.close()
