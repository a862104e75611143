"""A stage fed with, and emitting, states in the reference's wire format behaves exactly like the
same stage driven field by field."""
import numpy as np
import pytest

from glinthawk_amd import stage as S, wire
from glinthawk_amd._lib import GlintError
from test_gpu_stage import SHAPES, WCLS, load_weights, make_weights

pytestmark = pytest.mark.gpu


def prompts_for(batch, cids, tokens, pos, plen=64, mcl=0):
    p = wire.new_prompts(batch)
    p["active"] = 1
    p["context_id"], p["token"], p["token_pos"] = cids, tokens, pos
    p["prompt_length"], p["max_completion_length"] = plen, mcl
    p["kv_tier"] = 0
    p["prompt_id"] = np.arange(batch * 32, dtype=np.uint8).reshape(batch, 32)
    return p


def test_whole_model_stage_over_the_wire():
    name, dtype, np_dt = "test-gqa4", "f16", np.float16
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np_dt, seed=81, wcls=WCLS[name])
    batch = 3
    a = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True)
    b = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True)
    for st in (a, b):
        load_weights(st, cfg, layers, base, WCLS[name])
    cids = [21, 22, 23]
    tokens = [5, 600, 31000]
    meta = dict(id=4242, dtype=wire.DTYPE_CODE[dtype], route_id=7, model_id=1, next_layer=0, next_stage=S.STAGE_PRE)
    for pos in range(4):
        a.new_state(batch)
        for i in range(batch):
            a.set_prompt(i, cids[i], tokens[i], pos, 0.0, 64, 0)
        assert a.forward()
        b.set_state_bytes(wire.pack_state(meta, prompts_for(batch, cids, tokens, pos)))
        assert b.forward()
        m, p, acts, q, kv = wire.unpack_state(b.get_state_bytes(), cfg.dim, cfg.kv_dim)
        # identity travels untouched; the classifier wrote the next token and advanced the position
        assert int(m["id"]) == 4242 and int(m["route_id"]) == 7 and int(m["model_id"]) == 1
        sa = a.state()
        assert int(m["next_layer"]) == sa["next_layer"] and int(m["next_stage"]) == sa["next_stage"]
        assert np.array_equal(p["prompt_id"], np.arange(batch * 32, dtype=np.uint8).reshape(batch, 32))
        for i in range(batch):
            ra = a.row(i)
            assert (int(p[i]["token"]), int(p[i]["token_pos"]), bool(p[i]["finished"])) == (ra["token"], ra["token_pos"], bool(ra["finished"]))
            assert int(p[i]["context_id"]) == cids[i]
        tokens = [int(t) for t in p["token"]]
    a.close()
    b.close()


def test_middle_stage_carries_activations_over_the_wire():
    name, dtype, np_dt = "test-gqa4", "f16", np.float16
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np_dt, seed=82, wcls=True)
    batch = 2
    a = S.Stage(name, dtype, 1, 2, batch, batch)
    b = S.Stage(name, dtype, 1, 2, batch, batch)
    for st in (a, b):
        load_weights(st, cfg, layers, base, True, layer_range=[1, 2], with_embedding=False, with_cls=False)
    x = np.random.default_rng(83).standard_normal((batch, cfg.dim)).astype(np_dt)
    a.new_state(batch, next_layer=1)
    for i in range(batch):
        a.set_prompt(i, 30 + i, 9, 0)
    a.activations(allocate=True)[:] = x.reshape(-1)
    assert a.forward()
    meta = dict(id=1, dtype=wire.DTYPE_CODE[dtype], next_layer=1, next_stage=S.STAGE_PRE)
    b.set_state_bytes(wire.pack_state(meta, prompts_for(batch, [30, 31], [9, 9], [0, 0]), activations=x))
    assert b.forward()
    m, p, acts, q, kv = wire.unpack_state(b.get_state_bytes(), cfg.dim, cfg.kv_dim)
    assert acts is not None and np.array_equal(acts.reshape(-1), a.activations())
    assert int(m["next_layer"]) == a.state()["next_layer"] and int(m["next_stage"]) == a.state()["next_stage"]
    # a state of the wrong width is refused, the stage keeps its own
    before = b.get_state_bytes()
    with pytest.raises(GlintError):
        b.set_state_bytes(before[:-2])
    with pytest.raises(GlintError, match="data type"):
        b.set_state_bytes(wire.pack_state(dict(meta, dtype=wire.DTYPE_CODE["f32"]), prompts_for(batch, [30, 31], [9, 9], [1, 1])))
    assert b.get_state_bytes() == before
    a.close()
    b.close()
