"""Stage.load(): weights read from a model directory in the reference's format give the same
logits, bit for bit, as the same weights handed over tensor by tensor, and match the oracle."""
import numpy as np
import pytest

from glinthawk_amd import modeldir, stage as S
from helpers import assert_close, assert_half_parity
from test_gpu_stage import SHAPES, WCLS, OracleModel, d2h, load_weights, make_weights

pytestmark = pytest.mark.gpu


def run_steps(st, cfg, batch, tokens, np_dt, steps=3):
    out = []
    toks = list(tokens)
    st.new_state(batch)
    for pos in range(steps):
        for i in range(batch):
            st.set_prompt(i, 40 + i, int(toks[i]), pos)
        assert st.forward()
        out.append(d2h(st.scratch_ptr("logits"), (batch, cfg.vocab_size), np_dt).copy())
        toks = [st.row(i)["token"] for i in range(batch)]
    return out


@pytest.mark.parametrize("name,dtype", [("stories15m", "f32"), ("test-gqa4", "f16"), ("test-tiny", "f16")])
def test_loaded_stage_equals_tensor_by_tensor(tmp_path, name, dtype):
    cfg = SHAPES[name]
    np_dt = np.float16 if dtype == "f16" else np.float32
    wcls = WCLS[name]
    layers, base = make_weights(cfg, np_dt, seed=61, wcls=wcls)
    modeldir.write_model_dir(str(tmp_path), cfg, layers, base, np_dt, wcls)
    batch = 3
    a = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True)
    b = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True)
    a.load(str(tmp_path))
    load_weights(b, cfg, layers, base, wcls)
    tokens = np.random.default_rng(62).integers(0, cfg.vocab_size, batch)
    la = run_steps(a, cfg, batch, tokens, np_dt)
    lb = run_steps(b, cfg, batch, tokens, np_dt)
    for x, y in zip(la, lb):
        assert np.array_equal(x, y)
    ref = OracleModel(cfg, layers, base)
    want = ref.step(tokens.tolist(), [40 + i for i in range(batch)], [0] * batch)
    if dtype == "f16":
        want16 = OracleModel(cfg, layers, base, np.float16).step(tokens.tolist(), [40 + i for i in range(batch)], [0] * batch)
        assert_half_parity(la[0].astype(np.float32), want16, want, what=f"{name} logits from loaded weights",
                           mean_rel32=3e-3 if name == "test-tiny" else 2e-3)
    else:
        assert_close(la[0].astype(np.float32), want, mean_rel=1e-3, what=f"{name} logits from loaded weights")
    a.close()
    b.close()


def test_middle_stage_loads_its_slice(tmp_path):
    name, dtype, np_dt = "test-gqa4", "f16", np.float16
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np_dt, seed=63, wcls=True)
    modeldir.write_model_dir(str(tmp_path), cfg, layers, base, np_dt, True, only_layers=[1, 2])
    batch = 2
    a = S.Stage(name, dtype, 1, 2, batch, batch)
    b = S.Stage(name, dtype, 1, 2, batch, batch)
    a.load(str(tmp_path))
    load_weights(b, cfg, layers, base, True, layer_range=[1, 2], with_embedding=False, with_cls=False)
    x = np.random.default_rng(64).standard_normal((batch, cfg.dim)).astype(np_dt)
    outs = []
    for st in (a, b):
        st.new_state(batch, next_layer=1)
        for i in range(batch):
            st.set_prompt(i, 5 + i, 1, 0)
        st.activations(allocate=True)[:] = x.reshape(-1)
        assert st.forward()
        outs.append(st.activations().copy())
    assert np.array_equal(outs[0], outs[1])
    a.close()
    b.close()


def test_load_reports_a_wrong_directory(tmp_path):
    from glinthawk_amd._lib import GlintError
    st = S.Stage("test-tiny", "f16", 0, 2, 1, 1)
    with pytest.raises(GlintError, match="config file"):
        st.load(str(tmp_path))
    st.close()
