"""The on-disk model directory (reference: tools/bin2glint.py:45-86 writes it, models/llama2/model.hh:
180-270 and base.hh:216-282,357-400,477-530 read it): file names, tensor order, byte offsets, which
tensors a node copies, and the loader's refusals.  Host only, no GPU."""
import os
import struct
from types import SimpleNamespace

import numpy as np
import pytest

from glinthawk_amd import modeldir, stage as S
from glinthawk_amd._lib import GlintError

TINY = SimpleNamespace(dim=32, n_layers=2, n_heads=4, n_kv_heads=2, hidden_dim=48, seq_len=16, vocab_size=32000)     # "test-tiny", wcls
GQA4 = SimpleNamespace(dim=1024, n_layers=3, n_heads=8, n_kv_heads=2, hidden_dim=1536, seq_len=320, vocab_size=32000)  # "test-gqa4", wcls
STORIES = SimpleNamespace(dim=288, n_layers=6, n_heads=6, n_kv_heads=6, hidden_dim=768, seq_len=256, vocab_size=32000)  # no wcls


def kv_dim(c):
    return c.dim // (c.n_heads // c.n_kv_heads)


def zeros_model(c, dt, wcls):
    hs = c.dim // c.n_heads
    layers = [dict(rms_att_weight=np.zeros(c.dim, dt), wq=np.zeros((c.dim, c.dim), dt), wkv=np.zeros((2 * kv_dim(c), c.dim), dt),
                   wo=np.zeros((c.dim, c.dim), dt), rms_ffn_weight=np.zeros(c.dim, dt), w1=np.zeros((c.hidden_dim, c.dim), dt),
                   w2=np.zeros((c.dim, c.hidden_dim), dt), w3=np.zeros((c.hidden_dim, c.dim), dt)) for _ in range(c.n_layers)]
    base = dict(token_embedding_table=np.zeros((c.vocab_size, c.dim), dt), rms_final_weight=np.zeros(c.dim, dt),
                freq_cis_real=np.zeros((c.seq_len, hs // 2), dt), freq_cis_imag=np.zeros((c.seq_len, hs // 2), dt))
    if wcls:
        base["wcls"] = np.zeros((c.vocab_size, c.dim), dt)
    return layers, base


# sizes in the order of the files, straight from the converter's serialize() calls
def layer_sizes(c):
    return [("rms_att_weight", c.dim), ("wq", c.dim * c.dim), ("wkv", 2 * kv_dim(c) * c.dim), ("wo", c.dim * c.dim),
            ("rms_ffn_weight", c.dim), ("w1", c.dim * c.hidden_dim), ("w2", c.dim * c.hidden_dim), ("w3", c.dim * c.hidden_dim)]


def base_sizes(c, wcls):
    hs = c.dim // c.n_heads
    out = [("token_embedding_table", c.vocab_size * c.dim), ("rms_final_weight", c.dim), ("freq_cis_real", c.seq_len * hs // 2),
           ("freq_cis_imag", c.seq_len * hs // 2)]
    return out + ([("wcls", c.vocab_size * c.dim)] if wcls else [])


def offsets(sizes, item):
    off, out = 0, {}
    for name, n in sizes:
        out[name] = (off * item, n)
        off += n
    return out, off * item


def test_config_file_bytes(tmp_path):
    modeldir.write_config(str(tmp_path), 288, 768, 6, 6, 6, 32000, 256, wcls_present=False)
    raw = open(tmp_path / "CONFIG", "rb").read()
    assert raw == struct.pack("<7i", 288, 768, 6, 6, 6, 32000, 256) and len(raw) == 28
    modeldir.write_config(str(tmp_path), 32, 48, 2, 4, 2, 32000, 16, wcls_present=True)
    assert struct.unpack("<7i", open(tmp_path / "CONFIG", "rb").read())[5] == -32000


@pytest.mark.parametrize("name,c,wcls,dtype", [("test-tiny", TINY, True, "f16"), ("test-tiny", TINY, True, "f32"),
                                               ("stories15m", STORIES, False, "f32"), ("test-gqa4", GQA4, True, "f16")])
def test_whole_model_offsets_and_sizes(tmp_path, name, c, wcls, dtype):
    dt = np.float16 if dtype == "f16" else np.float32
    layers, base = zeros_model(c, dt, wcls)
    modeldir.write_model_dir(str(tmp_path), c, layers, base, dt, wcls)
    item = np.dtype(dt).itemsize
    lo, lbytes = offsets(layer_sizes(c), item)
    bo, bbytes = offsets(base_sizes(c, wcls), item)
    text = "FP16" if dtype == "f16" else "FP32"
    assert os.path.getsize(tmp_path / f"BASEWEIGHTS_{text}") == bbytes
    for i in range(c.n_layers):
        assert os.path.getsize(tmp_path / f"LAYER{i}_{text}") == lbytes

    recs = S.model_dir_walk(name, dtype, 0, c.n_layers, True, str(tmp_path))
    got_base = {r["tensor"]: (r["offset"], r["elements"]) for r in recs if r["is_base"]}
    assert got_base == bo                                      # everything resident, shared classifier is not a tensor of its own
    for i in range(c.n_layers):
        got = {r["tensor"]: (r["offset"], r["elements"]) for r in recs if not r["is_base"] and r["layer"] == i}
        assert got == lo


def test_partial_stage_copies_only_what_it_hosts(tmp_path):
    c, dt = GQA4, np.float16
    layers, base = zeros_model(c, dt, True)
    modeldir.write_model_dir(str(tmp_path), c, layers, base, dt, True)
    recs = S.model_dir_walk("test-gqa4", "f16", 1, 2, False, str(tmp_path))      # layers 1..2, no classifier
    # attention hosted -> only the RoPE tables out of the base file; no embedding (layer 0 is elsewhere), no classifier
    assert sorted(r["tensor"] for r in recs if r["is_base"]) == ["freq_cis_imag", "freq_cis_real"]
    assert sorted({r["layer"] for r in recs if not r["is_base"]}) == [1, 2]
    # with the classifier: final norm and wcls too, still no embedding because this model has its own wcls
    recs = S.model_dir_walk("test-gqa4", "f16", 1, 2, True, str(tmp_path))
    assert sorted(r["tensor"] for r in recs if r["is_base"]) == ["freq_cis_imag", "freq_cis_real", "rms_final_weight", "wcls"]
    # first stage: the embedding, no classifier tensors
    recs = S.model_dir_walk("test-gqa4", "f16", 0, 1, False, str(tmp_path))
    assert sorted(r["tensor"] for r in recs if r["is_base"]) == ["freq_cis_imag", "freq_cis_real", "token_embedding_table"]


def test_shared_classifier_keeps_the_embedding_on_the_last_stage(tmp_path):
    c, dt = STORIES, np.float32
    layers, base = zeros_model(c, dt, False)
    modeldir.write_model_dir(str(tmp_path), c, layers, base, dt, False)
    recs = S.model_dir_walk("stories15m", "f32", 4, 2, True, str(tmp_path))
    assert sorted(r["tensor"] for r in recs if r["is_base"]) == ["freq_cis_imag", "freq_cis_real", "rms_final_weight", "token_embedding_table"]


def test_files_of_other_layers_are_not_needed(tmp_path):
    c, dt = GQA4, np.float16
    layers, base = zeros_model(c, dt, True)
    modeldir.write_model_dir(str(tmp_path), c, layers, base, dt, True, only_layers=[1, 2])
    assert len(S.model_dir_walk("test-gqa4", "f16", 1, 2, False, str(tmp_path))) == 2 + 16
    with pytest.raises(GlintError, match="LAYER0_FP16"):
        S.model_dir_walk("test-gqa4", "f16", 0, 2, False, str(tmp_path))


def test_refusals(tmp_path):
    c, dt = TINY, np.float16
    layers, base = zeros_model(c, dt, True)
    d = str(tmp_path)
    with pytest.raises(GlintError, match="config file"):
        S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)                       # no CONFIG at all
    modeldir.write_model_dir(d, c, layers, base, dt, True)
    S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)
    with pytest.raises(GlintError, match="BASEWEIGHTS_FP32"):
        S.model_dir_walk("test-tiny", "f32", 0, 2, True, d)                       # the other dtype's files are absent
    with open(tmp_path / "LAYER1_FP16", "ab") as f:
        f.write(b"\0\0")
    with pytest.raises(GlintError, match="LAYER1_FP16 is not the expected size"):
        S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)
    open(tmp_path / "CONFIG", "wb").write(b"\0" * 27)
    with pytest.raises(GlintError, match="failed to read config file"):
        S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)
    fields = dict(dim=c.dim, hidden_dim=c.hidden_dim, n_layers=c.n_layers, n_heads=c.n_heads, n_kv_heads=c.n_kv_heads,
                  vocab_size=c.vocab_size, seq_len=c.seq_len)
    for bad, what in [("dim", "dim"), ("hidden_dim", "hidden_dim"), ("n_layers", "n_layers"), ("seq_len", "seq_len"), ("vocab_size", "vocab_size")]:
        f = dict(fields)
        f[bad] += 64
        modeldir.write_config(d, wcls_present=True, **f)
        with pytest.raises(GlintError, match=what + " does not match"):
            S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)
    modeldir.write_config(d, wcls_present=False, **fields)                       # positive vocabulary: no separate classifier
    with pytest.raises(GlintError, match="wcls_present does not match"):
        S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)
    f = dict(fields, n_kv_heads=4)                                               # MHA instead of GQA 2: kv_dim differs
    modeldir.write_config(d, wcls_present=True, **f)
    with pytest.raises(GlintError, match="kv_dim does not match"):
        S.model_dir_walk("test-tiny", "f16", 0, 2, True, d)
    with pytest.raises(GlintError, match="unknown configuration"):
        S.model_dir_walk("no-such-model", "f16", 0, 2, True, d)
