"""ctypes/numpy front-end of the CPU oracle (``libglint_oracle.so``).

TEST INFRASTRUCTURE ONLY.  This package restates the reference's amd64/OpenMP path on the CPU and
exists to *check* the HIP path (tests, the smoke check) and to be *timed beside it* (the
benchmark's ``cpu_baseline`` leg).  Product code under ``glinthawk_amd/`` never imports it.

Arrays are numpy; ``float32`` arrays select the reference's ``DType = float`` instantiation and
``float16`` arrays the ``DType = _Float16`` one.  A KV context is a numpy array of shape
``(n_hosted_layers, seq_len, 2 * kv_dim)`` (token-major ``[K | V]`` rows, the layout of
``models/llama2/context.hh:61-190``); ``None`` stands for the reference's empty context.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# GLINT_ORACLE_LIB: another build of the same source (the sanitizer build of the CPU test suite)
_LIB_PATH = os.environ.get("GLINT_ORACLE_LIB") or os.path.join(_HERE, "libglint_oracle.so")


def build(force: bool = False) -> str:
    """Compile the C restatement with the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class GoConfig(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "dim", "kv_dim", "hidden_dim", "n_layers", "head_size", "n_heads", "n_kv_heads",
        "gqa_size", "vocab_size", "seq_len", "attention_rounds")]


@dataclass(frozen=True)
class Config:
    """Shape of a Llama2 variant (``models/llama2/variants.hh``)."""
    dim: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    hidden_dim: int
    seq_len: int
    vocab_size: int = 32000
    attention_rounds: int = 1

    @property
    def head_size(self) -> int:
        return self.dim // self.n_heads

    @property
    def gqa_size(self) -> int:
        return self.n_heads // self.n_kv_heads

    @property
    def kv_dim(self) -> int:
        return self.dim // self.gqa_size

    def c(self) -> GoConfig:
        return GoConfig(self.dim, self.kv_dim, self.hidden_dim, self.n_layers, self.head_size,
                        self.n_heads, self.n_kv_heads, self.gqa_size, self.vocab_size,
                        self.seq_len, self.attention_rounds)


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(L: C.CDLL) -> None:
    u64, u32p, vp, f = C.c_uint64, C.POINTER(C.c_uint32), C.c_void_p, C.c_float
    cfgp = C.POINTER(GoConfig)
    L.go_half_to_float.restype = f
    L.go_half_to_float.argtypes = [C.c_uint16]
    L.go_float_to_half.restype = C.c_uint16
    L.go_float_to_half.argtypes = [f]
    L.go_convert_f16_to_f32.argtypes = [vp, vp, u64]
    L.go_convert_f32_to_f16.argtypes = [vp, vp, u64]
    for sfx in ("f32", "f16"):
        getattr(L, f"go_accum_{sfx}").argtypes = [vp, vp, u64, u64]
        getattr(L, f"go_rmsnorm_{sfx}").argtypes = [vp, vp, vp, u64, u64]
        getattr(L, f"go_argmax_{sfx}").argtypes = [vp, vp, u64, u64]
        getattr(L, f"go_silu_{sfx}").argtypes = [vp, vp, u64, u64]
        getattr(L, f"go_matmul_{sfx}").argtypes = [vp, vp, vp, u64, u64, u64]
        getattr(L, f"go_gumbel_{sfx}").argtypes = [vp, vp, vp, u64, u64]
        getattr(L, f"go_copy_kv_cache_{sfx}").argtypes = [cfgp, vp, vp, u64]
        getattr(L, f"go_apply_rope_{sfx}").argtypes = [cfgp, u64, vp, vp, vp, vp, vp]
        getattr(L, f"go_attention_0_gemm_{sfx}").argtypes = [cfgp, vp, vp, vp, u64, vp]
        getattr(L, f"go_attention_softmax_{sfx}").argtypes = [cfgp, vp, vp, u64]
        getattr(L, f"go_attention_2_gemm_{sfx}").argtypes = [cfgp, vp, vp, vp, u64, vp]
        getattr(L, f"go_softmax_row_{sfx}").argtypes = [vp, u64]
        getattr(L, f"go_attention_ops_{sfx}").argtypes = [cfgp, u64, vp, vp, vp, vp, vp, vp, vp]
    L.go_rope_tables_f32.argtypes = [vp, vp, u64, u64, f]
    for sfx in ("f32", "f16"):
        getattr(L, f"go_layer_forward_{sfx}").argtypes = [cfgp, vp, vp, vp, vp, vp, vp, u64]
        getattr(L, f"go_classify_{sfx}").argtypes = [cfgp, vp, vp, vp, vp, u64]
    for name in ("go_ctx_layer_offset", "go_ctx_token_offset", "go_ctx_key_head_offset",
                 "go_ctx_value_head_offset", "go_ctx_max_size_bytes", "go_dynctx_prepare",
                 "go_ctxman_free", "go_ctxman_allocated"):
        getattr(L, name).restype = u64
    L.go_ctx_layer_offset.argtypes = [cfgp, vp, u64]
    L.go_ctx_token_offset.argtypes = [cfgp, vp, u64, u64]
    L.go_ctx_key_head_offset.argtypes = [cfgp, vp, u64, u64, u64]
    L.go_ctx_value_head_offset.argtypes = [cfgp, vp, u64, u64, u64]
    L.go_ctx_max_size_bytes.argtypes = [cfgp, u64, u64]
    L.go_dynctx_prepare.argtypes = [cfgp, u64, vp, u64, u64, C.c_int, C.c_int, C.POINTER(C.c_int)]
    L.go_ctxman_new.restype = vp
    L.go_ctxman_new.argtypes = [u64]
    L.go_ctxman_delete.argtypes = [vp]
    L.go_ctxman_free.argtypes = [vp]
    L.go_ctxman_allocated.argtypes = [vp]
    L.go_ctxman_get_contexts.restype = C.c_int
    L.go_ctxman_get_contexts.argtypes = [vp, vp, vp, u64, u64, vp]
    L.go_ctxman_get_context.restype = C.c_int32
    L.go_ctxman_get_context.argtypes = [vp, C.c_uint32]
    L.go_ctxman_release.restype = C.c_int
    L.go_ctxman_release.argtypes = [vp, C.c_uint32]
    L.go_check_finished.restype = C.c_int
    L.go_check_finished.argtypes = [C.c_uint32] * 6 + [u64]
    L.go_encode_temperature.restype = C.c_uint8
    L.go_encode_temperature.argtypes = [f]
    L.go_decode_temperature.restype = f
    L.go_decode_temperature.argtypes = [C.c_uint8]
    L.go_num_threads.restype = C.c_int


# --------------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------------
def _sfx(a: np.ndarray) -> str:
    if a.dtype == np.float32:
        return "f32"
    if a.dtype == np.float16:
        return "f16"
    raise TypeError(f"oracle supports float32/float16 storage, got {a.dtype}")


def _p(a: Optional[np.ndarray]) -> Optional[int]:
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return a.ctypes.data


def _fn(name: str, a: np.ndarray):
    return getattr(lib(), f"{name}_{_sfx(a)}")


def _ptr_table(rows: Sequence[Optional[np.ndarray]]) -> "C.Array":
    tbl = (C.c_void_p * max(1, len(rows)))()
    for i, r in enumerate(rows):
        tbl[i] = None if r is None else r.ctypes.data
    return tbl


def _pos(token_positions) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(token_positions, dtype=np.uint32))


def num_threads() -> int:
    return int(lib().go_num_threads())


# --------------------------------------------------------------------------------------------
# common ops (arch/amd64/common/ops.hh)
# --------------------------------------------------------------------------------------------
def convert(src: np.ndarray, dst_dtype) -> np.ndarray:
    """convert_and_copy (arch/amd64/llama2/ops.hh:354-368): element-wise static_cast between float32 and float16
    storage; the same type is a plain copy."""
    src = np.ascontiguousarray(src)
    dst_dtype = np.dtype(dst_dtype)
    if src.dtype == dst_dtype:
        return src.copy()
    out = np.empty(src.shape, dtype=dst_dtype)
    if src.dtype == np.float16 and dst_dtype == np.float32:
        lib().go_convert_f16_to_f32(out.ctypes.data, src.ctypes.data, src.size)
    elif src.dtype == np.float32 and dst_dtype == np.float16:
        lib().go_convert_f32_to_f16(out.ctypes.data, src.ctypes.data, src.size)
    else:
        raise TypeError(f"oracle converts between float32 and float16, got {src.dtype} -> {dst_dtype}")
    return out


def accum(a: np.ndarray, b: np.ndarray) -> None:
    """In place ``a += b`` over a (batch, size) array."""
    batch, size = a.shape
    _fn("go_accum", a)(_p(a), _p(b), size, batch)


def rmsnorm(x: np.ndarray, weight: np.ndarray, out: Optional[np.ndarray] = None) -> np.ndarray:
    batch, size = x.shape
    out = np.empty_like(x) if out is None else out
    _fn("go_rmsnorm", x)(_p(out), _p(x), _p(weight), size, batch)
    return out


def argmax(v: np.ndarray) -> np.ndarray:
    batch, n = v.shape
    out = np.empty(batch, dtype=np.uint32)
    _fn("go_argmax", v)(_p(out), _p(v), n, batch)
    return out


def silu(hb: np.ndarray, hb2: np.ndarray) -> None:
    """In place ``hb = silu(hb) * hb2``."""
    batch, hidden = hb.shape
    _fn("go_silu", hb)(_p(hb), _p(hb2), hidden, batch)


def matmul(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """``x (b, s)``, ``w (r, s)`` -> ``(b, r)``."""
    b, s = x.shape
    r, s2 = w.shape
    assert s == s2
    out = np.empty((b, r), dtype=x.dtype)
    _fn("go_matmul", x)(_p(out), _p(x), _p(w), s, r, b)
    return out


def gumbel(v: np.ndarray, uniforms: np.ndarray, temperatures: np.ndarray) -> None:
    batch, vocab = v.shape
    u = np.ascontiguousarray(uniforms, dtype=np.float32)
    t = np.ascontiguousarray(temperatures, dtype=np.float32)
    _fn("go_gumbel", v)(_p(v), _p(u), _p(t), vocab, batch)


# --------------------------------------------------------------------------------------------
# llama2 ops (arch/amd64/llama2/ops.hh)
# --------------------------------------------------------------------------------------------
def copy_kv_cache(cfg: Config, token_rows: Sequence[Optional[np.ndarray]], state_kv: np.ndarray) -> None:
    """``token_rows[i]``: view of the (2*kv_dim,) cache row of context i, or None (empty)."""
    c = cfg.c()
    tbl = _ptr_table(token_rows)
    _fn("go_copy_kv_cache", state_kv)(C.byref(c), tbl, _p(state_kv), len(token_rows))


def apply_rope(cfg: Config, token_positions, freq_real: np.ndarray, freq_imag: np.ndarray,
               q: np.ndarray, token_rows: Sequence[Optional[np.ndarray]]) -> None:
    c = cfg.c()
    pos = _pos(token_positions)
    tbl = _ptr_table(token_rows)
    _fn("go_apply_rope", q)(C.byref(c), len(token_rows), _p(pos), _p(freq_real), _p(freq_imag),
                            _p(q), tbl)


def attention_0_gemm(cfg: Config, q: np.ndarray, layers: Sequence[Optional[np.ndarray]],
                     att: np.ndarray, token_positions) -> None:
    """``layers[i]``: (seq_len, 2*kv_dim) rows of context i for the current layer, or None."""
    c = cfg.c()
    pos = _pos(token_positions)
    _fn("go_attention_0_gemm", q)(C.byref(c), _p(q), _ptr_table(layers), _p(att), len(layers), _p(pos))


def attention_softmax(cfg: Config, att: np.ndarray, token_positions) -> None:
    c = cfg.c()
    pos = _pos(token_positions)
    _fn("go_attention_softmax", att)(C.byref(c), _p(att), _p(pos), len(pos))


def attention_2_gemm(cfg: Config, att: np.ndarray, layers: Sequence[Optional[np.ndarray]],
                     xb: np.ndarray, token_positions) -> None:
    c = cfg.c()
    pos = _pos(token_positions)
    _fn("go_attention_2_gemm", att)(C.byref(c), _p(att), _ptr_table(layers), _p(xb), len(layers), _p(pos))


def softmax_row(x: np.ndarray) -> None:
    _fn("go_softmax_row", x)(_p(x), x.shape[0])


def attention_ops(cfg: Config, token_positions, freq_real: np.ndarray, freq_imag: np.ndarray,
                  q: np.ndarray, layers: Sequence[Optional[np.ndarray]],
                  att: Optional[np.ndarray] = None) -> np.ndarray:
    """rope -> scores -> softmax -> weighted sum.  Rotates ``q`` and the current K rows in place,
    returns xb (batch, dim).  The current rows must already hold the appended [K|V]."""
    c = cfg.c()
    pos = _pos(token_positions)
    batch = len(layers)
    if att is None:
        att = np.zeros((batch, cfg.n_heads, cfg.seq_len), dtype=q.dtype)
    xb = np.zeros((batch, cfg.dim), dtype=q.dtype)
    _fn("go_attention_ops", q)(C.byref(c), batch, _p(pos), _p(freq_real), _p(freq_imag), _p(q),
                               _ptr_table(layers), _p(att), _p(xb))
    return xb


def rope_tables(seq_len: int, head_size: int, theta: float = 10000.0):
    real = np.empty((seq_len, head_size // 2), dtype=np.float32)
    imag = np.empty_like(real)
    lib().go_rope_tables_f32(_p(real), _p(imag), seq_len, head_size, theta)
    return real, imag


# --------------------------------------------------------------------------------------------
# model driver (models/llama2/model.hh)
# --------------------------------------------------------------------------------------------
class _LayerW(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("rms_att_weight", "wq", "wkv", "wo", "rms_ffn_weight",
                                          "w1", "w2", "w3")]


class _Scratch(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("x", "xb", "xb2", "q", "kv", "hb", "hb2", "att")]


def layer_forward(cfg: Config, weights: dict, freq_real: np.ndarray, freq_imag: np.ndarray,
                  x: np.ndarray, layers: Sequence[Optional[np.ndarray]], token_positions,
                  scratch: Optional[dict] = None) -> dict:
    """One full layer (pre-attention + attention + post-attention) in the storage type of ``x``: float32, or
    float16 with every op's result rounded to binary16 where the reference's DType = _Float16 build rounds it
    (weights, tables and cache rows must have the same type).  ``x`` (batch, dim) is updated in place;
    returns the scratch arrays (q, kv, xb, ...) for inspection."""
    dt = x.dtype
    assert dt in (np.float32, np.float16)
    names = ("rms_att_weight", "wq", "wkv", "wo", "rms_ffn_weight", "w1", "w2", "w3")
    assert all(weights[n].dtype == dt for n in names) and freq_real.dtype == dt and freq_imag.dtype == dt
    assert all(l is None or l.dtype == dt for l in layers)
    batch = x.shape[0]
    s = scratch or {}
    s.setdefault("xb", np.zeros((batch, cfg.dim), dt))
    s.setdefault("xb2", np.zeros((batch, cfg.dim), dt))
    s.setdefault("q", np.zeros((batch, cfg.dim), dt))
    s.setdefault("kv", np.zeros((batch, 2 * cfg.kv_dim), dt))
    s.setdefault("hb", np.zeros((batch, cfg.hidden_dim), dt))
    s.setdefault("hb2", np.zeros((batch, cfg.hidden_dim), dt))
    s.setdefault("att", np.zeros((batch, cfg.n_heads, cfg.seq_len), dt))
    s["x"] = x
    lw = _LayerW(*[_p(weights[n]) for n in names])
    sc = _Scratch(*[_p(s[n]) for n in ("x", "xb", "xb2", "q", "kv", "hb", "hb2", "att")])
    c = cfg.c()
    pos = _pos(token_positions)
    _fn("go_layer_forward", x)(C.byref(c), C.byref(lw), _p(freq_real), _p(freq_imag), C.byref(sc),
                               _ptr_table(layers), _p(pos), batch)
    return s


def classify(cfg: Config, rms_final: np.ndarray, wcls: np.ndarray, x: np.ndarray) -> np.ndarray:
    """Final rmsnorm (in place on ``x``) and the logits, in the storage type of ``x``."""
    assert rms_final.dtype == x.dtype and wcls.dtype == x.dtype
    batch = x.shape[0]
    logits = np.empty((batch, cfg.vocab_size), x.dtype)
    c = cfg.c()
    _fn("go_classify", x)(C.byref(c), _p(rms_final), _p(wcls), _p(x), _p(logits), batch)
    return logits


# --------------------------------------------------------------------------------------------
# bookkeeping
# --------------------------------------------------------------------------------------------
def _hosted(cfg: Config, hosted) -> np.ndarray:
    h = np.ascontiguousarray(np.asarray(hosted, dtype=np.uint8))
    assert h.shape == (cfg.n_layers,)
    return h


def ctx_layer_offset(cfg: Config, hosted, layer: int) -> Optional[int]:
    c = cfg.c()
    v = lib().go_ctx_layer_offset(C.byref(c), _p(_hosted(cfg, hosted)), layer)
    return None if v == 2 ** 64 - 1 else int(v)


def ctx_key_head_offset(cfg: Config, hosted, layer: int, pos: int, h: int) -> Optional[int]:
    c = cfg.c()
    v = lib().go_ctx_key_head_offset(C.byref(c), _p(_hosted(cfg, hosted)), layer, pos, h)
    return None if v == 2 ** 64 - 1 else int(v)


def ctx_value_head_offset(cfg: Config, hosted, layer: int, pos: int, h: int) -> Optional[int]:
    c = cfg.c()
    v = lib().go_ctx_value_head_offset(C.byref(c), _p(_hosted(cfg, hosted)), layer, pos, h)
    return None if v == 2 ** 64 - 1 else int(v)


def ctx_max_size_bytes(cfg: Config, n_hosted: int, elem_size: int) -> int:
    c = cfg.c()
    return int(lib().go_ctx_max_size_bytes(C.byref(c), n_hosted, elem_size))


def dynctx_prepare(cfg: Config, elem_size: int, allocated: np.ndarray, layer: int, token_pos: int,
                   can_release: bool, commit_all: bool = False):
    """Returns (blocks_committed, cleared); ``allocated`` (uint64 per layer) is updated in place."""
    assert allocated.dtype == np.uint64 and allocated.shape == (cfg.n_layers,)
    c = cfg.c()
    cleared = C.c_int(0)
    n = lib().go_dynctx_prepare(C.byref(c), elem_size, _p(allocated), layer, token_pos,
                                int(can_release), int(commit_all), C.byref(cleared))
    return int(n), bool(cleared.value)


class ContextManager:
    """``PreallocatingContextManager`` slot bookkeeping (compute/contextman.hh:56-196)."""

    def __init__(self, max_context_count: int):
        self._m = lib().go_ctxman_new(max_context_count)

    def __del__(self):
        if getattr(self, "_m", None):
            lib().go_ctxman_delete(self._m)
            self._m = None

    def free(self) -> int:
        return int(lib().go_ctxman_free(self._m))

    def allocated(self) -> int:
        return int(lib().go_ctxman_allocated(self._m))

    def get_contexts(self, active, context_ids, start: int = 0, end: Optional[int] = None):
        a = np.ascontiguousarray(np.asarray(active, dtype=np.uint8))
        ids = np.ascontiguousarray(np.asarray(context_ids, dtype=np.uint32))
        end = len(a) if end is None else end
        out = np.empty(max(1, end - start), dtype=np.int32)
        ok = lib().go_ctxman_get_contexts(self._m, _p(a), _p(ids), start, end, _p(out))
        return out[: end - start].tolist() if ok else None

    def get_context(self, context_id: int) -> int:
        return int(lib().go_ctxman_get_context(self._m, context_id))

    def release(self, context_id: int) -> bool:
        return bool(lib().go_ctxman_release(self._m, context_id))


def check_finished(token, token_pos, prompt_length, max_completion_length, seq_len,
                   token_eos=2, token_eot=2) -> bool:
    return bool(lib().go_check_finished(token, token_pos, prompt_length, max_completion_length,
                                        token_eos, token_eot, seq_len))


def encode_temperature(t: float) -> int:
    return int(lib().go_encode_temperature(t))


def decode_temperature(t: int) -> float:
    return float(lib().go_decode_temperature(t))
