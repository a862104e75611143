"""ctypes loader for libglint_hip.so.  Fails loudly when the library is absent: there is no
alternative code path."""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Optional

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG, "lib", "libglint_hip.so")

GH_F16, GH_F32, GH_BF16 = 0, 1, 2
GH_H2D, GH_D2H, GH_D2D, GH_H2H = 0, 1, 2, 3
GH_ATTN_AUTO, GH_ATTN_GENERIC, GH_ATTN_VALU, GH_ATTN_MFMA = 0, 1, 2, 3


class GlintError(RuntimeError):
    pass


class GhShape(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "dim", "kv_dim", "hidden_dim", "n_layers", "head_size", "n_heads", "n_kv_heads",
        "gqa_size", "vocab_size", "seq_len")]


@dataclass(frozen=True)
class Shape:
    """Llama2 shape (the constants of the reference's models/llama2/variants.hh)."""
    dim: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    hidden_dim: int
    seq_len: int
    vocab_size: int = 32000

    @property
    def head_size(self) -> int:
        return self.dim // self.n_heads

    @property
    def gqa_size(self) -> int:
        return self.n_heads // self.n_kv_heads

    @property
    def kv_dim(self) -> int:
        return self.dim // self.gqa_size

    def c(self) -> GhShape:
        return GhShape(self.dim, self.kv_dim, self.hidden_dim, self.n_layers, self.head_size,
                       self.n_heads, self.n_kv_heads, self.gqa_size, self.vocab_size, self.seq_len)


_lib: Optional[C.CDLL] = None

# name -> (restype, argtypes); every symbol declared in include/glint_hip.h
_u64, _u32, _vp, _i, _f = C.c_uint64, C.c_uint32, C.c_void_p, C.c_int, C.c_float
_shp = C.POINTER(GhShape)
SIGNATURES = {
    "gh_init": (_i, [_i]),
    "gh_last_error": (C.c_char_p, []),
    "gh_device_name": (_i, [C.c_char_p, C.c_size_t]),
    "gh_sync": (_i, [_vp]),
    "gh_stream_create": (_i, [C.POINTER(_vp)]),
    "gh_stream_destroy": (_i, [_vp]),
    "gh_event_create": (_i, [C.POINTER(_vp)]),
    "gh_event_destroy": (_i, [_vp]),
    "gh_event_create_timed": (_i, [C.POINTER(_vp)]),
    "gh_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(C.c_float)]),
    "gh_event_record": (_i, [_vp, _vp]),
    "gh_stream_wait_event": (_i, [_vp, _vp]),
    "gh_malloc": (_i, [C.POINTER(_vp), _u64]),
    "gh_free": (_i, [_vp]),
    "gh_allocation_count": (_u64, []),
    "gh_host_malloc": (_i, [C.POINTER(_vp), _u64]),
    "gh_host_free": (_i, [_vp]),
    "gh_memcpy": (_i, [_vp, _vp, _u64, _i, _i, _vp]),
    "gh_memset_zero": (_i, [_vp, _u64, _vp]),
    "gh_fill_uniform": (_i, [_vp, _u64, _f, _f, _u64, _i, _vp]),
    "gh_fill_normal": (_i, [_vp, _u64, _f, _f, _u64, _i, _vp]),
    "gh_convert_and_copy": (_i, [_vp, _i, _vp, _i, _u64, _i, _vp]),
    "gh_convert": (_i, [_vp, _i, _vp, _i, _u64, _vp]),
    "gh_vmm_granularity": (_i, [C.POINTER(_u64)]),
    "gh_vmm_reserve": (_i, [C.POINTER(_vp), _u64]),
    "gh_vmm_ptr": (_vp, [_vp]),
    "gh_vmm_max_len": (_u64, [_vp]),
    "gh_vmm_commit": (_i, [_vp, _u64, _u64]),
    "gh_vmm_clear": (_i, [_vp]),
    "gh_vmm_committed_bytes": (_u64, [_vp]),
    "gh_vmm_free": (_i, [_vp]),
    "gh_accum": (_i, [_vp, _vp, _u64, _u64, _i, _vp]),
    "gh_rmsnorm": (_i, [_vp, _vp, _vp, _u64, _u64, _i, _vp]),
    "gh_silu": (_i, [_vp, _vp, _u64, _u64, _i, _vp]),
    "gh_argmax": (_i, [_vp, _vp, _vp, _u64, _u64, _i, _vp]),
    "gh_gemm_set_tuning": (_i, [_i, _i, _i]),
    "gh_gemm_set_gate_waves": (_i, [_i]),
    "gh_gemm_set_library_rows": (_i, [_u64]),
    "gh_gemm_library_rows": (_u64, []),
    "gh_gemm_library_calls": (_u64, []),
    "gh_matmul_fuses_many_rows": (_i, [_u64, _u64, _u64, _i]),
    "gh_gemm_stream_plan": (_i, [_u64, _u64, _u64, _vp, _vp, _vp]),
    "gh_matmul": (_i, [_vp, _vp, _vp, _u64, _u64, _u64, _i, _vp]),
    "gh_matmul_pair": (_i, [_vp, _vp, _vp, _vp, _u64, _u64, _u64, _u64, _i, _vp]),
    "gh_matmul_accum": (_i, [_vp, _vp, _vp, _u64, _u64, _u64, _vp, _vp, _i, _vp]),
    "gh_matmul_silu_gate": (_i, [_vp, _vp, _vp, _u64, _u64, _u64, _i, _vp]),
    "gh_matmul_qkv_rope_append": (_i, [_vp, _vp, _vp, _vp, _u64, _u64, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _i, _vp]),
    "gh_soft_sample": (_i, [_vp, _vp, _u64, _u64, _u64, _i, _vp]),
    "gh_kv_append": (_i, [_vp, _vp, _u64, _u32, _i, _vp]),
    "gh_kv_append_host": (_i, [_vp, _vp, _u64, _u32, _i, _vp]),
    "gh_rope": (_i, [_u64, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _i, _vp]),
    "gh_rope_host": (_i, [_u64, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _i, _vp]),
    "gh_attn_scores": (_i, [_vp, _vp, _vp, _u64, _vp, _shp, _i, _vp]),
    "gh_attn_scores_host": (_i, [_vp, _vp, _vp, _u64, _vp, _shp, _i, _vp]),
    "gh_attn_softmax": (_i, [_vp, _vp, _u64, _shp, _i, _vp]),
    "gh_attn_softmax_host": (_i, [_vp, _vp, _u64, _shp, _i, _vp]),
    "gh_attn_pv": (_i, [_vp, _vp, _vp, _u64, _vp, _shp, _i, _vp]),
    "gh_attn_pv_host": (_i, [_vp, _vp, _vp, _u64, _vp, _shp, _i, _vp]),
    "gh_attn_set_chunk": (_i, [_u32]),
    "gh_attn_set_split_join": (_i, [_i]),
    "gh_attn_set_auto_variant": (_i, [_i]),
    "gh_attn_decode_workspace": (_u64, [_u64, _u32, _shp]),
    "gh_attn_decode_plan": (_i, [_u64, _u32, _shp, _i, _i, C.POINTER(_u32), C.POINTER(_u32), C.POINTER(_u64)]),
    "gh_attn_decode_join_waves": (_u32, [_u64, _u32, _shp, _i, _i]),
    "gh_attn_decode": (_i, [_vp, _vp, _vp, _vp, _u64, _u32, _shp, _i, _vp, _u64, _i, _vp]),
    "gh_attn_decode_static_limit": (_u64, []),
    "gh_attn_decode_static": (_i, [_vp, _vp, _vp, _vp, _u64, _u32, _shp, _i, _i, _vp]),
    "gh_attn_decode_host": (_i, [_vp, _vp, _vp, _vp, _u64, _shp, _i, _vp, _u64, _i, _vp]),
    "gh_attn_balanced_workspace": (_u64, [_u64, _shp]),
    "gh_attn_balance": (_i, [_vp, _vp, _u64, _u32, _shp, _vp, _u64, _vp]),
    "gh_attn_decode_balanced": (_i, [_vp, _vp, _vp, _u64, _u32, _shp, _i, _vp, _u64, _vp]),
    "gh_prefill_tables": (_i, [_vp, _vp, _u64, _u32, _u64, _vp, _vp, _vp, _vp]),
    "gh_attn_set_prefill_tiles": (_i, [_i]),
    "gh_attn_prefill_workspace": (_u64, [_u64, _u32, _shp]),
    "gh_attn_prefill": (_i, [_vp, _vp, _vp, _vp, _u64, _u32, _u32, _shp, _i, _vp, _u64, _i, _vp]),
    "gh_attn_timing_enable": (_i, [_i]),
    "gh_attn_timing_reset": (_i, []),
    "gh_attn_timing_read": (_i, [C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(_u64)]),
}


def lib_path() -> str:
    return _LIB_PATH


def lib() -> C.CDLL:
    """The loaded library.  Raises GlintError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise GlintError(
                f"{_LIB_PATH} is missing: build it with `python -m glinthawk_amd.build` "
                "(there is no fallback implementation)")
        L = C.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        msg = lib().gh_last_error().decode(errors="replace")
        raise GlintError(f"{what or 'libglint_hip'} failed ({rc}): {msg}")
