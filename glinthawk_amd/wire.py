"""The reference's serialized BatchedInferenceState (models/common/state.hh:17-50,512-594) as numpy
record types: packing and unpacking on the Python side of a pipeline, and `HostState`, a handle on
the C++ host layer's state object (fixed to the "test-tiny" shape, dim 32 / kv_dim 16) for the
host-only tests of refill, split and merge."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import numpy as np

from ._lib import GlintError
from .stage import host_lib as _stage_host_lib

# packed structs, host (little-endian) byte order
META_DTYPE = np.dtype([
    ("id", "<u8"), ("batch_size", "<u4"), ("dtype", "u1"), ("route_id", "<u4"), ("model_id", "<u4"),
    ("next_layer", "<u4"), ("next_stage", "u1"), ("next_tier", "i1"), ("next_rank", "u1"),
    ("has_activations", "u1"), ("has_queries", "u1"), ("has_kvs", "u1"), ("is_sharded", "u1")])
PROMPT_DTYPE = np.dtype([
    ("active", "u1"), ("prompt_id", "u1", (32,)), ("context_id", "<u4"), ("token", "<u4"), ("token_pos", "<u4"),
    ("temperature", "u1"), ("prompt_length", "<u4"), ("max_completion_length", "<u4"), ("finished", "u1"),
    ("kv_tier", "i1"), ("kv_rank", "u1")])
assert META_DTYPE.itemsize == 32 and PROMPT_DTYPE.itemsize == 57

DTYPE_CODE = {"f16": 0, "f32": 1, "bf16": 2}
ELEM_SIZE = {0: 2, 1: 4, 2: 2}


def new_prompts(batch: int) -> np.ndarray:
    """Default-initialised prompt records (inactive, kv_tier -1 = unassigned)."""
    p = np.zeros(batch, dtype=PROMPT_DTYPE)
    p["kv_tier"] = -1
    return p


def pack_state(meta: dict, prompts: np.ndarray, activations: Optional[np.ndarray] = None,
               queries: Optional[np.ndarray] = None, kvs: Optional[np.ndarray] = None) -> bytes:
    """`meta` gives the metadata fields that are not implied (id, dtype code, route_id, model_id, next_layer,
    next_stage, next_tier, next_rank, is_sharded); batch size and the has_* flags follow from the arguments."""
    m = np.zeros((), dtype=META_DTYPE)
    for k, v in meta.items():
        m[k] = v
    m["batch_size"] = len(prompts)
    m["has_activations"], m["has_queries"], m["has_kvs"] = activations is not None, queries is not None, kvs is not None
    out = m.tobytes() + np.ascontiguousarray(prompts, dtype=PROMPT_DTYPE).tobytes()
    for buf in (activations, queries, kvs):
        if buf is not None:
            out += np.ascontiguousarray(buf).tobytes()
    return out


def unpack_state(raw: bytes, dim: int, kv_dim: int):
    """-> (meta record, prompt records, activations, queries, kvs) with absent buffers None; buffers come back
    as (batch, n) arrays of float16 / float32 (uint16 for bf16).  Raises ValueError on a wrong length."""
    if len(raw) < META_DTYPE.itemsize:
        raise ValueError("too short for the metadata")
    m = np.frombuffer(raw[:32], dtype=META_DTYPE)[0]
    b = int(m["batch_size"])
    code = int(m["dtype"])
    if code not in ELEM_SIZE:
        raise ValueError("unknown data type")
    elem = ELEM_SIZE[code]
    np_dt = {0: np.float16, 1: np.float32, 2: np.uint16}[code]
    need = 32 + 57 * b + elem * b * (dim * (int(m["has_activations"]) + int(m["has_queries"])) + 2 * kv_dim * int(m["has_kvs"]))
    if len(raw) != need:
        raise ValueError(f"{len(raw)} bytes, {need} expected")
    off = 32
    prompts = np.frombuffer(raw[off:off + 57 * b], dtype=PROMPT_DTYPE).copy()
    off += 57 * b
    bufs = []
    for present, n in ((m["has_activations"], dim), (m["has_queries"], dim), (m["has_kvs"], 2 * kv_dim)):
        if present:
            bufs.append(np.frombuffer(raw[off:off + b * n * elem], dtype=np_dt).reshape(b, n).copy())
            off += b * n * elem
        else:
            bufs.append(None)
    return m, prompts, bufs[0], bufs[1], bufs[2]


_signed = False


def _lib():
    global _signed
    L = _stage_host_lib()
    if not _signed:
        vp, u32, u64, i = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int
        sig = {
            "glint_state_new": (vp, [u32, i, u32, u32]),
            "glint_state_parse": (vp, [vp, u64]),
            "glint_state_delete": (None, [vp]),
            "glint_state_serialize": (vp, [vp, C.POINTER(u64)]),
            "glint_state_set_meta": (None, [vp, u64, u32, i, i, u32, i]),
            "glint_state_set_prompt": (None, [vp, u32, vp, u32, u32, u32, C.c_float, u32, u32, i, u32]),
            "glint_state_discard": (None, [vp, u32]),
            "glint_state_set_finished": (None, [vp, u32]),
            "glint_state_check_finished": (i, [vp, u32]),
            "glint_state_positions_fit": (i, [vp, u64]),
            "glint_state_free_slots": (u64, [vp]),
            "glint_state_batch_size": (u32, [vp]),
            "glint_state_all_assigned": (i, [vp]),
            "glint_state_buffer": (vp, [vp, i, C.POINTER(u64), i]),
            "glint_state_replenish_from": (i, [vp, vp]),
            "glint_state_merge": (None, [vp, vp]),
            "glint_state_split": (None, [vp, u64, C.POINTER(vp), C.POINTER(vp)]),
            "glint_state_split_on_kv": (u64, [vp, C.POINTER(vp), u64]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _signed = True
    return L


class HostState:
    """A BatchedInferenceState of the "test-tiny" shape living in the C++ host layer."""
    DIM, KV_DIM, SEQ_LEN = 32, 16, 16

    def __init__(self, batch: int = 0, dtype: str = "f16", route_id: int = 0, model_id: int = 0, _handle=None):
        self._h = _handle if _handle is not None else _lib().glint_state_new(batch, DTYPE_CODE[dtype], route_id, model_id)

    @classmethod
    def parse(cls, raw: bytes) -> "HostState":
        buf = C.create_string_buffer(raw, len(raw))
        h = _lib().glint_state_parse(C.cast(buf, C.c_void_p), len(raw))
        if not h:
            raise GlintError(_lib().glint_last_error().decode(errors="replace"))
        return cls(_handle=h)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                _lib().glint_state_delete(self._h)
                self._h = None
        except Exception:
            pass

    def serialize(self) -> bytes:
        n = C.c_uint64(0)
        p = _lib().glint_state_serialize(self._h, C.byref(n))
        return C.string_at(p, n.value)

    def set_meta(self, id=0, next_layer=0, next_stage=0, next_tier=0, next_rank=0, is_sharded=False):
        _lib().glint_state_set_meta(self._h, id, next_layer, next_stage, next_tier, next_rank, int(is_sharded))

    def set_prompt(self, i, prompt_id: bytes, context_id, token, token_pos, temperature, prompt_length,
                   max_completion_length, kv_tier, kv_rank):
        pid = (C.c_uint8 * 32).from_buffer_copy(prompt_id.ljust(32, b"\0")[:32])
        _lib().glint_state_set_prompt(self._h, i, C.cast(pid, C.c_void_p), context_id, token, token_pos, temperature,
                                      prompt_length, max_completion_length, kv_tier, kv_rank)

    def discard(self, i):
        _lib().glint_state_discard(self._h, i)

    def set_finished(self, i):
        _lib().glint_state_set_finished(self._h, i)

    def check_finished(self, i) -> bool:
        return bool(_lib().glint_state_check_finished(self._h, i))

    def positions_fit(self, seq_len: int) -> bool:
        """The stage driver's host-side check of the rows' positions against the context window."""
        return bool(_lib().glint_state_positions_fit(self._h, seq_len))

    def free_slots(self) -> int:
        return _lib().glint_state_free_slots(self._h)

    def batch_size(self) -> int:
        return _lib().glint_state_batch_size(self._h)

    def all_assigned_to_nodes(self) -> bool:
        return bool(_lib().glint_state_all_assigned(self._h))

    def buffer(self, which: int, allocate: bool = False) -> Optional[np.ndarray]:
        """which: 0 activations, 1 queries, 2 kvs.  A writable byte view into the state, None when absent."""
        n = C.c_uint64(0)
        p = _lib().glint_state_buffer(self._h, which, C.byref(n), int(allocate))
        if n.value == 0:
            return None
        return np.ctypeslib.as_array((C.c_uint8 * n.value).from_address(p))

    def replenish_from(self, other: "HostState") -> bool:
        return bool(_lib().glint_state_replenish_from(self._h, other._h))

    def merge(self, other: "HostState") -> None:
        _lib().glint_state_merge(self._h, other._h)

    def split(self, n: int):
        a, b = C.c_void_p(), C.c_void_p()
        _lib().glint_state_split(self._h, n, C.byref(a), C.byref(b))
        return HostState(_handle=a.value), HostState(_handle=b.value)

    def split_on_kv(self):
        cap = 1024
        arr = (C.c_void_p * cap)()
        n = _lib().glint_state_split_on_kv(self._h, arr, cap)
        return [HostState(_handle=arr[i]) for i in range(n)]
