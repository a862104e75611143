"""ctypes front-end of libglint_host.so: the C++ stage harness (model driver + context manager + one
batched state) and the host-only bookkeeping hooks.  Used by the tests and the benchmark; all
compute happens in the C++/HIP layers."""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import numpy as np

from ._lib import GlintError

_PKG = os.path.dirname(os.path.abspath(__file__))
# GLINT_HOST_LIB: another build of the same sources (the sanitizer build of the CPU test suite)
_HOST_LIB_PATH = os.environ.get("GLINT_HOST_LIB") or os.path.join(_PKG, "lib", "libglint_host.so")

STAGE_PRE, STAGE_ATT, STAGE_POST, STAGE_CLS = 0, 1, 2, 3
FWD_ALL, FWD_PRE, FWD_ATT, FWD_POST, FWD_CLS = 0, 1, 2, 3, 4
FLAG_FUSED, FLAG_CLS, FLAG_PAGED, FLAG_UNFUSED_PROJ, FLAG_BALANCED, FLAG_NOT_BALANCED = 1, 2, 4, 8, 16, 32

# layer tensors in file order (rms_att_weight, wq, wkv, wo, rms_ffn_weight, w1, w2, w3)
LAYER_TENSORS = ("rms_att_weight", "wq", "wkv", "wo", "rms_ffn_weight", "w1", "w2", "w3")
BASE_TENSORS = ("token_embedding_table", "rms_final_weight", "freq_cis_real", "freq_cis_imag", "wcls")

_host: Optional[C.CDLL] = None


def host_lib_path() -> str:
    return _HOST_LIB_PATH


def host_lib() -> C.CDLL:
    global _host
    if _host is None:
        if not os.path.exists(_HOST_LIB_PATH):
            raise GlintError(f"{_HOST_LIB_PATH} is missing: build it with `python -m glinthawk_amd.build`")
        L = C.CDLL(_HOST_LIB_PATH)
        vp, u32, u64, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32
        sig = {
            "glint_stage_create": (vp, [C.c_char_p, C.c_int, u32, u32, u32, u32, u32, u64, C.c_float]),
            "glint_stage_destroy": (None, [vp]),
            "glint_stage_set_layer_tensor": (None, [vp, u32, u32, vp, u64]),
            "glint_stage_set_base_tensor": (None, [vp, u32, vp, u64]),
            "glint_stage_layer_tensor_ptr": (vp, [vp, u32, u32, C.POINTER(u64)]),
            "glint_stage_base_tensor_ptr": (vp, [vp, u32, C.POINTER(u64)]),
            "glint_stage_new_state": (None, [vp, u32, u32, C.c_int]),
            "glint_stage_set_prompt": (None, [vp, u32, u32, u32, u32, C.c_float, u32, u32]),
            "glint_stage_set_prompts": (None, [vp, u32, vp, vp, vp, C.c_float, u32, u32]),
            "glint_stage_discard": (None, [vp, u32]),
            "glint_stage_set_next": (None, [vp, u32, C.c_int]),
            "glint_stage_acquire_contexts": (C.c_int, [vp]),
            "glint_stage_forward": (C.c_int, [vp, C.c_int]),
            "glint_stage_buffer": (vp, [vp, C.c_int, C.POINTER(u64), C.c_int]),
            "glint_stage_row_info": (None, [vp, u32, C.POINTER(u32)]),
            "glint_stage_state_info": (None, [vp, C.POINTER(u32)]),
            "glint_stage_context_layer_ptr": (vp, [vp, u32, u32]),
            "glint_stage_context_slot": (i32, [vp, u32]),
            "glint_stage_slot_counts": (None, [vp, C.POINTER(u64)]),
            "glint_stage_release_context": (C.c_int, [vp, u32]),
            "glint_stage_paging_info": (None, [vp, u32, u32, C.POINTER(u64)]),
            "glint_stage_scratch": (vp, [vp, C.c_int]),
            "glint_stage_sync": (None, [vp]),
            "glint_stage_copy_bytes": (None, [vp, vp, vp, u64, C.c_int]),
            "glint_stage_time_device_spans": (None, [vp, C.c_int]),
            "glint_stage_device_spans": (None, [vp, C.POINTER(C.c_double), C.POINTER(u64)]),
            "glint_stage_prefill": (C.c_int, [vp, u32, vp, vp, u32, u32, vp, vp, vp, vp]),
            "glint_stage_load": (C.c_int, [vp, C.c_char_p]),
            "glint_last_error": (C.c_char_p, []),
            "glint_stage_set_state_bytes": (C.c_int, [vp, vp, C.c_uint64]),
            "glint_stage_get_state_bytes": (vp, [vp, C.POINTER(C.c_uint64)]),
            "glint_model_dir_walk": (C.c_int64, [C.c_char_p, C.c_int, u32, u32, u32, C.c_char_p, vp, C.c_uint64]),
            "glint_book_manager_new": (vp, [u64]),
            "glint_book_manager_delete": (None, [vp]),
            "glint_book_manager_free": (u64, [vp]),
            "glint_book_manager_allocated": (u64, [vp]),
            "glint_book_manager_get_contexts": (C.c_int, [vp, vp, vp, u64, u64, u64, vp]),
            "glint_book_manager_get_context": (i32, [vp, u32]),
            "glint_book_manager_release": (C.c_int, [vp, u32]),
            "glint_book_paged_new": (vp, [u32]),
            "glint_book_paged_delete": (None, [vp]),
            "glint_book_paged_prepare": (u64, [vp, u32, u32, C.c_int, C.POINTER(u64)]),
            "glint_book_key_head_offset": (u64, [vp, u32, u32, u32, C.c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _host = L
    return _host


class Stage:
    """One pipeline stage on the GPU: `n_hosted` consecutive layers of `config` starting at
    `first_layer`, with `max_contexts` preallocated context slots."""

    def __init__(self, config: str, dtype: str, first_layer: int, n_hosted: int, concurrency: int,
                 max_contexts: int, fused: bool = True, with_cls: bool = False, paged: bool = False,
                 seed: int = 1, weight_std: float = 0.02, fused_projections: bool = True, balanced=None):
        # balanced: decode attention over equal runs of keys always (True) / never (False); None: where a step's lengths call for it
        self.np_dtype = np.float16 if dtype == "f16" else np.float32
        flags = ((FLAG_FUSED if fused else 0) | (FLAG_CLS if with_cls else 0) | (FLAG_PAGED if paged else 0)
                 | (0 if fused_projections else FLAG_UNFUSED_PROJ)
                 | (0 if balanced is None else FLAG_BALANCED if balanced else FLAG_NOT_BALANCED))
        self._h = host_lib().glint_stage_create(config.encode(), 0 if dtype == "f16" else 1, first_layer, n_hosted,
                                                concurrency, max_contexts, flags, seed, weight_std)
        if not self._h:
            raise GlintError(f"unknown stage configuration {config!r}")

    def close(self):
        if getattr(self, "_h", None):
            host_lib().glint_stage_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:       # interpreter shutdown: module globals may already be gone
            pass

    def set_state_bytes(self, raw: bytes) -> None:
        """Replaces the stage's batched state by one in the reference's wire format (as it arrives from the
        previous stage)."""
        buf = C.create_string_buffer(raw, len(raw))
        if host_lib().glint_stage_set_state_bytes(self._h, C.cast(buf, C.c_void_p), len(raw)) != 0:
            raise GlintError(host_lib().glint_last_error().decode(errors="replace"))

    def get_state_bytes(self) -> bytes:
        """The stage's batched state in the reference's wire format (what the next stage receives)."""
        n = C.c_uint64(0)
        p = host_lib().glint_stage_get_state_bytes(self._h, C.byref(n))
        return C.string_at(p, n.value)

    def load(self, model_dir: str) -> None:
        """Copies the tensors this stage hosts out of a model directory in the reference's format
        (CONFIG, BASEWEIGHTS_<FP16|FP32>, LAYER<i>_<FP16|FP32>)."""
        if host_lib().glint_stage_load(self._h, os.fsencode(model_dir)) != 0:
            raise GlintError(host_lib().glint_last_error().decode(errors="replace"))

    # ---- weights
    def get_layer_tensor(self, layer: int, name: str) -> np.ndarray:
        """A copy of a resident tensor of a hosted layer (1-D, the stage's storage type)."""
        n = C.c_uint64(0)
        ptr = host_lib().glint_stage_layer_tensor_ptr(self._h, layer, LAYER_TENSORS.index(name), C.byref(n))
        return self._download(ptr, n.value, f"layer {layer} {name}")

    def get_base_tensor(self, name: str) -> np.ndarray:
        n = C.c_uint64(0)
        ptr = host_lib().glint_stage_base_tensor_ptr(self._h, BASE_TENSORS.index(name), C.byref(n))
        return self._download(ptr, n.value, name)

    def _download(self, ptr, n: int, what: str) -> np.ndarray:
        from . import _lib
        if not ptr or n == 0:
            raise GlintError(f"the stage does not host {what}")
        out = np.empty(n, dtype=self.np_dtype)
        _lib.check(_lib.lib().gh_memcpy(out.ctypes.data, ptr, out.nbytes, _lib.GH_D2H, 0, None), "gh_memcpy")
        return out

    def set_layer_tensor(self, layer: int, name: str, arr: np.ndarray) -> None:
        a = np.ascontiguousarray(arr, dtype=self.np_dtype)
        host_lib().glint_stage_set_layer_tensor(self._h, layer, LAYER_TENSORS.index(name), a.ctypes.data, a.size)

    def set_base_tensor(self, name: str, arr: np.ndarray) -> None:
        a = np.ascontiguousarray(arr, dtype=self.np_dtype)
        host_lib().glint_stage_set_base_tensor(self._h, BASE_TENSORS.index(name), a.ctypes.data, a.size)

    # ---- state
    def new_state(self, batch: int, next_layer: int = 0, next_stage: int = STAGE_PRE) -> None:
        host_lib().glint_stage_new_state(self._h, batch, next_layer, next_stage)

    def set_prompt(self, row: int, context_id: int, token: int, pos: int, temperature: float = 0.0,
                   prompt_length: int = 1, max_completion_length: int = 0) -> None:
        host_lib().glint_stage_set_prompt(self._h, row, context_id, token, pos, temperature, prompt_length,
                                          max_completion_length)

    def set_prompts(self, context_ids, tokens, positions, temperature: float = 0.0, prompt_length: int = 1,
                    max_completion_length: int = 0) -> None:
        """set_prompt for rows 0 .. n-1 in one call (three arrays of n values)."""
        ids = np.ascontiguousarray(context_ids, dtype=np.uint32)
        tok = np.ascontiguousarray(tokens, dtype=np.uint32)
        pos = np.ascontiguousarray(positions, dtype=np.uint32)
        if not (ids.ndim == tok.ndim == pos.ndim == 1 and ids.size == tok.size == pos.size):
            raise ValueError("set_prompts: three one-dimensional arrays of equal length")
        host_lib().glint_stage_set_prompts(self._h, ids.size, ids.ctypes.data, tok.ctypes.data, pos.ctypes.data, temperature,
                                           prompt_length, max_completion_length)

    def discard(self, row: int) -> None:
        host_lib().glint_stage_discard(self._h, row)

    def set_next(self, layer: int, stage: int = STAGE_PRE) -> None:
        host_lib().glint_stage_set_next(self._h, layer, stage)

    def acquire_contexts(self) -> bool:
        return host_lib().glint_stage_acquire_contexts(self._h) == 0

    def forward(self, which: int = FWD_ALL) -> bool:
        """False when the context manager could not serve the batch (nothing ran)."""
        rc = host_lib().glint_stage_forward(self._h, which)
        if rc == -2:
            raise GlintError("bad forward selector")
        return rc == 0

    def _buffer(self, which: int, allocate: bool) -> np.ndarray:
        n = C.c_uint64(0)
        p = host_lib().glint_stage_buffer(self._h, which, C.byref(n), int(allocate))
        if not p or n.value == 0:
            return np.empty(0, dtype=self.np_dtype)
        buf = (C.c_uint8 * n.value).from_address(p)
        return np.frombuffer(buf, dtype=self.np_dtype)

    def activations(self, allocate: bool = False) -> np.ndarray:
        return self._buffer(0, allocate)

    def queries(self, allocate: bool = False) -> np.ndarray:
        return self._buffer(1, allocate)

    def kvs(self, allocate: bool = False) -> np.ndarray:
        return self._buffer(2, allocate)

    def row(self, i: int) -> dict:
        out = (C.c_uint32 * 6)()
        host_lib().glint_stage_row_info(self._h, i, out)
        return dict(active=bool(out[0]), context_id=out[1], token=out[2], token_pos=out[3], finished=bool(out[4]),
                    temperature_u8=out[5])

    def state(self) -> dict:
        out = (C.c_uint32 * 4)()
        host_lib().glint_stage_state_info(self._h, out)
        return dict(batch_size=out[0], next_layer=out[1], next_stage=out[2], has_activations=bool(out[3] & 1),
                    has_queries=bool(out[3] & 2), has_kvs=bool(out[3] & 4))

    # ---- contexts
    def context_layer_ptr(self, row: int, layer: int) -> int:
        return host_lib().glint_stage_context_layer_ptr(self._h, row, layer) or 0

    def context_slot(self, row: int) -> int:
        return host_lib().glint_stage_context_slot(self._h, row)

    def slot_counts(self) -> dict:
        out = (C.c_uint64 * 3)()
        host_lib().glint_stage_slot_counts(self._h, out)
        return dict(free=out[0], allocated=out[1], total=out[2])

    def release_context(self, context_id: int) -> bool:
        return bool(host_lib().glint_stage_release_context(self._h, context_id))

    def paging_info(self, row: int, layer: int) -> dict:
        out = (C.c_uint64 * 3)()
        host_lib().glint_stage_paging_info(self._h, row, layer, out)
        return dict(allocated_bytes=out[0], blocks_committed=out[1], clears=out[2])

    def scratch_ptr(self, name: str) -> int:
        return host_lib().glint_stage_scratch(self._h, ("x", "xb", "q", "kv", "logits").index(name)) or 0

    def sync(self) -> None:
        host_lib().glint_stage_sync(self._h)

    def copy_bytes(self, dst: int, src: int, n_bytes: int, kind: int) -> None:
        """The ops class's convert_and_copy<void, void>: a synchronous copy of n_bytes bytes (kind: 0 host to device,
        1 device to host, 2 device to device, 3 host to host)."""
        host_lib().glint_stage_copy_bytes(self._h, dst, src, n_bytes, kind)

    def time_device_spans(self, on: bool) -> None:
        """Times forward() on the device, first kernel to last, without the copies of the state over the host boundary."""
        host_lib().glint_stage_time_device_spans(self._h, int(on))

    def device_spans(self):
        """(milliseconds, steps) accumulated since the last read."""
        ms, n = C.c_double(0), C.c_uint64(0)
        host_lib().glint_stage_device_spans(self._h, C.byref(ms), C.byref(n))
        return ms.value, int(n.value)

    def prefill(self, context_ids, start_pos, n_tokens: int, first_layer: int = 0, token_ids=None, activations=None,
                want_activations: bool = True, want_next_tokens: bool = False, out=None):
        """Batched prefill of `n_tokens` tokens per context.  Returns (activations_out or None,
        next_tokens or None); None overall when the contexts could not be served."""
        batch = len(context_ids)
        ids = np.ascontiguousarray(np.asarray(context_ids, dtype=np.uint32))
        start = np.ascontiguousarray(np.asarray(start_pos, dtype=np.uint32))
        toks = None if token_ids is None else np.ascontiguousarray(np.asarray(token_ids, dtype=np.uint32).reshape(-1))
        acts = None if activations is None else np.ascontiguousarray(activations, dtype=self.np_dtype)   # no copy when already so
        if toks is not None:
            assert toks.size == batch * n_tokens
        dim = None if acts is None else acts.reshape(batch * n_tokens, -1).shape[1]
        if not want_activations:
            out = None
        if want_activations:
            if dim is None:
                raise ValueError("pass dim via activations or call with want_activations=False")
            if out is None:
                out = np.empty((batch * n_tokens, dim), dtype=self.np_dtype)
            assert out.dtype == self.np_dtype and out.size == batch * n_tokens * dim and out.flags["C_CONTIGUOUS"]
        nxt = np.zeros(batch, dtype=np.uint32) if want_next_tokens else None
        rc = host_lib().glint_stage_prefill(self._h, batch, ids.ctypes.data, start.ctypes.data, n_tokens, first_layer,
                                            None if toks is None else toks.ctypes.data,
                                            None if acts is None else acts.ctypes.data,
                                            None if out is None else out.ctypes.data,
                                            None if nxt is None else nxt.ctypes.data)
        if rc != 0:
            return None
        return out, nxt


class BookManager:
    """Host-only instance of the slot manager (no device memory), for bookkeeping tests."""

    def __init__(self, max_context_count: int):
        self._m = host_lib().glint_book_manager_new(max_context_count)

    def __del__(self):
        if getattr(self, "_m", None):
            host_lib().glint_book_manager_delete(self._m)
            self._m = None

    def free(self) -> int:
        return int(host_lib().glint_book_manager_free(self._m))

    def allocated(self) -> int:
        return int(host_lib().glint_book_manager_allocated(self._m))

    def get_contexts(self, active, context_ids, start: int = 0, end: Optional[int] = None):
        a = np.ascontiguousarray(np.asarray(active, dtype=np.uint8))
        ids = np.ascontiguousarray(np.asarray(context_ids, dtype=np.uint32))
        end = len(a) if end is None else end
        out = np.empty(max(1, end - start), dtype=np.int32)
        ok = host_lib().glint_book_manager_get_contexts(self._m, a.ctypes.data, ids.ctypes.data, len(a), start, end,
                                                        out.ctypes.data)
        return out[: end - start].tolist() if ok else None

    def get_context(self, context_id: int) -> int:
        return int(host_lib().glint_book_manager_get_context(self._m, context_id))

    def release(self, context_id: int) -> bool:
        return bool(host_lib().glint_book_manager_release(self._m, context_id))


class BookPagedContext:
    """Host-only paged context (70B-4K shape, fp16) over a region that only records commits."""

    def __init__(self, n_hosted: int):
        self._c = host_lib().glint_book_paged_new(n_hosted)

    def __del__(self):
        if getattr(self, "_c", None):
            host_lib().glint_book_paged_delete(self._c)
            self._c = None

    def prepare(self, layer: int, token_pos: int, can_release: bool):
        out = (C.c_uint64 * 2)()
        allocated = host_lib().glint_book_paged_prepare(self._c, layer, token_pos, int(can_release), out)
        return int(allocated), int(out[0]), int(out[1])


def model_dir_walk(config: str, dtype: str, first_layer: int, n_hosted: int, with_cls: bool, model_dir: str):
    """Host-only: validates CONFIG and the weight files a stage of layers [first_layer, first_layer +
    n_hosted) would open, and lists the tensors it would copy as dicts (is_base, layer, tensor name,
    byte offset in its file, elements).  Raises GlintError with the loader's message on failure."""
    cap = 1024
    rec = np.zeros((cap, 5), dtype=np.uint64)
    n = host_lib().glint_model_dir_walk(config.encode(), 0 if dtype == "f16" else 1, first_layer, n_hosted,
                                        FLAG_CLS if with_cls else 0, os.fsencode(model_dir), rec.ctypes.data, cap)
    if n < 0:
        raise GlintError(host_lib().glint_last_error().decode(errors="replace"))
    out = []
    for r in rec[:n]:
        is_base = bool(r[0])
        out.append(dict(is_base=is_base, layer=int(r[1]), tensor=(BASE_TENSORS if is_base else LAYER_TENSORS)[int(r[2])],
                        offset=int(r[3]), elements=int(r[4])))
    return out


def book_head_offset(hosted, layer: int, pos: int, head: int, value: bool) -> Optional[int]:
    h = np.ascontiguousarray(np.asarray(hosted, dtype=np.uint8))
    assert h.size == 80
    v = host_lib().glint_book_key_head_offset(h.ctypes.data, layer, pos, head, int(value))
    return None if v == 2 ** 64 - 1 else int(v)
