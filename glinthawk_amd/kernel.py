"""ComputeKernel: the host layer's BatchedComputeKernel (push / pop / eventfd over a model and its
context manager, as a Glinthawk worker drives it).  States cross as wire-format bytes (see
glinthawk_amd.wire)."""
from __future__ import annotations

import ctypes as C
import os
import select
from typing import Optional

from ._lib import GlintError
from .stage import FLAG_CLS, FLAG_FUSED, FLAG_UNFUSED_PROJ, host_lib

_signed = False


def _lib():
    global _signed
    L = host_lib()
    if not _signed:
        vp, u32, u64, i = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int
        sig = {
            "glint_kernel_create": (vp, [C.c_char_p, i, u32, u32, u32, u32, u32, u64, C.c_float]),
            "glint_kernel_create_echo": (vp, [u32, u32]),
            "glint_kernel_destroy": (None, [vp]),
            "glint_kernel_load": (i, [vp, C.c_char_p]),
            "glint_kernel_push": (i, [vp, vp, u64]),
            "glint_kernel_pop": (vp, [vp, C.POINTER(u64)]),
            "glint_kernel_event_fd": (i, [vp]),
            "glint_kernel_read_event": (i, [vp, C.POINTER(u64)]),
            "glint_kernel_slot_counts": (None, [vp, C.POINTER(u64 * 3)]),
            "glint_last_error": (C.c_char_p, []),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _signed = True
    return L


class ComputeKernel:
    def __init__(self, config: Optional[str] = None, dtype: str = "f16", first_layer: int = 0, n_hosted: int = 1,
                 concurrency: int = 1, max_contexts: int = 1, with_cls: bool = False, fused: bool = True,
                 fused_projections: bool = True, seed: int = 1, weight_std: float = 0.02, echo: bool = False):
        """`echo=True`: a host-only kernel (no GPU) whose model advances every active row by one token."""
        if echo:
            self._h = _lib().glint_kernel_create_echo(concurrency, max_contexts)
        else:
            flags = (FLAG_FUSED if fused else 0) | (FLAG_CLS if with_cls else 0) | (0 if fused_projections else FLAG_UNFUSED_PROJ)
            self._h = _lib().glint_kernel_create(config.encode(), 0 if dtype == "f16" else 1, first_layer, n_hosted,
                                                 concurrency, max_contexts, flags, seed, weight_std)
        if not self._h:
            raise GlintError(f"unknown kernel configuration {config!r}")
        self._poll = select.poll()
        self._poll.register(self.fileno(), select.POLLIN)

    def close(self) -> None:
        """Stops and joins the kernel's threads; states still inside are dropped."""
        if getattr(self, "_h", None):
            _lib().glint_kernel_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load(self, model_dir: str) -> None:
        if _lib().glint_kernel_load(self._h, os.fsencode(model_dir)) != 0:
            raise GlintError(_lib().glint_last_error().decode(errors="replace"))

    def push(self, raw: bytes) -> None:
        buf = C.create_string_buffer(raw, len(raw))
        if _lib().glint_kernel_push(self._h, C.cast(buf, C.c_void_p), len(raw)) != 0:
            raise GlintError(_lib().glint_last_error().decode(errors="replace"))

    def pop(self) -> Optional[bytes]:
        n = C.c_uint64(0)
        p = _lib().glint_kernel_pop(self._h, C.byref(n))
        return C.string_at(p, n.value) if p else None

    def fileno(self) -> int:
        return _lib().glint_kernel_event_fd(self._h)

    def read_event(self) -> int:
        """Number of states finished since the last read (0 when none); clears the counter."""
        n = C.c_uint64(0)
        return n.value if _lib().glint_kernel_read_event(self._h, C.byref(n)) else 0

    def wait(self, timeout_s: float) -> bool:
        """Blocks until the eventfd is readable or the timeout passes."""
        return bool(self._poll.poll(int(timeout_s * 1000)))

    def slot_counts(self) -> dict:
        out = (C.c_uint64 * 3)()
        _lib().glint_kernel_slot_counts(self._h, C.byref(out))
        return dict(free=out[0], allocated=out[1], total=out[2])
