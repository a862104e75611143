"""glinthawk_amd -- MI355X (gfx950) backend for Glinthawk's per-stage Llama2 KV-cache path.

The product is ``lib/libglint_hip.so`` (hand-written HIP kernels behind the C-ABI declared in
``include/glint_hip.h``) and the C++ host layer under ``host/`` that mirrors the reference's
``Operations`` / ``LlamaOperations`` / ``Context`` interface.  This Python package is only the
loader and thin ctypes bindings used by the tests and the benchmark; it holds no compute and no
CPU fallback: if the library is missing or no gfx950 device is present, calls raise.
"""
from ._lib import GlintError, Shape, lib, lib_path  # noqa: F401
