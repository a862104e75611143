"""Builds libglint_hip.so (the gfx950 kernels and their C-ABI) in-tree with hipcc.

Usage: ``python -m glinthawk_amd.build``.  hipcc cross-compiles for gfx950 without a GPU.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIB_DIR = os.path.join(PKG, "lib")
LIB = os.path.join(LIB_DIR, "libglint_hip.so")
HOST_LIB = os.path.join(LIB_DIR, "libglint_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# packed fp32 instructions are switched off for every device compile of this library
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-fPIC", "-Wall", "-Wno-unused-function", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        sys.stderr.write(out + "\n")
        raise RuntimeError("build failed: " + " ".join(cmd))
    if out.strip():
        print(out)


def build_kernels() -> str:
    """Every .hip source to an object file (in parallel), then one shared library."""
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(PKG, "build")
    os.makedirs(obj_dir, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    jobs = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 1, 16))
    objects = [os.path.join(obj_dir, os.path.splitext(os.path.basename(src))[0] + ".o") for src in sources]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _run([HIPCC, *DEVICE_FLAGS, *COMMON_FLAGS, "-std=c++17", "-c", so[0], "-o", so[1]]), zip(sources, objects)))
    _run([HIPCC, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", LIB, *objects])
    return LIB


def build_host() -> str | None:
    """The C++20 host layer (the reference-shaped classes) plus its C test hooks."""
    sources = sorted(glob.glob(os.path.join(HOST, "*.cc")))
    if not sources:
        return None
    os.makedirs(LIB_DIR, exist_ok=True)
    _run([HIPCC, *COMMON_FLAGS, "-std=c++20", "-x", "c++", "-I" + HOST, "-shared", "-o", HOST_LIB, *sources,
          "-L" + LIB_DIR, "-lglint_hip", "-Wl,-rpath,$ORIGIN", "-pthread"])
    return HOST_LIB


def build_host_sanitized() -> str:
    """The host layer with AddressSanitizer and UndefinedBehaviorSanitizer (host code only; GPU sanitizers are not used), for the
    CPU test suite: tests/test_sanitizers.py loads it through GLINT_HOST_LIB with the sanitizer runtime preloaded."""
    sources = sorted(glob.glob(os.path.join(HOST, "*.cc")))
    out = os.path.join(LIB_DIR, "libglint_host_san.so")
    _run([HIPCC, *COMMON_FLAGS[1:], "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
          "-shared-libasan", "-std=c++20", "-x", "c++", "-I" + HOST, "-shared", "-o", out, *sources,
          "-L" + LIB_DIR, "-lglint_hip", "-Wl,-rpath,$ORIGIN", "-pthread"])
    return out


def build_tools() -> list[str]:
    """profile-stage-hip and profile-gemm-hip: the reference's profiling front ends for this target."""
    built = []
    for src in sorted(glob.glob(os.path.join(HOST, "bin", "*.cc"))):
        name = os.path.splitext(os.path.basename(src))[0].replace("_", "-") + "-hip"
        exe = os.path.join(LIB_DIR, name)
        _run([HIPCC, *COMMON_FLAGS, "-std=c++20", "-x", "c++", "-I" + HOST, "-o", exe, src,
              "-L" + LIB_DIR, "-lglint_hip", "-Wl,-rpath,$ORIGIN", "-pthread"])
        built.append(exe)
    return built


def build_all() -> None:
    build_kernels()
    build_host()
    build_tools()


if __name__ == "__main__":
    build_all()
    print("built", LIB)
