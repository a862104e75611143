"""The CPU side under AddressSanitizer and UndefinedBehaviorSanitizer: the oracle's C restatement and the C++
host layer (bookkeeping, state wire format, loader, compute-kernel queues; host code only, no GPU) are rebuilt
with -fsanitize=address,undefined and their own test files are run again against those builds in a child
process that has the sanitizer runtime preloaded.  A finding aborts the child."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def run_suite(files, env_extra, runtime):
    env = dict(os.environ)
    env.update(env_extra)
    # the runtime has to be in the process before the interpreter starts; whatever is preloaded already stays in front of it
    env["LD_PRELOAD"] = ":".join(x for x in (os.environ.get("LD_PRELOAD", ""), runtime) if x)
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=1:halt_on_error=1"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    proc = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", *files], cwd=ROOT, env=env,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    tail = "\n".join(proc.stdout.splitlines()[-40:])
    assert proc.returncode == 0, tail
    assert " passed" in tail and "AddressSanitizer" not in proc.stdout and "runtime error" not in proc.stdout, tail
    return tail


def test_oracle_under_asan_and_ubsan():
    runtime = subprocess.run(["gcc", "-print-file-name=libasan.so"], stdout=subprocess.PIPE, text=True).stdout.strip()
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("gcc has no shared AddressSanitizer runtime here")
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "sanitize"], stdout=subprocess.DEVNULL)
    lib = os.path.join(ROOT, "oracle", "libglint_oracle_san.so")
    tail = run_suite(["tests/test_oracle_ops.py", "tests/test_oracle_book.py"], {"GLINT_ORACLE_LIB": lib, "OMP_NUM_THREADS": "4"}, runtime)
    assert "failed" not in tail


def test_host_layer_under_asan_and_ubsan():
    probe = subprocess.run([HIPCC, "-print-file-name=libclang_rt.asan-x86_64.so"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
    runtime = probe.stdout.strip()
    if probe.returncode != 0 or not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("this compiler has no shared AddressSanitizer runtime")
    from glinthawk_amd import build
    if not os.path.exists(build.LIB):
        pytest.skip("libglint_hip.so is not built")
    lib = build.build_host_sanitized()
    files = ["tests/test_host_book.py", "tests/test_host_state.py", "tests/test_host_loader.py", "tests/test_host_kernel.py"]
    tail = run_suite(files, {"GLINT_HOST_LIB": lib}, runtime)
    assert "failed" not in tail
