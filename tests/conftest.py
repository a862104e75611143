import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    """Keeps the measured fp16 distances of the stage tests (helpers.DRIFT) next to the other GPU run outputs."""
    try:
        import helpers
    except Exception:
        return
    if not helpers.DRIFT:
        return
    out = os.path.join(ROOT, os.environ.get("GLINT_TEST_OUTPUT_DIR", "gpurun_out"))
    os.makedirs(out, exist_ok=True)
    with open(os.path.join(out, "fp16_drift.txt"), "w") as f:
        f.write("mean-relative distances: HIP vs fp16 oracle | HIP vs fp32 oracle | fp16 oracle vs fp32 oracle\n")
        worst = {}
        for what, r16, r32, rs in helpers.DRIFT:
            key = what.split(" step ")[0]
            w = worst.setdefault(key, [0.0, 0.0, 0.0, 0])
            w[0], w[1], w[2], w[3] = max(w[0], r16), max(w[1], r32), max(w[2], rs), w[3] + 1
        for key, (r16, r32, rs, n) in worst.items():
            f.write(f"{key}: max over {n} outputs  {r16:.3e} | {r32:.3e} | {rs:.3e}\n")


@pytest.fixture(params=["vendor-library", "own-kernels"])
def product_route(request):
    """Plain products of many rows both ways: through the vendor's GEMM library (the default from 768 rows on) and on
    the tile kernels of this library."""
    from glinthawk_amd import _lib
    _lib.check(_lib.lib().gh_gemm_set_library_rows(768 if request.param == "vendor-library" else 0))
    yield request.param
    _lib.check(_lib.lib().gh_gemm_set_library_rows(768))
