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


LIBRARY_ROWS = 768   # the row count the vendor-library route is tested at (the library's default is 0: never)


class ProductRoute(str):
    """Which GEMM route a test runs on, and a check that it did: the vendor library declines silently (no library, no
    algorithm) and the product then runs on the tile kernels, so a test that means to cover the library route asks the
    library's own call counter."""

    ROWS = LIBRARY_ROWS

    def library_calls(self) -> int:
        from glinthawk_amd import _lib
        return int(_lib.lib().gh_gemm_library_calls()) - self.calls_at_start

    @staticmethod
    def wanted(b: int, s: int, r: int) -> bool:
        """gh_matmul's rule for a plain f16 product of 16-byte aligned operands at LIBRARY_ROWS."""
        rows_enough = b >= LIBRARY_ROWS or (2 * b >= LIBRARY_ROWS and 2 * r >= s)
        return rows_enough and s % 8 == 0 and r % 8 == 0

    def check(self, expected_calls=None) -> None:
        """After the test's products: the library ran `expected_calls` of them (None: at least one) on its route, none on
        the other."""
        if self != "vendor-library":
            assert self.library_calls() == 0, "the vendor library ran although the own-kernel route was asked for"
            return
        got = self.library_calls()
        if got == 0 and expected_calls != 0:
            import ctypes
            try:
                ctypes.CDLL("libhipblaslt.so.1")
            except OSError as e:
                pytest.skip(f"libhipblaslt.so.1 cannot be loaded ({e}): the vendor-library route cannot run here")
        if expected_calls is None:
            assert got > 0, "the vendor library ran no product on its own route"
        else:
            assert got == expected_calls, f"the vendor library ran {got} products, {expected_calls} expected"


@pytest.fixture(params=["vendor-library", "own-kernels"])
def product_route(request):
    """Plain products of many rows both ways: on the tile kernels of this library (the default) and through the vendor's
    GEMM library (opt-in, here from LIBRARY_ROWS rows on)."""
    from glinthawk_amd import _lib
    L = _lib.lib()
    before = int(L.gh_gemm_library_rows())
    _lib.check(L.gh_gemm_set_library_rows(LIBRARY_ROWS if request.param == "vendor-library" else 0))
    route = ProductRoute(request.param)
    route.calls_at_start = int(L.gh_gemm_library_calls())
    yield route
    _lib.check(L.gh_gemm_set_library_rows(before))
