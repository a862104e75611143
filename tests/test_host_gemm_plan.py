"""The weight-streaming GEMM's plan (K split and row tile) is host logic: properties every plan must
have, and the plans of the shapes the benchmark configurations use (256 compute units, the value
the library assumes before a device is initialised)."""
import ctypes as C

import numpy as np
import pytest

from glinthawk_amd import _lib


def plan(s, r, b):
    splits, kps, rows = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    _lib.check(_lib.lib().gh_gemm_stream_plan(s, r, b, C.byref(splits), C.byref(kps), C.byref(rows)))
    return splits.value, kps.value, rows.value


def test_every_plan_covers_k_exactly_once():
    rng = np.random.default_rng(5)
    shapes = [(256, 4, 1), (256, 100000, 64), (1 << 16, 128, 3)]
    shapes += [(256 * int(rng.integers(1, 200)), 4 * int(rng.integers(1, 20000)), int(rng.integers(1, 300))) for _ in range(300)]
    for s, r, b in shapes:
        splits, kps, rows = plan(s, r, b)
        assert splits >= 1 and kps % 256 == 0 and kps >= 256
        assert (splits - 1) * kps < s <= splits * kps, (s, r, b, splits, kps)      # no empty range, nothing left over
        assert rows in (96, 112, 128)
        if splits > 1:
            assert rows == 128 and kps >= 512, (s, r, b, splits, kps, rows)          # small tiles only without a split; at least two slabs per range
        assert splits <= 16


@pytest.mark.parametrize("name,s,r,b,want", [
    ("70B wo", 8192, 8192, 64, (4, 2048, 128)),                 # 64 row blocks x 4 = one work-group per CU
    ("70B wq+wkv", 8192, 10240, 64, (3, 2816, 128)),            # 80 x 3 = 240, not 320
    ("70B w2", 28672, 8192, 64, (8, 3584, 128)),                # two work-groups per CU
    ("70B w1+w3", 8192, 57344, 64, (1, 8192, 112)),             # 512 work-groups of 112 rows instead of 448 of 128
    ("7B wo", 4096, 4096, 32, (8, 512, 128)),
    ("13B w1+w3", 5120, 27648, 8, (2, 2560, 128)),
])
def test_plans_of_the_benchmark_shapes(name, s, r, b, want):
    assert plan(s, r, b) == want, name


def test_rejects_what_the_kernel_does_not_take():
    splits, kps, rows = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    rc = _lib.lib().gh_gemm_stream_plan(100, 64, 1, C.byref(splits), C.byref(kps), C.byref(rows))
    assert rc != 0 and b"256" in _lib.lib().gh_last_error()
