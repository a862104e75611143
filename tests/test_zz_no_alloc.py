"""gh_attn_decode_static: the fused decode attention for callers that cannot allocate.  Its split
partials live in a fixed array of the library's device image; the kernels, the plan and therefore the
result are those of gh_attn_decode, bit for bit.  Two calls in a row share the array (the second one
smaller, so stale partials of the first lie beyond what it writes), and a call that would need more
than the array holds is refused before anything is launched."""
import ctypes as C

import numpy as np
import pytest
import torch

from glinthawk_amd import _lib, ops
from glinthawk_amd._lib import GH_ATTN_AUTO, GH_ATTN_GENERIC, GH_ATTN_MFMA, GH_ATTN_VALU, GH_F16, Shape
from helpers import Arena

pytestmark = pytest.mark.gpu


def decode_static(q, rows, pos, xb, max_pos, shape, variant=GH_ATTN_AUTO):
    s = shape.c()
    return _lib.lib().gh_attn_decode_static(q.data_ptr(), rows.data_ptr(), pos.data_ptr(), xb.data_ptr(), rows.numel(), max_pos,
                                            C.byref(s), ops._dt(q), variant, torch.cuda.current_stream().cuda_stream)


def plan_bytes(batch, max_pos, shape, dt=GH_F16, variant=GH_ATTN_AUTO):
    s = shape.c()
    chunk, splits, need = C.c_uint32(0), C.c_uint32(0), C.c_uint64(0)
    _lib.check(_lib.lib().gh_attn_decode_plan(batch, max_pos, C.byref(s), dt, variant, C.byref(chunk), C.byref(splits), C.byref(need)))
    return splits.value, need.value


def run_both(shape, dtype, positions, seed, variant=GH_ATTN_AUTO, empty=()):
    batch = len(positions)
    arena = Arena(shape, batch, dtype, seed=seed)
    rng = np.random.default_rng(seed + 1)
    np_dt = np.float16 if dtype == torch.float16 else np.float32
    q = torch.from_numpy(rng.standard_normal((batch, shape.dim)).astype(np_dt)).cuda()
    rows = ops.row_table([0 if i in empty else arena.layer_ptr(i) for i in range(batch)])
    pos = torch.tensor(positions, dtype=torch.int32, device="cuda")
    max_pos = max(p for i, p in enumerate(positions) if i not in empty)
    want = torch.full((batch, shape.dim), 7.0, dtype=dtype, device="cuda")
    got = want.clone()
    ops.attn_decode(q, rows, pos, want, max_pos, shape, variant=variant)
    rc = decode_static(q, rows, pos, got, max_pos, shape, variant)
    assert rc == 0, _lib.lib().gh_last_error()
    ops.sync()
    return got, want


def test_static_scratch_entry_point_equals_the_workspace_one():
    ops.init(0)
    assert _lib.lib().gh_attn_decode_static_limit() == 16 << 20
    gqa = Shape(dim=2048, n_layers=1, n_heads=16, n_kv_heads=2, hidden_dim=64, seq_len=2048)      # head 128, gqa 8: MFMA kernel
    first = [2047, 1500, 1033, 300, 0]
    splits, need = plan_bytes(len(first), max(first), gqa)
    assert splits > 1 and 0 < need <= 16 << 20                                                    # the scratch array is really used
    got, want = run_both(gqa, torch.float16, first, seed=11)
    assert torch.equal(got, want)
    assert torch.isfinite(got.float()).all() and float(got.float().abs().max()) < 7.0             # every row was written
    # second call right behind it on the same array: fewer rows, shorter contexts, one context empty
    second = [700, 5, 257]
    splits2, need2 = plan_bytes(len(second), 700, gqa)
    assert splits2 > 1 and need2 < need
    got2, want2 = run_both(gqa, torch.float16, second, seed=12, empty=(1,))
    assert torch.equal(got2, want2)
    assert float(got2[1].float().min()) == 7.0 and float(got2[1].float().max()) == 7.0            # the empty context's row is untouched


@pytest.mark.parametrize("variant", [GH_ATTN_GENERIC, GH_ATTN_VALU, GH_ATTN_MFMA])
def test_static_scratch_entry_point_every_kernel(variant):
    ops.init(0)
    shape = Shape(dim=1024, n_layers=1, n_heads=8, n_kv_heads=2, hidden_dim=64, seq_len=1024)     # head 128, gqa 4
    got, want = run_both(shape, torch.float16, [1023, 511, 17, 600], seed=21, variant=variant)
    assert torch.equal(got, want)
    got, want = run_both(shape, torch.float16, [300, 40], seed=22, variant=variant)
    assert torch.equal(got, want)


def test_static_scratch_entry_point_fp32_and_no_split():
    ops.init(0)
    small = Shape(dim=288, n_layers=1, n_heads=6, n_kv_heads=6, hidden_dim=768, seq_len=256)      # stories15M shape, fp32, generic kernel
    got, want = run_both(small, torch.float32, [255, 100, 0, 31], seed=31)
    assert torch.equal(got, want)
    got, want = run_both(small, torch.float32, [9], seed=32)                                       # a single split: no partials at all
    assert torch.equal(got, want)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    ops.init(0)
    wide = Shape(dim=4096, n_layers=1, n_heads=32, n_kv_heads=2, hidden_dim=64, seq_len=1024)     # gqa 16
    batch = 300
    q = torch.zeros((batch, wide.dim), dtype=torch.float16, device="cuda")
    xb = torch.full((batch, wide.dim), 3.0, dtype=torch.float16, device="cuda")
    cache = torch.zeros((wide.seq_len, 2 * wide.kv_dim), dtype=torch.float16, device="cuda")      # every context reads the same rows
    rows = ops.row_table([cache.data_ptr()] * batch)
    pos = torch.full((batch,), 1023, dtype=torch.int32, device="cuda")
    # As the library would run this call its splits are added up inside the work-groups: nothing goes into the array.  With
    # that route switched off the plan's partial sums exceed it.
    assert plan_bytes(batch, 1023, wide)[1] == 0 and ops.attn_decode_join_waves(batch, 1023, wide) > 0
    ops.attn_set_split_join(0)
    try:
        splits, need = plan_bytes(batch, 1023, wide)
        assert need > 16 << 20
        rc = decode_static(q, rows, pos, xb, 1023, wide)
        assert rc == -5                                                                           # GH_ERR_WORKSPACE
        assert b"gh_attn_decode_static" in _lib.lib().gh_last_error() and b"available" in _lib.lib().gh_last_error()
        ops.sync()
        assert float(xb.float().min()) == 3.0                                                     # nothing was launched
        # the same call through the workspace entry point is fine
        ops.attn_decode(q, rows, pos, xb, 1023, wide)
        ops.sync()
        assert float(xb.float().abs().max()) == 0.0                                               # all-zero V rows
    finally:
        ops.attn_set_split_join(1)
    xb.fill_(3.0)
    assert decode_static(q, rows, pos, xb, 1023, wide) == 0
    ops.sync()
    assert float(xb.float().abs().max()) == 0.0


def test_static_scratch_entry_point_allocates_nothing():
    """The property the entry point exists for.  Around a call on a shape and batch this process has not run before (a plan of its
    own, several splits): the library's count of its own allocations stands still and so does the driver's count of free device
    memory; the same call through the workspace entry point is what the result is compared with, afterwards."""
    ops.init(0)
    L = _lib.lib()
    shape = Shape(dim=1536, n_layers=1, n_heads=12, n_kv_heads=3, hidden_dim=64, seq_len=1536)     # head 128, gqa 4; used nowhere else
    positions = [1535, 1201, 77, 640, 1024, 3]
    batch = len(positions)
    splits, need = plan_bytes(batch, max(positions), shape)
    assert splits > 1 and 0 < need <= 16 << 20
    arena = Arena(shape, batch, torch.float16, seed=51)
    rng = np.random.default_rng(52)
    q = torch.from_numpy(rng.standard_normal((batch, shape.dim)).astype(np.float16)).cuda()
    rows = ops.row_table([arena.layer_ptr(i) for i in range(batch)])
    pos = torch.tensor(positions, dtype=torch.int32, device="cuda")
    got = torch.full((batch, shape.dim), 7.0, dtype=torch.float16, device="cuda")
    want = got.clone()
    # the code object is on the device and the launch path warm before anything is counted (a first launch loads code)
    warm = Shape(dim=1024, n_layers=1, n_heads=8, n_kv_heads=2, hidden_dim=64, seq_len=1024)
    run_both(warm, torch.float16, [1023, 5], seed=53)
    torch.cuda.synchronize()
    allocations = int(L.gh_allocation_count())
    free_before, _ = torch.cuda.mem_get_info()
    rc = decode_static(q, rows, pos, got, max(positions), shape)
    ops.sync()
    free_after, _ = torch.cuda.mem_get_info()
    assert rc == 0, L.gh_last_error()
    assert int(L.gh_allocation_count()) == allocations          # no hipMalloc / hipHostMalloc / hipMemCreate of the library's
    assert free_after == free_before                            # and none of anybody else's on its behalf
    ops.attn_decode(q, rows, pos, want, max(positions), shape)
    ops.sync()
    assert torch.equal(got, want)
    assert int(L.gh_allocation_count()) == allocations          # (the workspace above is torch's, not the library's)
