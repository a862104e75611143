"""The split plan of the fused decode attention is host logic.  A stage allocates its workspace once,
for its concurrency limit and the longest position; every legal call afterwards (any batch up to the
limit, any position) must fit into it, although a smaller batch is cut into more splits per context."""
import ctypes as C

import pytest

from glinthawk_amd import _lib
from glinthawk_amd._lib import GH_ATTN_AUTO, GH_ATTN_GENERIC, Shape

SHAPES = {
    "7B": Shape(dim=4096, n_layers=1, n_heads=32, n_kv_heads=32, hidden_dim=11008, seq_len=2048),
    "13B": Shape(dim=5120, n_layers=1, n_heads=40, n_kv_heads=40, hidden_dim=13824, seq_len=4096),
    "70B": Shape(dim=8192, n_layers=1, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096),
    "tiny": Shape(dim=288, n_layers=1, n_heads=6, n_kv_heads=6, hidden_dim=768, seq_len=256),
}


def plan(batch, max_pos, shape, dt, variant):
    s = shape.c()
    chunk, splits, need = C.c_uint32(0), C.c_uint32(0), C.c_uint64(0)
    _lib.check(_lib.lib().gh_attn_decode_plan(batch, max_pos, C.byref(s), dt, variant, C.byref(chunk), C.byref(splits), C.byref(need)))
    return chunk.value, splits.value, need.value


def workspace(batch, max_pos, shape):
    s = shape.c()
    return int(_lib.lib().gh_attn_decode_workspace(batch, max_pos, C.byref(s)))


@pytest.mark.parametrize("name", sorted(SHAPES))
@pytest.mark.parametrize("cap", [1, 8, 32, 64, 128, 256])
def test_workspace_of_the_limit_serves_every_smaller_batch(name, cap):
    shape = SHAPES[name]
    have = workspace(cap, shape.seq_len - 1, shape)
    positions = sorted({0, 1, 15, 16, 255, 256, 257, 511, 1000, shape.seq_len // 2, shape.seq_len - 2, shape.seq_len - 1} & set(range(shape.seq_len)))
    for batch in range(1, cap + 1):
        for max_pos in positions:
            for dt, variant in ((0, GH_ATTN_AUTO), (0, GH_ATTN_GENERIC), (1, GH_ATTN_AUTO)):
                chunk, splits, need = plan(batch, max_pos, shape, dt, variant)
                assert need <= have, (name, cap, batch, max_pos, dt, variant, need, have)
                assert chunk % 16 == 0 and splits >= 1
                assert (splits - 1) * chunk < max_pos + 1 <= splits * chunk          # every key in exactly one split


def test_the_case_that_used_to_overflow():
    # 70B shape, limit 64: a batch of 17 rows at the last position is cut into more partials than the full batch
    shape = SHAPES["70B"]
    _, _, need17 = plan(17, 4095, shape, 0, GH_ATTN_AUTO)
    _, _, need64 = plan(64, 4095, shape, 0, GH_ATTN_AUTO)
    assert need17 > need64
    assert workspace(64, 4095, shape) >= need17


def test_workspace_grows_with_the_limit():
    shape = SHAPES["70B"]
    sizes = [workspace(b, 4095, shape) for b in (1, 2, 16, 17, 64, 65, 256)]
    assert sizes == sorted(sizes)


def join_waves(batch, max_pos, shape, dt=0, variant=GH_ATTN_AUTO):
    s = shape.c()
    return int(_lib.lib().gh_attn_decode_join_waves(batch, max_pos, C.byref(s), dt, variant))


def test_joined_plans_are_well_formed_and_the_workspace_serves_both_routes():
    """Where a plan's splits are added up inside the work-groups it has 2 or 4 splits of at least 256 keys, work-groups of 4 or 8
    waves that hold whole streams, and asks for no workspace; with that route switched off the same call's partial sums still
    fit the workspace that was sized beforehand, whichever way the switch stood then."""
    L = _lib.lib()
    for name in ("7B", "13B", "70B"):
        shape = SHAPES[name]
        have = workspace(256, shape.seq_len - 1, shape)
        joined = 0
        for batch in list(range(1, 70)) + [80, 96, 100, 128, 130, 160, 200, 256]:
            for max_pos in (255, 511, 1023, 1500, shape.seq_len - 1):
                waves = join_waves(batch, max_pos, shape)
                chunk, splits, need = plan(batch, max_pos, shape, 0, GH_ATTN_AUTO)
                assert waves in (0, 4, 8)
                if waves:
                    joined += 1
                    assert splits in (2, 4) and splits <= waves and chunk >= 256 and need == 0
                _lib.check(L.gh_attn_set_split_join(0))
                try:
                    assert join_waves(batch, max_pos, shape) == 0
                    _, splits_off, need_off = plan(batch, max_pos, shape, 0, GH_ATTN_AUTO)
                    assert need_off <= have and (splits_off == 1) == (need_off == 0)
                    if waves:
                        assert splits_off >= splits                     # joined plans never cut finer than the route with partial sums
                finally:
                    _lib.check(L.gh_attn_set_split_join(1))
        assert joined > 20
    # fp32 and the generic kernel never join
    assert join_waves(64, 4095, SHAPES["70B"], dt=1) == 0
    assert join_waves(64, 4095, SHAPES["70B"], variant=GH_ATTN_GENERIC) == 0
    assert join_waves(64, 255, SHAPES["tiny"]) == 0


def test_joined_plans_of_the_benchmark_shapes():
    # (waves per work-group, splits) as measured best: see join_choice in csrc/gh_attn_decode.hip
    def both(batch, max_pos, shape):
        return join_waves(batch, max_pos, shape), plan(batch, max_pos, shape, 0, GH_ATTN_AUTO)[1]
    assert both(64, 4095, SHAPES["70B"]) == (8, 4)       # the headline configuration: 2 kv heads x 4 splits per work-group
    assert both(32, 1023, SHAPES["7B"]) == (4, 2)
    assert both(32, 1150, SHAPES["7B"]) == (4, 2)
    assert both(32, 4095, SHAPES["70B"]) == (4, 4)
    assert both(96, 4095, SHAPES["70B"]) == (8, 2)
    assert both(8, 2047, SHAPES["13B"]) == (8, 4)
    assert both(16, 4095, SHAPES["70B"])[0] == 0         # too few streams: many short splits and the merge kernel
    assert both(256, 4095, SHAPES["70B"])[0] == 0        # a stream per wave slot: no split at all
    assert both(32, 2047, SHAPES["13B"])[0] == 0
