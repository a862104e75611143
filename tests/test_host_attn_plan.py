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
