"""GPU parity tests, op by op, through the C-ABI against the CPU oracle on the same seeded inputs.

Bit-exact: KV append.  Everything floating point: the north-star tolerance (2e-2 max-abs, 1e-3
mean-relative) against the oracle's fp32 path, and tighter self-consistency bounds where stated."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O
from glinthawk_amd import Shape, _lib, ops
from glinthawk_amd._lib import GH_ATTN_AUTO, GH_ATTN_GENERIC, GH_ATTN_MFMA, GH_ATTN_VALU, GlintError
from helpers import half_ulp_diff, Arena, assert_close, errors, oracle_cfg

pytestmark = pytest.mark.gpu

TINY = Shape(dim=32, n_layers=2, n_heads=4, n_kv_heads=2, hidden_dim=48, seq_len=16, vocab_size=64)
STORIES = Shape(dim=288, n_layers=6, n_heads=6, n_kv_heads=6, hidden_dim=768, seq_len=256)      # config 1 shape
MHA128 = Shape(dim=512, n_layers=1, n_heads=4, n_kv_heads=4, hidden_dim=64, seq_len=640)          # 7B-like heads
MHA128_ODD = Shape(dim=768, n_layers=1, n_heads=6, n_kv_heads=6, hidden_dim=64, seq_len=300)      # kv heads % 4 != 0
GQA8 = Shape(dim=2048, n_layers=1, n_heads=16, n_kv_heads=2, hidden_dim=64, seq_len=700)          # 70B-like heads
GQA4 = Shape(dim=1536, n_layers=1, n_heads=12, n_kv_heads=3, hidden_dim=64, seq_len=330)
GQA2 = Shape(dim=1024, n_layers=1, n_heads=8, n_kv_heads=4, hidden_dim=64, seq_len=280)
GQA16 = Shape(dim=2048, n_layers=1, n_heads=16, n_kv_heads=1, hidden_dim=64, seq_len=300)


def tdt(name):
    return torch.float16 if name == "f16" else torch.float32


def ndt(name):
    return np.float16 if name == "f16" else np.float32


@pytest.fixture(scope="module", autouse=True)
def _init():
    ops.init(0)
    assert ops.device_name().startswith("gfx950")
    yield
    ops.attn_set_chunk(0)


# ------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("batch,size", [(1, 8), (3, 37), (4, 288), (64, 8192)])
def test_accum(dt, batch, size):
    rng = np.random.default_rng(1)
    a = rng.standard_normal((batch, size)).astype(ndt(dt))
    b = rng.standard_normal((batch, size)).astype(ndt(dt))
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    ops.accum(da, db)
    O.accum(a, b)
    # one fp32 add and one rounding on both sides: identical bits
    assert np.array_equal(da.cpu().numpy().view(np.uint8), a.view(np.uint8))


@pytest.mark.parametrize("dt,tol", [("f16", 2e-3), ("f32", 2e-6)])
@pytest.mark.parametrize("batch,size", [(1, 8), (4, 288), (5, 100), (64, 8192)])
def test_rmsnorm(dt, tol, batch, size):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((batch, size)).astype(ndt(dt))
    w = (1 + 0.1 * rng.standard_normal(size)).astype(ndt(dt))
    dx, dw = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    got = ops.rmsnorm(dx, dw).cpu().numpy()
    want = O.rmsnorm(x, w)
    np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=tol, atol=tol)
    if dt == "f16":
        # against the fp16-storage instantiation: same rounding points, only the order of the sum of squares differs
        worst, differing = half_ulp_diff(got, want)
        assert worst <= 1 and differing < 0.01, (worst, differing)
    want32 = O.rmsnorm(x.astype(np.float32), w.astype(np.float32))
    assert_close(got, want32, what="rmsnorm vs fp32 path")
    # in place
    ops.rmsnorm(dx, dw, out=dx)
    assert np.array_equal(dx.cpu().numpy(), got)


@pytest.mark.parametrize("dt,tol", [("f16", 2e-3), ("f32", 3e-6)])
@pytest.mark.parametrize("batch,hidden", [(1, 8), (4, 768), (3, 1001), (64, 28672)])
def test_silu(dt, tol, batch, hidden):
    rng = np.random.default_rng(3)
    x = (2 * rng.standard_normal((batch, hidden))).astype(ndt(dt))
    y = rng.standard_normal((batch, hidden)).astype(ndt(dt))
    dx, dy = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    ops.silu(dx, dy)
    O.silu(x, y)
    np.testing.assert_allclose(dx.cpu().numpy().astype(np.float64), x.astype(np.float64), rtol=tol, atol=tol)
    if dt == "f16":
        # one rounding per element on both sides; the exponential is the only difference
        worst, differing = half_ulp_diff(dx.cpu().numpy(), x)
        assert worst <= 1 and differing < 1e-3, (worst, differing)


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_argmax_bit_exact(dt):
    rng = np.random.default_rng(4)
    v = rng.standard_normal((7, 32000)).astype(ndt(dt))
    v[1, 17] = v[1, 20000] = 9.0     # tie across waves: first index
    v[2, :] = 0.5                    # all equal
    v[3, 31999] = 50.0
    v[4, 0] = 50.0
    v[5, 255] = v[5, 256] = 11.0     # tie across neighbouring threads
    dv = torch.from_numpy(v).cuda()
    got = ops.argmax(dv)
    assert got == O.argmax(v).tolist()
    small = rng.standard_normal((3, 5)).astype(ndt(dt))
    assert ops.argmax(torch.from_numpy(small).cuda()) == O.argmax(small).tolist()


def test_soft_sample_only_touches_warm_rows():
    rng = np.random.default_rng(5)
    v = rng.standard_normal((3, 1000)).astype(np.float32)
    dv = torch.from_numpy(v).cuda()
    ops.soft_sample(dv, [0.0, 0.7, 0.0], seed=9)
    got = dv.cpu().numpy()
    assert np.array_equal(got[0], v[0]) and np.array_equal(got[2], v[2])
    # row 1 = v / T - log(-log(u)) for some u in (0,1): recover u and check its range and spread
    noise = v[1].astype(np.float64) / 0.7 - got[1]
    u = np.exp(-np.exp(noise))
    assert np.all((u > 0) & (u < 1)) and 0.4 < u.mean() < 0.6
    # greedy batches are a no-op
    dv2 = torch.from_numpy(v).cuda()
    ops.soft_sample(dv2, [0.0, 0.0, 0.0])
    assert np.array_equal(dv2.cpu().numpy(), v)


def test_fill_is_seeded_and_distributed():
    t = torch.empty(1 << 20, dtype=torch.float16, device="cuda")
    ops.fill_normal(t, 0.0, 1.0, seed=42)
    a = t.float().cpu().numpy()
    ops.fill_normal(t, 0.0, 1.0, seed=42)
    assert np.array_equal(a, t.float().cpu().numpy())
    ops.fill_normal(t, 0.0, 1.0, seed=43)
    assert not np.array_equal(a, t.float().cpu().numpy())
    assert abs(a.mean()) < 0.01 and abs(a.std() - 1) < 0.01
    u = torch.empty(100003, dtype=torch.float32, device="cuda")
    ops.fill_uniform(u, -2.0, 3.0, seed=1)
    un = u.cpu().numpy()
    assert un.min() >= -2.0 and un.max() <= 3.0 and abs(un.mean() - 0.5) < 0.05


# ------------------------------------------------------------------ matmul
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("b,s,r", [(1, 8, 8), (4, 288, 288), (4, 288, 768), (3, 100, 37), (64, 1024, 512),
                                   (5, 768, 1000), (70, 512, 130), (32, 4096, 256)])
def test_matmul(dt, b, s, r):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((b, s)).astype(ndt(dt))
    w = (rng.standard_normal((r, s)) / np.sqrt(s)).astype(ndt(dt))
    got = ops.matmul(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    want = O.matmul(x.astype(np.float32), w.astype(np.float32))
    assert got.shape == (b, r)
    assert_close(got, want, what=f"matmul {dt} {b}x{s}x{r}")
    if dt == "f32":
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)


# many rows of x at once (prompt tokens): the MFMA tile kernel, ragged edges in both dimensions
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("b,s,r", [(128, 64, 128), (130, 512, 200), (257, 288, 288), (300, 72, 37), (512, 1024, 130),
                                   (1000, 776, 514), (129, 100, 64)])
def test_matmul_many_rows(dt, b, s, r):
    rng = np.random.default_rng(16)
    x = rng.standard_normal((b, s)).astype(ndt(dt))
    w = (rng.standard_normal((r, s)) / np.sqrt(s)).astype(ndt(dt))
    got = ops.matmul(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    want = O.matmul(x.astype(np.float32), w.astype(np.float32))
    assert got.shape == (b, r)
    assert_close(got, want, what=f"matmul {dt} {b}x{s}x{r}")


# enough 256-token tiles for the second tile kernel (forced with 256 and with 384 rows per work-group, and
# whatever the dispatcher picks), ragged edges; the row counts leave 4, 0 and 6 (256) / 3, 6 and 7 (384)
# row tiles beyond a multiple of 8, the part of the tile order that is cut into equal runs per XCD
@pytest.mark.parametrize("force,rows", [(4, 256), (4, 384), (4, 128), (4, 129), (4, 0), (0, 0)])
@pytest.mark.parametrize("b,s,r", [(3000, 8192, 4100), (8200, 128, 8190), (700, 8256, 18000)])
def test_matmul_256_tiles(force, rows, b, s, r):
    from glinthawk_amd import _lib
    if rows in (128, 129) and s % 128:
        pytest.skip("the four-wave kernel (tile rows 128: one tile per work-group, 129: equal shares of all steps) takes K ranges of an even "
                    "number of 64-k steps; the dispatcher takes the eight-wave one here")
    rng = np.random.default_rng(26)
    x = rng.standard_normal((b, s)).astype(np.float16)
    w = (rng.standard_normal((r, s)) / np.sqrt(s)).astype(np.float16)
    _lib.lib().gh_gemm_set_tuning(force, 0, rows)
    try:
        got = ops.matmul(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda())
    finally:
        _lib.lib().gh_gemm_set_tuning(0, 0, 0)
    want = (torch.from_numpy(x).cuda().float() @ torch.from_numpy(w).cuda().float().t())
    err = (got.float() - want).abs()
    assert got.shape == (b, r) and err.max().item() < 2e-2 and (err.mean() / want.abs().mean()).item() < 1e-3
    # a strip against the CPU oracle as well
    want_cpu = O.matmul(x[:8].astype(np.float32), w.astype(np.float32))
    assert_close(got[:8].cpu().numpy(), want_cpu, what=f"matmul 256-tile {b}x{s}x{r}")


@pytest.mark.parametrize("rows", [256, 384, 128, 129])
@pytest.mark.parametrize("s,r,b", [(8192, 12544, 1030),    # 49 / 33 row tiles x 5: one left-over row tile
                                   (1024, 5000, 16390),    # 20 / 14 row tiles x 65: 4 / 6 left over, ragged last token tile
                                   (256, 1700, 9000)])     # 7 / 5 row tiles: left-over tiles only
def test_matmul_256_tile_one_hot_layout(rows, s, r, b):
    """One-hot activations: every output is one weight, so each tile of the order must land bit for bit."""
    from glinthawk_amd import _lib
    w = torch.arange(r * s, dtype=torch.float32, device="cuda").reshape(r, s).remainder(1000).half()
    x = torch.zeros((b, s), dtype=torch.float16, device="cuda")
    cols = [(7919 * i + 3) % s for i in range(b)]
    x[torch.arange(b), torch.tensor(cols)] = 1
    _lib.lib().gh_gemm_set_tuning(4, 0, rows)
    try:
        got = ops.matmul(x, w)
    finally:
        _lib.lib().gh_gemm_set_tuning(0, 0, 0)
    assert torch.equal(got, w[:, cols].t().contiguous())


@pytest.mark.parametrize("epilogue", ["store", "accum", "pair"])
def test_matmul_equal_shares_of_all_steps(epilogue):
    """The four-wave kernel over equal shares of all 64-k steps (tile rows 129): shares that end inside tiles leave pieces that a
    second kernel adds in a fixed order.  Ragged tiles in both directions, shares shorter and longer than a tile, all three outputs
    (plain, residual add, two matrices); one-hot activations bit for bit, a random product twice with identical bits."""
    from glinthawk_amd import _lib
    for b, s, r in [(3000, 1280, 4104), (1100, 2560, 15880), (2300, 768, 8968)]:     # 204, 315 and 324 tiles of 20, 40 and 12 steps; shares of 16, 50 and 16
        w = torch.arange(r * s, dtype=torch.float32, device="cuda").reshape(r, s).remainder(1000).half()
        hot = torch.zeros((b, s), dtype=torch.float16, device="cuda")
        cols = torch.tensor([(7919 * i + 3) % s for i in range(b)], device="cuda")
        hot[torch.arange(b, device="cuda"), cols] = 1
        g = torch.Generator(device="cuda").manual_seed(b + r)
        x = torch.randn((b, s), generator=g, device="cuda").half()
        wr = (torch.randn((r, s), generator=g, device="cuda") / s ** 0.5).half()
        res = torch.randn((b, r), generator=g, device="cuda").half()
        _lib.lib().gh_gemm_set_tuning(4 if epilogue == "store" else 0, 0, 129)
        try:
            if epilogue == "store":
                got_hot, first, again = ops.matmul(hot, w), ops.matmul(x, wr), ops.matmul(x, wr)
                want_hot = w[:, cols].t().contiguous()
                want = x.float() @ wr.float().t()
            elif epilogue == "accum":
                got_hot = res.clone()
                ops.matmul_accum(got_hot, hot, w)
                first, again = res.clone(), res.clone()
                ops.matmul_accum(first, x, wr)
                ops.matmul_accum(again, x, wr)
                want_hot = (res.float() + w[:, cols].t().float()).half()
                want = res.float() + (x.float() @ wr.float().t()).half().float()
            else:
                ra = (r // 16) * 8
                a, c = ops.matmul_pair(hot, w, ra)
                got_hot = torch.cat([a, c], dim=1)
                first, again = (torch.cat(ops.matmul_pair(x, wr, ra), dim=1) for _ in range(2))
                want_hot = w[:, cols].t().contiguous()
                want = x.float() @ wr.float().t()
        finally:
            _lib.lib().gh_gemm_set_tuning(0, 0, 0)
        assert torch.equal(got_hot, want_hot), (b, s, r)
        assert torch.equal(first, again), (b, s, r)
        err = (first.float() - want).abs()
        assert err.max().item() < 2e-2 and (err.mean() / want.abs().mean()).item() < 1e-3, (b, s, r)


def test_matmul_many_rows_layout_one_hot():
    # x rows that select single columns of w: the tile kernel must return them bit for bit
    s, r, b = 320, 200, 260
    w = torch.arange(r * s, dtype=torch.float32).reshape(r, s).remainder(1000).half().cuda()
    x = torch.zeros((b, s), dtype=torch.float16, device="cuda")
    cols = [(7 * i + 3) % s for i in range(b)]
    x[torch.arange(b), torch.tensor(cols)] = 1
    got = ops.matmul(x, w)
    assert torch.equal(got, w[:, cols].t().contiguous())


def _streaming_shapes():
    rng = np.random.default_rng(77)
    shapes = [(64, 8192, 10240), (64, 2048, 57344), (33, 1024, 28672), (200, 512, 1100)]   # 3 splits; 112-row tiles; ragged batch; 4 column slabs
    for _ in range(20):
        shapes.append((int(rng.integers(1, 200)), 256 * int(rng.integers(1, 24)), 4 * int(rng.integers(1, 5000))))
    return shapes


@pytest.mark.parametrize("b,s,r", _streaming_shapes())
def test_matmul_streaming_kernel_sweep(b, s, r):
    """The weight-streaming kernel forced on shapes that walk through its plans: K splits, row tiles
    below 128, ragged last row blocks, one to four column slabs.  One-hot activations make the check
    bit exact (every output is one weight), a random product bounds the arithmetic."""
    from glinthawk_amd import _lib
    g = torch.Generator(device="cuda").manual_seed(b * 7 + r)
    w = (torch.randn((r, s), generator=g, device="cuda") / s ** 0.5).half()
    hot = torch.zeros((b, s), dtype=torch.float16, device="cuda")
    cols = torch.tensor([(7919 * i + 3) % s for i in range(b)], device="cuda")
    hot[torch.arange(b, device="cuda"), cols] = 1
    x = torch.randn((b, s), generator=g, device="cuda").half()
    _lib.lib().gh_gemm_set_tuning(2, 0, 0)
    try:
        got_hot = ops.matmul(hot, w)
        got = ops.matmul(x, w)
    finally:
        _lib.lib().gh_gemm_set_tuning(0, 0, 0)
    assert torch.equal(got_hot, w[:, cols].t().contiguous())
    want = x.float() @ w.float().t()
    err = (got.float() - want).abs()
    assert err.max().item() < 2e-2 and (err.mean() / want.abs().mean()).item() < 1e-3


# some hundred rows (the decode step of a large slot arena): whatever the dispatcher picks at each batch size (streaming kernel up
# to 64 rows, 128 x 128 tiles with or without a K split, 256-token tiles with the K range split over work-groups when the tiles are
# few), ragged edges in rows, tokens and K steps.  One-hot activations: every output is one weight, bit for bit.
@pytest.mark.parametrize("b", [65, 128, 192, 256, 300, 512])
@pytest.mark.parametrize("s,r", [(2048, 1024), (2112, 1000), (8192, 2560), (4096, 516)])
def test_matmul_some_hundred_rows(b, s, r):
    g = torch.Generator(device="cuda").manual_seed(b * 13 + r)
    w = (torch.randn((r, s), generator=g, device="cuda") / s ** 0.5).half()
    hot = torch.zeros((b, s), dtype=torch.float16, device="cuda")
    cols = torch.tensor([(7919 * i + 3) % s for i in range(b)], device="cuda")
    hot[torch.arange(b, device="cuda"), cols] = 1
    x = torch.randn((b, s), generator=g, device="cuda").half()
    got_hot = ops.matmul(hot, w)
    got = ops.matmul(x, w)
    assert torch.equal(got_hot, w[:, cols].t().contiguous())
    want = x.float() @ w.float().t()
    err = (got.float() - want).abs()
    assert err.max().item() < 2e-2 and (err.mean() / want.abs().mean()).item() < 1e-3


# many rows whose 256-token tiles would leave the last round nearly empty: the library runs such a product as two products along
# the tokens (here 2048 + 252 and 4096 + 404 tokens); one-hot activations, every output is one weight
@pytest.mark.parametrize("b,s,r", [(2300, 512, 8192), (4500, 256, 8192), (2300, 512, 8200)])
def test_matmul_token_split_one_hot(b, s, r, product_route):
    w = torch.arange(r * s, dtype=torch.float32, device="cuda").reshape(r, s).remainder(1000).half()
    x = torch.zeros((b, s), dtype=torch.float16, device="cuda")
    cols = torch.tensor([(7919 * i + 3) % s for i in range(b)], device="cuda")
    x[torch.arange(b, device="cuda"), cols] = 1
    got = ops.matmul(x, w)
    assert torch.equal(got, w[:, cols].t().contiguous())
    product_route.check(1)


# two products that share their activations (wq and wkv): few rows take the two-call route, many rows one launch of the large tile
# kernel whose work-groups store to the matrix their rows belong to, also cut along the tokens; one-hot activations, bit for bit
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("b,s,ra,rb", [(3, 256, 64, 32), (300, 512, 512, 200), (2048, 256, 8192, 2048), (2300, 256, 8192, 2048),
                                       (1500, 320, 5120, 10240), (1024, 256, 8200, 2056), (1024, 256, 8196, 2052)])
def test_matmul_pair(dt, b, s, ra, rb, product_route):
    if dt == "f32" and b > 300:
        pytest.skip("the fp32 route is the same two calls at every size")
    tdt = torch.float16 if dt == "f16" else torch.float32
    w = torch.arange((ra + rb) * s, dtype=torch.float32, device="cuda").reshape(ra + rb, s).remainder(1000).to(tdt)
    x = torch.zeros((b, s), dtype=tdt, device="cuda")
    cols = torch.tensor([(7919 * i + 3) % s for i in range(b)], device="cuda")
    x[torch.arange(b, device="cuda"), cols] = 1
    got_a, got_b = ops.matmul_pair(x, w, ra)
    assert got_a.shape == (b, ra) and got_b.shape == (b, rb)
    assert torch.equal(got_a, w[:ra, cols].t().contiguous())
    assert torch.equal(got_b, w[ra:, cols].t().contiguous())
    g = torch.Generator(device="cuda").manual_seed(b + ra)
    xr = torch.randn((b, s), generator=g, device="cuda").to(tdt)
    wr = (torch.randn((ra + rb, s), generator=g, device="cuda") / s ** 0.5).to(tdt)
    got_a, got_b = ops.matmul_pair(xr, wr, ra)
    want = xr.float() @ wr.float().t()
    err = (torch.cat([got_a, got_b], dim=1).float() - want).abs()
    assert err.max().item() < 2e-2 and (err.mean() / want.abs().mean()).item() < 1e-3
    both = dt == "f16" and product_route.wanted(b, s, ra) and product_route.wanted(b, s, rb)   # else one launch of the tile kernel, or two plain calls
    product_route.check(4 if both else 0)


def test_matmul_many_rows_repeatable(product_route):
    # the same product twice, other work in between: bit-identical results on either route (no sums in arrival order)
    b, s, r = 3328, 1024, 2560
    g = torch.Generator(device="cuda").manual_seed(77)
    x = torch.randn((b, s), generator=g, device="cuda").half()
    w = (torch.randn((r, s), generator=g, device="cuda") / s ** 0.5).half()
    first = ops.matmul(x, w)
    ops.matmul(torch.flip(x, dims=[0]).contiguous(), w)
    again = ops.matmul(x, w)
    assert torch.equal(first, again)
    product_route.check(3)
    want = x.float() @ w.float().t()
    err = (first.float() - want).abs()
    assert err.max().item() < 2e-2 and (err.mean() / want.abs().mean()).item() < 1e-3


def test_matmul_layout_one_hot():
    s, r = 256, 192
    w = torch.arange(r * s, dtype=torch.float32).reshape(r, s).remainder(1000).half().cuda()
    x = torch.zeros((3, s), dtype=torch.float16, device="cuda")
    x[0, 2] = x[1, 255] = x[2, 128] = 1
    got = ops.matmul(x, w)
    assert torch.equal(got[0], w[:, 2]) and torch.equal(got[1], w[:, 255]) and torch.equal(got[2], w[:, 128])


# ------------------------------------------------------------------ KV append (bit exact)
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("shape", [TINY, STORIES, GQA8], ids=["tiny", "stories15m", "gqa8"])
@pytest.mark.parametrize("host_tables", [False, True])
def test_kv_append_bit_exact(dt, shape, host_tables):
    batch = 5
    arena = Arena(shape, batch, tdt(dt), seed=7)
    rng = np.random.default_rng(8)
    kv = rng.standard_normal((batch, 2 * shape.kv_dim)).astype(ndt(dt))
    U = np.uint16 if dt == "f16" else np.uint32
    kv.view(U)[0, 1] = 0x7e01 if dt == "f16" else 0x7fc00123      # NaN payload must survive
    pos = [0, 3, shape.seq_len - 1, 7, 1]
    present = [True, True, True, False, True]
    rows = [arena.row_ptr(i, pos[i]) if present[i] else 0 for i in range(batch)]
    dkv = torch.from_numpy(kv).cuda()
    if host_tables:
        ops.kv_append_host(rows, dkv, shape.kv_dim)
    else:
        ops.kv_append(ops.row_table(rows), dkv, shape.kv_dim)
    want = arena.host.copy()
    O.copy_kv_cache(oracle_cfg(shape), [want[i, pos[i]] if present[i] else None for i in range(batch)], kv)
    got = arena.dev.cpu().numpy()
    assert np.array_equal(got.view(U), want.view(U))


# ------------------------------------------------------------------ RoPE
@pytest.mark.parametrize("dt,tol", [("f16", 2e-3), ("f32", 3e-6)])
@pytest.mark.parametrize("shape", [TINY, STORIES, GQA8, MHA128], ids=["tiny", "stories15m", "gqa8", "mha128"])
@pytest.mark.parametrize("host_tables", [False, True])
def test_rope(dt, tol, shape, host_tables):
    batch = 4
    arena = Arena(shape, batch, tdt(dt), seed=9)
    re32, im32 = O.rope_tables(shape.seq_len, shape.head_size)
    re, im = re32.astype(ndt(dt)), im32.astype(ndt(dt))
    rng = np.random.default_rng(10)
    q = rng.standard_normal((batch, shape.dim)).astype(ndt(dt))
    pos = [0, 5, shape.seq_len - 1, 2]
    present = [True, True, True, False]
    rows = [arena.row_ptr(i, pos[i]) if present[i] else 0 for i in range(batch)]
    dq = torch.from_numpy(q).cuda()
    dre, dim_ = torch.from_numpy(re).cuda(), torch.from_numpy(im).cuda()
    if host_tables:
        ops.rope_host(pos, dre, dim_, dq, rows, shape)
    else:
        ops.rope(torch.tensor(pos, dtype=torch.int32, device="cuda"), dre, dim_, dq, ops.row_table(rows), shape)
    want_cache = arena.host.copy()
    O.apply_rope(oracle_cfg(shape), pos, re, im, q, [want_cache[i, pos[i]] if present[i] else None for i in range(batch)])
    got_cache = arena.dev.cpu().numpy()
    np.testing.assert_allclose(dq.cpu().numpy().astype(np.float64), q.astype(np.float64), rtol=tol, atol=tol)
    np.testing.assert_allclose(got_cache.astype(np.float64), want_cache.astype(np.float64), rtol=tol, atol=tol)
    if dt == "f16":
        # fp32 rotation and one rounding on both sides: at most the last bit (fused against separate multiply-add)
        present_rows = [i for i in range(batch) if present[i]]
        worst, _ = half_ulp_diff(dq.cpu().numpy()[present_rows], q[present_rows])
        assert worst <= 1, worst
        worst, _ = half_ulp_diff(got_cache, want_cache)
        assert worst <= 1, worst
    # V halves and all other rows are untouched bit for bit
    U = np.uint16 if dt == "f16" else np.uint32
    mask = np.ones(got_cache.shape, bool)
    for i in range(batch):
        if present[i]:
            mask[i, pos[i], : shape.kv_dim] = False
    assert np.array_equal(got_cache.view(U)[mask], arena.host.view(U)[mask])


def test_rope_cache_row_not_16_byte_aligned():
    """The f16 kernel takes 16-byte accesses when it can; a cache row at an odd element offset has to come out the same."""
    shape = GQA8
    re32, im32 = O.rope_tables(shape.seq_len, shape.head_size)
    re, im = re32.astype(np.float16), im32.astype(np.float16)
    rng = np.random.default_rng(21)
    q = rng.standard_normal((2, shape.dim)).astype(np.float16)
    rows = rng.standard_normal((2, 2 * shape.kv_dim + 8)).astype(np.float16)
    drows = torch.from_numpy(rows).cuda()
    dq = torch.from_numpy(q).cuda()
    pos = [7, shape.seq_len - 1]
    ptrs = [drows[0].data_ptr() + 2, drows[1].data_ptr()]          # first row starts one element in
    ops.rope(torch.tensor(pos, dtype=torch.int32, device="cuda"), torch.from_numpy(re).cuda(), torch.from_numpy(im).cuda(), dq, ops.row_table(ptrs), shape)
    want_rows = [rows[0, 1:1 + 2 * shape.kv_dim].copy(), rows[1, :2 * shape.kv_dim].copy()]
    O.apply_rope(oracle_cfg(shape), pos, re, im, q, want_rows)
    got = drows.cpu().numpy()
    assert half_ulp_diff(got[0, 1:1 + 2 * shape.kv_dim], want_rows[0])[0] <= 1
    assert half_ulp_diff(got[1, :2 * shape.kv_dim], want_rows[1])[0] <= 1
    assert half_ulp_diff(dq.cpu().numpy(), q)[0] <= 1
    # nothing outside the K halves moved
    assert np.array_equal(got[0, :1], rows[0, :1]) and np.array_equal(got[0, 1 + shape.kv_dim:], rows[0, 1 + shape.kv_dim:])
    assert np.array_equal(got[1, shape.kv_dim:], rows[1, shape.kv_dim:])


# The positions of the device-table entry points never pass through the host, so the kernels bound them themselves: a position at
# or beyond seq_len reads no cache row past the context's last one and writes no score past the end of its row, also where the
# token ranges of the launch are rounded up beyond seq_len (seq_len not a multiple of the range granularity).
@pytest.mark.parametrize("shape", [Shape(dim=1024, n_layers=1, n_heads=8, n_kv_heads=1, hidden_dim=64, seq_len=1000),     # gqa 8: MFMA kernels
                                   Shape(dim=512, n_layers=1, n_heads=4, n_kv_heads=4, hidden_dim=64, seq_len=1000)],    # MHA: dot2 kernels
                         ids=["gqa8", "mha"])
def test_unfused_attention_ops_bound_a_bad_position_by_seq_len(shape):
    batch, guard = 3, 4096
    arena = Arena(shape, batch + 1, torch.float16, seed=41)                 # the context behind the last one is the guard: all NaN
    arena.dev[batch].fill_(float("nan"))
    rng = np.random.default_rng(42)
    dq = torch.from_numpy(rng.standard_normal((batch, shape.dim)).astype(np.float16)).cuda()
    rows = ops.row_table([arena.layer_ptr(i) for i in range(batch)])
    n_att = batch * shape.n_heads * shape.seq_len
    good = torch.tensor([999, 999, 5], dtype=torch.int32, device="cuda")
    bad = torch.tensor([999, 1010, 5], dtype=torch.int32, device="cuda")    # context 1: beyond its 1000 rows
    outs = []
    for pos in (good, bad):
        buf = torch.full((n_att + guard,), 3.0, dtype=torch.float16, device="cuda")
        att = buf[:n_att].view(batch, shape.n_heads, shape.seq_len)
        ops.attn_scores(dq, rows, att, pos, shape)
        ops.sync()
        assert torch.all(buf[n_att:] == 3.0)                                # nothing written behind the last row of scores
        assert torch.isfinite(att.float()).all()                            # no row of the guard context was read
        outs.append(att.clone())
        ops.attn_softmax(att, pos, shape)
        xb = torch.full((batch + 1, shape.dim), 5.0, dtype=torch.float16, device="cuda")
        ops.attn_pv(att, rows, xb[:batch], pos, shape)
        ops.sync()
        assert torch.all(buf[n_att:] == 3.0) and torch.all(xb[batch] == 5.0)
        assert torch.isfinite(xb[:batch].float()).all()
        outs.append(xb[:batch].clone())
    # the bad position behaves as the last valid one, and the other contexts are what they are without it
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])


# ------------------------------------------------------------------ unfused attention ops
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("shape", [TINY, STORIES, GQA8], ids=["tiny", "stories15m", "gqa8"])
@pytest.mark.parametrize("host_tables", [False, True])
def test_unfused_attention_ops(dt, shape, host_tables):
    batch = 4
    cfg = oracle_cfg(shape)
    arena = Arena(shape, batch, tdt(dt), seed=11)
    rng = np.random.default_rng(12)
    q = rng.standard_normal((batch, shape.dim)).astype(ndt(dt))
    pos = [0, min(37, shape.seq_len - 2), shape.seq_len - 1, 3]
    present = [True, True, True, False]
    layers = [arena.layer_ptr(i) if present[i] else 0 for i in range(batch)]
    att0 = np.full((batch, shape.n_heads, shape.seq_len), 3.0, ndt(dt))
    datt = torch.from_numpy(att0).cuda()
    dq = torch.from_numpy(q).cuda()
    dpos = torch.tensor(pos, dtype=torch.int32, device="cuda")
    dxb = torch.full((batch, shape.dim), 5.0, dtype=tdt(dt), device="cuda")

    host_layers = [arena.host[i] if present[i] else None for i in range(batch)]
    att = att0.copy()
    O.attention_0_gemm(cfg, q, host_layers, att, pos)
    if host_tables:
        ops.attn_scores_host(dq, layers, datt, pos, shape)
    else:
        ops.attn_scores(dq, ops.row_table(layers), datt, dpos, shape)
    got = datt.cpu().numpy()
    tol = 4e-3 if dt == "f16" else 2e-5
    np.testing.assert_allclose(got.astype(np.float64), att.astype(np.float64), rtol=tol, atol=tol)
    for i in range(batch):       # beyond pos and empty contexts: untouched
        n = pos[i] + 1 if present[i] else 0
        assert np.all(got[i, :, n:] == 3.0)

    # softmax on identical inputs (the oracle's scores) so that only the softmax is compared
    datt = torch.from_numpy(att).cuda()
    O.attention_softmax(cfg, att, pos)
    if host_tables:
        ops.attn_softmax_host(datt, pos, shape)
    else:
        ops.attn_softmax(datt, dpos, shape)
    got = datt.cpu().numpy()
    tol = 2e-3 if dt == "f16" else 3e-6
    for i in range(batch):
        n = pos[i] + 1
        np.testing.assert_allclose(got[i, :, :n].astype(np.float64), att[i, :, :n].astype(np.float64), rtol=tol, atol=tol)
        assert np.array_equal(got[i, :, n:], att[i, :, n:])

    datt = torch.from_numpy(att).cuda()
    xb = np.full((batch, shape.dim), 5.0, ndt(dt))
    O.attention_2_gemm(cfg, att, host_layers, xb, pos)
    if host_tables:
        ops.attn_pv_host(datt, layers, dxb, pos, shape)
    else:
        ops.attn_pv(datt, ops.row_table(layers), dxb, dpos, shape)
    got = dxb.cpu().numpy()
    tol = 3e-3 if dt == "f16" else 2e-5
    np.testing.assert_allclose(got.astype(np.float64), xb.astype(np.float64), rtol=tol, atol=tol)
    assert np.all(got[3] == 5.0)


def _seq(shape, seq_len):
    return Shape(dim=shape.dim, n_layers=1, n_heads=shape.n_heads, n_kv_heads=shape.n_kv_heads, hidden_dim=64, seq_len=seq_len)


# the streaming kernels (f16, head size 128, row length a multiple of 8): every gqa they take, kv head counts that do not fill
# a block, ragged positions around the 8- and 32-token boundaries, ranges long enough to be cut into several token ranges
STREAM_CASES = [
    ("mha", _seq(MHA128, 640), [639, 0, 31, 32, 300]),
    ("mha-odd", _seq(MHA128_ODD, 304), [303, 7, 8, 9]),
    ("gqa2", _seq(GQA2, 280), [279, 255, 256, 257]),
    ("gqa4", _seq(GQA4, 336), [335, 33, 1]),
    ("gqa8", _seq(GQA8, 704), [703, 500, 15, 16]),
    ("gqa16", _seq(GQA16, 304), [303, 63, 64]),
    ("gqa8-long", _seq(GQA8, 4096), [4095, 2048, 777]),
    ("mha-long", _seq(MHA128, 2048), [2047, 1025]),
]


@pytest.mark.parametrize("name,shape,pos", STREAM_CASES, ids=[c[0] for c in STREAM_CASES])
@pytest.mark.parametrize("host_tables", [False, True])
def test_unfused_attention_ops_streaming_kernels(name, shape, pos, host_tables):
    batch = len(pos) + 1
    pos = list(pos) + [5]
    present = [True] * (batch - 1) + [False]
    cfg = oracle_cfg(shape)
    arena = Arena(shape, batch, torch.float16, seed=21)
    rng = np.random.default_rng(22)
    q = rng.standard_normal((batch, shape.dim)).astype(np.float16)
    layers = [arena.layer_ptr(i) if present[i] else 0 for i in range(batch)]
    host_layers = [arena.host[i] if present[i] else None for i in range(batch)]
    att0 = np.full((batch, shape.n_heads, shape.seq_len), 3.0, np.float16)
    datt = torch.from_numpy(att0).cuda()
    dq = torch.from_numpy(q).cuda()
    dpos = torch.tensor(pos, dtype=torch.int32, device="cuda")

    att = att0.copy()
    O.attention_0_gemm(cfg, q, host_layers, att, pos)
    if host_tables:
        ops.attn_scores_host(dq, layers, datt, pos, shape)
    else:
        ops.attn_scores(dq, ops.row_table(layers), datt, dpos, shape)
    got = datt.cpu().numpy()
    np.testing.assert_allclose(got.astype(np.float64), att.astype(np.float64), rtol=4e-3, atol=4e-3)
    _, frac = half_ulp_diff(got, att)
    assert frac < 0.02                                   # same fp32 sums up to their order: nearly every score is bit-equal
    for i in range(batch):                               # beyond pos and empty contexts: untouched
        n = pos[i] + 1 if present[i] else 0
        assert np.all(got[i, :, n:] == 3.0)

    datt = torch.from_numpy(att).cuda()
    O.attention_softmax(cfg, att, pos)
    if host_tables:
        ops.attn_softmax_host(datt, pos, shape)
    else:
        ops.attn_softmax(datt, dpos, shape)
    got = datt.cpu().numpy()
    for i in range(batch):
        n = pos[i] + 1
        ulps, frac = half_ulp_diff(got[i, :, :n], att[i, :, :n])
        assert ulps <= 1 and frac < 0.05, (i, ulps, frac)   # same rounding points; the sum's order and expf may move the last place
        assert np.array_equal(got[i, :, n:], att[i, :, n:])

    datt = torch.from_numpy(att).cuda()
    xb = np.full((batch, shape.dim), 5.0, np.float16)
    dxb = torch.full((batch, shape.dim), 5.0, dtype=torch.float16, device="cuda")
    O.attention_2_gemm(cfg, att, host_layers, xb, pos)
    if host_tables:
        ops.attn_pv_host(datt, layers, dxb, pos, shape)
    else:
        ops.attn_pv(datt, ops.row_table(layers), dxb, dpos, shape)
    got = dxb.cpu().numpy()
    np.testing.assert_allclose(got.astype(np.float64), xb.astype(np.float64), rtol=3e-3, atol=3e-3)
    assert np.all(got[batch - 1] == 5.0)


# ------------------------------------------------------------------ fused decode attention
def run_fused_case(shape, dt, variant, pos, present, chunk, seed=13, host_tables=False, std=1.0, balanced=False, join=1):
    batch = len(pos)
    cfg = oracle_cfg(shape)
    arena = Arena(shape, batch, tdt(dt), seed=seed, std=std)
    rng = np.random.default_rng(seed + 1)
    q = rng.standard_normal((batch, shape.dim)).astype(ndt(dt))
    layers = [arena.layer_ptr(i) if present[i] else 0 for i in range(batch)]
    dq = torch.from_numpy(q).cuda()
    dxb = torch.full((batch, shape.dim), 5.0, dtype=tdt(dt), device="cuda")
    ops.attn_set_chunk(chunk)
    ops.attn_set_split_join(join)
    try:
        if balanced:
            max_pos = max([p for p, ok in zip(pos, present) if ok] + [0])
            ws = torch.empty(ops.attn_balanced_workspace(batch, shape), dtype=torch.uint8, device="cuda")
            table = ops.row_table(layers)
            ops.attn_balance(table, torch.tensor(pos, dtype=torch.int32, device="cuda"), max_pos, shape, ws)
            ops.attn_decode_balanced(dq, table, dxb, max_pos, shape, ws)
        elif host_tables:
            ops.attn_decode_host(dq, layers, pos, dxb, shape, variant=variant)
        else:
            max_pos = max([p for p, ok in zip(pos, present) if ok] + [0])
            ops.attn_decode(dq, ops.row_table(layers), torch.tensor(pos, dtype=torch.int32, device="cuda"), dxb,
                            max_pos, shape, variant=variant)
        got = dxb.cpu().numpy()
    finally:
        ops.attn_set_chunk(0)
        ops.attn_set_split_join(1)

    # oracle: the reference's fp32 CPU path on the same (exactly converted) inputs
    q32 = q.astype(np.float32)
    l32 = arena.host_layers_f32(present)
    att = np.zeros((batch, shape.n_heads, shape.seq_len), np.float32)
    xb = np.full((batch, shape.dim), 5.0, np.float32)
    O.attention_0_gemm(cfg, q32, l32, att, pos)
    O.attention_softmax(cfg, att, pos)
    O.attention_2_gemm(cfg, att, l32, xb, pos)
    live = [i for i in range(batch) if present[i]]
    assert_close(got[live], xb[live], what=f"fused attention {dt} variant {variant} chunk {chunk}")
    for i in range(batch):
        if not present[i]:
            assert np.all(got[i] == 5.0), "row of an empty context must stay untouched"
    return got, xb


RAGGED = [0, 1, 15, 16, 17, 63, 64, 255, 256, 257]


@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("shape", [TINY, STORIES], ids=["tiny", "stories15m"])
@pytest.mark.parametrize("chunk", [0, 16, 48])
def test_fused_generic(dt, shape, chunk):
    pos = [p for p in RAGGED if p < shape.seq_len] + [shape.seq_len - 1, 2]
    present = [True] * (len(pos) - 1) + [False]
    got, want = run_fused_case(shape, dt, GH_ATTN_GENERIC, pos, present, chunk)
    if dt == "f32":
        np.testing.assert_allclose(got[:-1], want[:-1], rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("shape", [MHA128, MHA128_ODD, GQA2, GQA4, GQA8], ids=["mha", "mha6", "gqa2", "gqa4", "gqa8"])
@pytest.mark.parametrize("chunk", [0, 16, 80, 256])
def test_fused_valu(shape, chunk):
    pos = [p for p in RAGGED if p < shape.seq_len] + [shape.seq_len - 1, 2]
    present = [True] * (len(pos) - 1) + [False]
    run_fused_case(shape, "f16", GH_ATTN_VALU, pos, present, chunk)


@pytest.mark.parametrize("shape", [GQA2, GQA4, GQA8, GQA16], ids=["gqa2", "gqa4", "gqa8", "gqa16"])
@pytest.mark.parametrize("chunk", [0, 16, 80, 256])
def test_fused_mfma(shape, chunk):
    pos = [p for p in RAGGED if p < shape.seq_len] + [shape.seq_len - 1, 2]
    present = [True] * (len(pos) - 1) + [False]
    run_fused_case(shape, "f16", GH_ATTN_MFMA, pos, present, chunk)


@pytest.mark.parametrize("waves", [4, 8])
@pytest.mark.parametrize("splits", [2, 4])
@pytest.mark.parametrize("variant,shape", [(GH_ATTN_VALU, MHA128), (GH_ATTN_VALU, MHA128_ODD), (GH_ATTN_VALU, GQA2), (GH_ATTN_VALU, GQA8),
                                           (GH_ATTN_MFMA, GQA2), (GH_ATTN_MFMA, GQA4), (GH_ATTN_MFMA, GQA8), (GH_ATTN_MFMA, GQA16)],
                         ids=["valu-mha", "valu-mha6", "valu-gqa2", "valu-gqa8", "mfma-gqa2", "mfma-gqa4", "mfma-gqa8", "mfma-gqa16"])
def test_fused_splits_joined_inside_the_work_group(variant, shape, splits, waves):
    """Plans of 2 or 4 splits: the splits of a (context, kv head) stream are waves of one work-group, which adds them up itself, in
    work-groups of 4 or of 8 waves.  Contexts that reach into every split, into some, into the first only; an empty context in the
    middle; head counts that do not fill the last work-group.  Against the oracle, and against the route with partial sums and the
    merge kernel, which does the same arithmetic in another kernel (contraction may differ: one rounding)."""
    top = shape.seq_len - 1
    chunk = -(-(-(-shape.seq_len // splits)) // 16) * 16
    pos = [top, 0, chunk - 1, chunk, chunk + 1, top - 1, 5, 2 * chunk - 1 if splits > 2 else 17, top, 3 * chunk + 1 if splits > 2 else chunk // 2, 40]
    present = [True] * len(pos)
    present[4] = False
    ops.attn_set_chunk(chunk)
    ops.attn_set_split_join(waves)
    try:
        c_shape, got_chunk, got_splits, need = shape.c(), C.c_uint32(0), C.c_uint32(0), C.c_uint64(1)
        _lib.check(_lib.lib().gh_attn_decode_plan(len(pos), top, C.byref(c_shape), _lib.GH_F16, variant, C.byref(got_chunk), C.byref(got_splits), C.byref(need)))
        assert (got_chunk.value, got_splits.value, need.value) == (chunk, splits, 0)        # no partial sums in the workspace
        assert ops.attn_decode_join_waves(len(pos), top, shape, variant=variant) == waves
        ops.attn_set_split_join(0)
        assert ops.attn_decode_join_waves(len(pos), top, shape, variant=variant) == 0
    finally:
        ops.attn_set_chunk(0)
        ops.attn_set_split_join(1)
    joined, _ = run_fused_case(shape, "f16", variant, pos, present, chunk, seed=71, join=waves)
    merged, _ = run_fused_case(shape, "f16", variant, pos, present, chunk, seed=71, join=0)
    live = [i for i, ok in enumerate(present) if ok]
    assert half_ulp_diff(joined[live], merged[live])[0] <= 1
    # large scores: the splits' maxima lie far apart
    run_fused_case(shape, "f16", variant, pos, present, chunk, seed=72, std=5.0, join=waves)


@pytest.mark.parametrize("shape", [TINY, MHA128, GQA8], ids=["tiny", "mha", "gqa8"])
def test_fused_auto_and_host_tables(shape):
    pos = [0, 5, shape.seq_len - 1, shape.seq_len // 2]
    run_fused_case(shape, "f16", GH_ATTN_AUTO, pos, [True, True, True, True], 0, host_tables=True)
    run_fused_case(shape, "f16", GH_ATTN_AUTO, pos, [True, False, True, True], 32, host_tables=True)


@pytest.mark.parametrize("shape", [MHA128, MHA128_ODD, GQA2, GQA4, GQA8, GQA16], ids=["mha", "mha6", "gqa2", "gqa4", "gqa8", "gqa16"])
def test_fused_balanced_ragged(shape):
    # keys cut into equal runs over the work-groups: contexts shorter than a run share one, longer ones are divided
    # (a run is at least 256 keys), an empty context in the middle and at the end
    pos = [p for p in RAGGED if p < shape.seq_len] + [shape.seq_len - 1, 2, shape.seq_len - 1, 100, 2]
    present = [True] * len(pos)
    present[3] = False
    present[-1] = False
    run_fused_case(shape, "f16", GH_ATTN_MFMA, pos, present, 0, balanced=True)


def test_fused_balanced_cases():
    shape = GQA8
    # one context; one long context among short ones; every context equal; only empty contexts but one
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [699], [True], 0, balanced=True, seed=51)
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [0], [True], 0, balanced=True, seed=52)
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [3] * 5 + [699] + [7] * 6, [True] * 12, 0, balanced=True, seed=53)
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [511] * 9, [True] * 9, 0, balanced=True, seed=54)
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [10, 20, 300, 40], [False, False, True, False], 0, balanced=True, seed=55)
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [10, 20], [False, False], 0, balanced=True, seed=56)
    # large scores
    run_fused_case(shape, "f16", GH_ATTN_MFMA, [699, 256, 30], [True] * 3, 0, balanced=True, seed=57, std=6.0)


def test_fused_balanced_many_contexts_equal_plain_kernel():
    # more contexts than the planning kernel has threads (it then takes several per thread), against the plain kernel
    shape = Shape(dim=256, n_layers=1, n_heads=2, n_kv_heads=1, hidden_dim=64, seq_len=96)
    batch = 2500
    rng = np.random.default_rng(61)
    pos = rng.integers(0, shape.seq_len, batch)
    pos[::97] = shape.seq_len - 1
    arena = Arena(shape, batch, torch.float16, seed=62)
    ptrs = [arena.layer_ptr(i) for i in range(batch)]
    for i in range(5, batch, 41):
        ptrs[i] = 0
    table = ops.row_table(ptrs)
    dpos = torch.tensor(pos, dtype=torch.int32, device="cuda")
    q = torch.randn((batch, shape.dim), dtype=torch.float16, device="cuda")
    plain = torch.full((batch, shape.dim), 5.0, dtype=torch.float16, device="cuda")
    bal = torch.full((batch, shape.dim), 5.0, dtype=torch.float16, device="cuda")
    max_pos = int(pos.max())
    ops.attn_decode(q, table, dpos, plain, max_pos, shape, variant=GH_ATTN_MFMA)
    ws = torch.empty(ops.attn_balanced_workspace(batch, shape), dtype=torch.uint8, device="cuda")
    ops.attn_balance(table, dpos, max_pos, shape, ws)
    for _ in range(2):  # the cuts serve every layer of a step: a second call on the same workspace gives the same
        bal.fill_(5.0)
        ops.attn_decode_balanced(q, table, bal, max_pos, shape, ws)
        a, r = errors(bal.cpu().numpy(), plain.cpu().numpy())
        assert a < 4e-3 and r < 1e-3, (a, r)
    assert torch.all(bal[5] == 5.0) and torch.all(bal[46] == 5.0)


def test_fused_balanced_random_batches_equal_plain_kernel():
    # seeded sweep over shapes (gqa 8, 1, 4 with three kv heads, 16, 2 with five kv heads), batch sizes, length patterns (uniform
    # random, all short, all full, one long among short ones, lengths at chunk boundaries) and empty contexts; the workspace holds
    # stale bytes before every call
    shapes = [GQA8, MHA128, GQA4, GQA16, Shape(dim=1280, n_layers=1, n_heads=10, n_kv_heads=5, hidden_dim=64, seq_len=1100)]
    rng = np.random.default_rng(123)
    for it in range(60):
        shape = shapes[it % len(shapes)]
        batch = int(rng.choice([1, 2, 3, 7, 16, 33, 64, 130]))
        kind = it // len(shapes) % 5
        if kind == 0:
            p = rng.integers(0, shape.seq_len, batch)
        elif kind == 1:
            p = rng.integers(0, 64, batch)
        elif kind == 2:
            p = np.full(batch, shape.seq_len - 1)
        elif kind == 3:
            p = rng.integers(0, 30, batch)
            p[rng.integers(0, batch)] = shape.seq_len - 1
        else:
            p = (rng.integers(0, shape.seq_len // 64, batch) * 64 + rng.choice([-1, 0, 1, 63], batch)).clip(0, shape.seq_len - 1)
        row_bytes = 2 * shape.kv_dim * 2
        cache = torch.randn((batch, shape.seq_len, 2 * shape.kv_dim), dtype=torch.float16, device="cuda")
        ptrs = [cache.data_ptr() + i * shape.seq_len * row_bytes for i in range(batch)]
        holes = rng.random(batch) < (0.2 if it % 3 == 0 else 0.0)
        if holes.all():
            holes[0] = False
        for i in np.nonzero(holes)[0]:
            ptrs[i] = 0
        table = ops.row_table(ptrs)
        pos = torch.tensor(p, dtype=torch.int32, device="cuda")
        max_pos = int(p.max())
        q = torch.randn((batch, shape.dim), dtype=torch.float16, device="cuda")
        plain = torch.full((batch, shape.dim), 7.0, dtype=torch.float16, device="cuda")
        bal = torch.full((batch, shape.dim), 7.0, dtype=torch.float16, device="cuda")
        ops.attn_decode(q, table, pos, plain, max_pos, shape)
        ws = torch.empty(ops.attn_balanced_workspace(batch, shape), dtype=torch.uint8, device="cuda")
        ws.fill_(0xFF)
        ops.attn_balance(table, pos, max_pos, shape, ws)
        ops.attn_decode_balanced(q, table, bal, max_pos, shape, ws)
        what = f"case {it}: kv heads {shape.n_kv_heads}, gqa {shape.gqa_size}, batch {batch}, pattern {kind}, {int(holes.sum())} empty"
        assert bool(torch.isfinite(bal).all()), what
        assert (plain.float() - bal.float()).abs().max().item() < 6e-3, what
        for i in np.nonzero(holes)[0]:
            assert torch.all(bal[i] == 7.0), what


def test_fused_balanced_bound_below_the_true_maximum_truncates_and_bad_arguments():
    shape = GQA8
    batch = 3
    arena = Arena(shape, batch, torch.float16, seed=71)
    table = ops.row_table([arena.layer_ptr(i) for i in range(batch)])
    q = torch.randn((batch, shape.dim), dtype=torch.float16, device="cuda")
    ws = torch.empty(ops.attn_balanced_workspace(batch, shape), dtype=torch.uint8, device="cuda")
    true_pos = torch.tensor([699, 500, 90], dtype=torch.int32, device="cuda")
    cut_pos = torch.tensor([299, 299, 90], dtype=torch.int32, device="cuda")
    a = torch.zeros((batch, shape.dim), dtype=torch.float16, device="cuda")
    b = torch.zeros_like(a)
    ops.attn_balance(table, true_pos, 299, shape, ws)   # positions above the bound count as the bound
    ops.attn_decode_balanced(q, table, a, 299, shape, ws)
    ops.attn_balance(table, cut_pos, 299, shape, ws)
    ops.attn_decode_balanced(q, table, b, 299, shape, ws)
    assert torch.equal(a, b)
    import ctypes as C
    from glinthawk_amd import _lib
    from glinthawk_amd._lib import GH_F16, GH_F32
    GH_ERR_INVALID, GH_ERR_WORKSPACE = -1, -5
    L = _lib.lib()
    s = shape.c()
    small = torch.empty(1024, dtype=torch.uint8, device="cuda")
    assert L.gh_attn_balance(table.data_ptr(), true_pos.data_ptr(), batch, 299, C.byref(s), small.data_ptr(), 1024, None) == GH_ERR_WORKSPACE
    assert L.gh_attn_decode_balanced(q.data_ptr(), table.data_ptr(), a.data_ptr(), batch, 299, C.byref(s), GH_F16, small.data_ptr(), 1024, None) == GH_ERR_WORKSPACE
    assert L.gh_attn_balance(table.data_ptr(), true_pos.data_ptr(), batch, shape.seq_len, C.byref(s), ws.data_ptr(), ws.numel(), None) == GH_ERR_INVALID
    odd = Shape(dim=768, n_layers=1, n_heads=6, n_kv_heads=2, hidden_dim=64, seq_len=300).c()      # gqa 3
    assert L.gh_attn_balance(table.data_ptr(), true_pos.data_ptr(), batch, 10, C.byref(odd), ws.data_ptr(), ws.numel(), None) == GH_ERR_INVALID
    assert L.gh_attn_decode_balanced(q.data_ptr(), table.data_ptr(), a.data_ptr(), batch, 299, C.byref(s), GH_F32, ws.data_ptr(), ws.numel(), None) == GH_ERR_INVALID
    assert L.gh_attn_decode_balanced(None, table.data_ptr(), a.data_ptr(), batch, 299, C.byref(s), GH_F16, ws.data_ptr(), ws.numel(), None) == GH_ERR_INVALID


def test_attention_timing_hooks_count_calls_in_both_modes():
    import ctypes as C
    from glinthawk_amd import _lib
    L = _lib.lib()
    shape = GQA8
    batch = 4
    arena = Arena(shape, batch, torch.float16, seed=81)
    table = ops.row_table([arena.layer_ptr(i) for i in range(batch)])
    pos = torch.tensor([699, 650, 600, 512], dtype=torch.int32, device="cuda")
    q = torch.randn((batch, shape.dim), dtype=torch.float16, device="cuda")
    xb = torch.zeros_like(q)
    k_ms, m_ms, n = C.c_double(0), C.c_double(0), C.c_uint64(0)
    spans = {}
    try:
        for mode in (1, 2):
            _lib.check(L.gh_attn_timing_enable(mode))
            _lib.check(L.gh_attn_timing_reset())
            for _ in range(5):
                ops.attn_decode(q, table, pos, xb, 699, shape, variant=GH_ATTN_MFMA)
            _lib.check(L.gh_attn_timing_read(C.byref(k_ms), C.byref(m_ms), C.byref(n)))
            assert n.value == 5 and k_ms.value > 0
            spans[mode] = (k_ms.value, m_ms.value)
    finally:
        _lib.check(L.gh_attn_timing_enable(0))
    assert spans[1][1] > 0          # split kernel and merge timed apart
    assert spans[2][1] == 0         # one span over the pair
    _lib.check(L.gh_attn_timing_reset())
    ops.attn_decode(q, table, pos, xb, 699, shape, variant=GH_ATTN_MFMA)   # off: nothing recorded
    _lib.check(L.gh_attn_timing_read(C.byref(k_ms), C.byref(m_ms), C.byref(n)))
    assert n.value == 0


def test_fused_variants_agree():
    # the three kernels on the same input: differences are rounding only
    shape = GQA8
    pos = [699, 300, 17]
    outs = [run_fused_case(shape, "f16", v, pos, [True] * 3, 64, seed=21)[0]
            for v in (GH_ATTN_GENERIC, GH_ATTN_VALU, GH_ATTN_MFMA)]
    for o in outs[1:]:
        a, r = errors(o, outs[0])
        assert a < 4e-3 and r < 1e-3


def test_fused_large_scores_are_stable():
    # scores of magnitude ~ +-60 (std 6 K rows): exp() without the running max would overflow fp16/fp32 sums
    run_fused_case(GQA8, "f16", GH_ATTN_MFMA, [699, 256], [True, True], 64, seed=31, std=6.0)
    run_fused_case(MHA128, "f16", GH_ATTN_VALU, [639, 256], [True, True], 64, seed=32, std=6.0)


def test_fused_properties_uniform_values_and_single_key():
    shape = GQA8
    batch = 3
    arena = Arena(shape, batch, torch.float16, seed=41)
    v = torch.randn(shape.kv_dim, dtype=torch.float16, device="cuda")
    arena.dev[:, :, shape.kv_dim:] = v                     # every cached V row identical
    q = torch.randn((batch, shape.dim), dtype=torch.float16, device="cuda")
    pos = [0, 333, 699]
    want = v.reshape(shape.n_kv_heads, 1, shape.head_size).expand(-1, shape.gqa_size, -1).reshape(-1).float()
    for variant in (GH_ATTN_GENERIC, GH_ATTN_VALU, GH_ATTN_MFMA):
        xb = torch.zeros((batch, shape.dim), dtype=torch.float16, device="cuda")
        ops.attn_decode(q, ops.row_table([arena.layer_ptr(i) for i in range(batch)]),
                        torch.tensor(pos, dtype=torch.int32, device="cuda"), xb, max(pos), shape, variant=variant)
        assert torch.equal(xb[0].float(), want)            # one key: weight exactly 1
        assert torch.allclose(xb.float(), want.expand(batch, -1), atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("variant", [GH_ATTN_MFMA, GH_ATTN_VALU, GH_ATTN_GENERIC], ids=["mfma", "valu", "generic"])
def test_fused_max_pos_below_the_true_maximum_truncates(variant):
    """`max_pos` is the caller's upper bound of the positions; the split plan and the workspace follow from it.  A bound below
    the true maximum must not take a kernel outside the workspace or into another head's partial sums: the result is the
    attention over the first max_splits * tokens_per_split keys, and the bytes behind the workspace stay as they were."""
    import ctypes as C
    from glinthawk_amd import _lib
    shape = GQA8
    batch, bound = 5, 199
    arena = Arena(shape, batch, torch.float16, seed=77)
    rows = ops.row_table([arena.layer_ptr(i) for i in range(batch)])
    q = torch.randn((batch, shape.dim), dtype=torch.float16, device="cuda")
    true_pos = [650, 10, 699, 199, 400]
    s = shape.c()
    chunk, splits, need = C.c_uint32(), C.c_uint32(), C.c_uint64()
    ops.attn_set_chunk(64)                       # several splits even at this small bound
    try:
        _lib.check(_lib.lib().gh_attn_decode_plan(batch, bound, C.byref(s), _lib.GH_F16, variant, C.byref(chunk), C.byref(splits), C.byref(need)))
        covered = chunk.value * splits.value
        assert splits.value > 1 and bound < covered < max(true_pos)
        ws_bytes = ops.attn_decode_workspace(batch, bound, shape)
        guard = 1 << 16
        buf = torch.full((ws_bytes + guard,), 0x5A, dtype=torch.uint8, device="cuda")
        got = torch.zeros_like(q)
        ops.attn_decode(q, rows, torch.tensor(true_pos, dtype=torch.int32, device="cuda"), got, bound, shape,
                        workspace=buf[:ws_bytes], variant=variant)
        torch.cuda.synchronize()
        assert torch.all(buf[ws_bytes:] == 0x5A)
        assert torch.isfinite(got).all()
        want = torch.zeros_like(q)
        clamped = [min(p, covered - 1) for p in true_pos]
        ops.attn_decode(q, rows, torch.tensor(clamped, dtype=torch.int32, device="cuda"), want, max(clamped), shape, variant=variant)
    finally:
        ops.attn_set_chunk(0)
    assert torch.allclose(got.float(), want.float(), atol=2e-3, rtol=2e-3)


def test_fused_rejects_bad_arguments():
    shape = GQA8
    q = torch.zeros((1, shape.dim), dtype=torch.float16, device="cuda")
    xb = torch.zeros_like(q)
    rows = ops.row_table([0])
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(GlintError):
        ops.attn_decode(q, rows, pos, xb, shape.seq_len, shape)            # max_pos outside seq_len
    with pytest.raises(GlintError):
        ops.attn_decode(q.float(), rows, pos, xb.float(), 5, shape, variant=GH_ATTN_MFMA)   # f32 on the f16 kernel
    with pytest.raises(GlintError):                                         # workspace too small
        ops.attn_set_chunk(16)
        try:
            ops.attn_decode(q, rows, pos, xb, 500, shape, workspace=torch.empty(64, dtype=torch.uint8, device="cuda"))
        finally:
            ops.attn_set_chunk(0)


# ------------------------------------------------------------------ paged arena, straight through the C-ABI
def test_vmm_commit_out_of_range_is_refused():
    """VirtualMemoryRegion::allocate_span refuses a span outside the reservation ("Out of bounds allocation",
    arch/amd64/common/vmem.hh:67-69); the C-ABI reports it as GH_ERR_INVALID and leaves the region as it was."""
    import ctypes as C
    from glinthawk_amd import _lib
    L = _lib.lib()
    gran = C.c_uint64(0)
    _lib.check(L.gh_vmm_granularity(C.byref(gran)))
    g = gran.value
    assert g > 0 and g & (g - 1) == 0
    region = C.c_void_p()
    _lib.check(L.gh_vmm_reserve(C.byref(region), 4 * g))
    assert L.gh_vmm_max_len(region) == 4 * g and L.gh_vmm_ptr(region)
    assert L.gh_vmm_commit(region, g, g) == 0                         # inside: fine
    assert L.gh_vmm_committed_bytes(region) == g
    for off, length in ((4 * g, g), (3 * g, 2 * g), (0, 5 * g), (1 << 60, g)):
        assert L.gh_vmm_commit(region, off, length) == -1, (off, length)      # GH_ERR_INVALID
        assert b"outside" in L.gh_last_error()
    assert L.gh_vmm_commit(region, 0, 0) == -1                        # empty span
    assert L.gh_vmm_commit(region, g // 2, g) == -1 and b"granularity" in L.gh_last_error()
    assert L.gh_vmm_commit(None, 0, g) == -1
    assert L.gh_vmm_committed_bytes(region) == g                      # nothing of the refused spans was mapped
    # the committed block is ordinary device memory
    t = torch.arange(1024, dtype=torch.int32, device="cuda")
    _lib.check(L.gh_memcpy(L.gh_vmm_ptr(region) + g, t.data_ptr(), 4096, _lib.GH_D2D, 0, None))
    back = torch.zeros_like(t)
    _lib.check(L.gh_memcpy(back.data_ptr(), L.gh_vmm_ptr(region) + g, 4096, _lib.GH_D2D, 0, None))
    assert torch.equal(back, t)
    _lib.check(L.gh_vmm_clear(region))
    assert L.gh_vmm_committed_bytes(region) == 0
    _lib.check(L.gh_vmm_free(region))


# ------------------------------------------------------------------ streams and events of the C-ABI
def test_streams_and_events_order_a_copy_before_a_kernel():
    import ctypes as C
    from glinthawk_amd import _lib
    L = _lib.lib()
    stream, event = C.c_void_p(), C.c_void_p()
    _lib.check(L.gh_stream_create(C.byref(stream)))
    _lib.check(L.gh_event_create(C.byref(event)))
    assert stream.value and event.value
    n = 1 << 22
    src = ops.pinned_empty((n,), np.float16)
    src[:] = (np.arange(n) % 1000).astype(np.float16)
    a = torch.zeros(n, dtype=torch.float16, device="cuda")
    b = torch.ones(n, dtype=torch.float16, device="cuda")
    # upload on the caller's stream, kernel on the default stream behind the event
    _lib.check(L.gh_memcpy(a.data_ptr(), src.ctypes.data, 2 * n, _lib.GH_H2D, 1, stream))
    _lib.check(L.gh_event_record(event, stream))
    _lib.check(L.gh_stream_wait_event(None, event))
    _lib.check(L.gh_accum(b.data_ptr(), a.data_ptr(), n, 1, _lib.GH_F16, None))
    _lib.check(L.gh_sync(None))
    assert torch.equal(b.cpu(), torch.from_numpy(src.copy()) + 1)
    # and the other way round: the download on the caller's stream waits for the kernel on the default stream
    out = ops.pinned_empty((n,), np.float16)
    out[:] = 0
    _lib.check(L.gh_accum(b.data_ptr(), a.data_ptr(), n, 1, _lib.GH_F16, None))
    _lib.check(L.gh_event_record(event, None))
    _lib.check(L.gh_stream_wait_event(stream, event))
    _lib.check(L.gh_memcpy(out.ctypes.data, b.data_ptr(), 2 * n, _lib.GH_D2H, 1, stream))
    _lib.check(L.gh_sync(stream))
    assert np.array_equal(out, (src.astype(np.float32) * 2 + 1).astype(np.float16))
    for call in (lambda: L.gh_event_record(None, stream), lambda: L.gh_stream_wait_event(stream, None), lambda: L.gh_stream_destroy(None),
                 lambda: L.gh_event_destroy(None), lambda: L.gh_stream_create(None)):
        assert call() == -1
    _lib.check(L.gh_event_destroy(event))
    _lib.check(L.gh_stream_destroy(stream))


@pytest.mark.gpu
def test_timed_events_bracket_the_work_between_them():
    import ctypes as C
    import time
    from glinthawk_amd import _lib
    L = _lib.lib()
    e0, e1 = C.c_void_p(), C.c_void_p()
    _lib.check(L.gh_event_create_timed(C.byref(e0)))
    _lib.check(L.gh_event_create_timed(C.byref(e1)))
    n = 1 << 26
    a = torch.zeros(n, dtype=torch.float16, device="cuda")
    b = torch.ones(n, dtype=torch.float16, device="cuda")
    _lib.check(L.gh_sync(None))
    t0 = time.perf_counter()
    _lib.check(L.gh_event_record(e0, None))
    for _ in range(20):
        _lib.check(L.gh_accum(a.data_ptr(), b.data_ptr(), n, 1, _lib.GH_F16, None))
    _lib.check(L.gh_event_record(e1, None))
    ms = C.c_float(-1)
    _lib.check(L.gh_event_elapsed_ms(e0, e1, C.byref(ms)))  # waits for the second event
    wall_ms = (time.perf_counter() - t0) * 1e3
    assert torch.all(a.cpu() == 20)
    # 20 passes over 384 MiB each: above what 8 TB/s allows (1 ms), within the wall time around the same work
    assert 1.0 < ms.value <= wall_ms, (ms.value, wall_ms)
    for call in (lambda: L.gh_event_elapsed_ms(None, e1, C.byref(ms)), lambda: L.gh_event_elapsed_ms(e0, e1, None),
                 lambda: L.gh_event_create_timed(None)):
        assert call() == -1
    _lib.check(L.gh_event_destroy(e0))
    _lib.check(L.gh_event_destroy(e1))
