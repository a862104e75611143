"""Projections fused with their follow-up ops against the same ops issued one by one (bit-exact where
the arithmetic is element-wise, tolerance where a reduction order differs) and against the oracle."""
import numpy as np
import pytest
import torch

import oracle as O
from glinthawk_amd import Shape, _lib, ops, stage as S
from helpers import Arena, assert_close, assert_half_parity, oracle_cfg
from test_gpu_stage import SHAPES, OracleModel, d2h, load_weights, make_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    ops.init(0)


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("b,s,r", [(4, 288, 288), (64, 1024, 512), (5, 768, 1000), (3, 100, 36),
                                   # more rows than one streaming slab: the tile kernels write the partials
                                   (100, 512, 260), (256, 1024, 512), (300, 4096, 1000),
                                   # enough 256-token tiles: the residual is added in the large tile kernel's epilogue (f16, r % 8 == 0)
                                   (768, 8192, 16384), (2048, 512, 6152), (3000, 1024, 6144), (2300, 512, 8192),
                                   (2048, 512, 6150)])          # r % 8 != 0: fp32 partials and the row kernel
def test_matmul_accum_and_norm(dt, b, s, r, product_route):
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((b, s), generator=g, device="cuda").to(dt)
    w = (torch.randn((r, s), generator=g, device="cuda") / s ** 0.5).to(dt)
    res = torch.randn((b, r), generator=g, device="cuda").to(dt)
    nw = (1 + 0.1 * torch.randn(r, generator=g, device="cuda")).to(dt)
    # separate ops
    want_res = res.clone()
    ops.accum(want_res, ops.matmul(x, w))
    want_norm = ops.rmsnorm(want_res, nw)
    # fused, without and with the norm
    got_res = res.clone()
    assert ops.matmul_accum(got_res, x, w) is None
    assert torch.equal(got_res, want_res)
    got_res2 = res.clone()
    got_norm = ops.matmul_accum(got_res2, x, w, nw)
    assert torch.equal(got_res2, want_res)
    tol = 2e-3 if dt == torch.float16 else 3e-6
    assert torch.allclose(got_norm.float(), want_norm.float(), rtol=tol, atol=tol)
    # and against the oracle's fp32 path
    o_res = res.float().cpu().numpy()
    O.accum(o_res, O.matmul(x.float().cpu().numpy(), w.float().cpu().numpy()))
    assert_close(got_norm.float().cpu().numpy(), O.rmsnorm(o_res, nw.float().cpu().numpy()), what="fused accum+rmsnorm")
    # the plain product of the separate ops and the product inside each of the two fused calls
    product_route.check(3 if dt == torch.float16 and product_route.wanted(b, s, r) else 0)


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("b,s,hidden", [(4, 288, 768), (64, 512, 1536), (3, 100, 50), (130, 512, 1536), (512, 8192, 12544),
                                        # enough row tiles for one launch without a K split: both factors in one kernel
                                        (64, 512, 16384), (5, 256, 16404), (33, 1024, 28672),
                                        (5, 256, 16386)])     # rows not a multiple of 4: the two-kernel route
def test_matmul_silu_gate(dt, b, s, hidden, product_route):
    check_matmul_silu_gate(dt, b, s, hidden, product_route)


@pytest.mark.parametrize("waves", [4, 8])
@pytest.mark.parametrize("b,s,hidden", [(64, 512, 16384), (5, 256, 16404), (33, 1024, 28672), (64, 8192, 3584), (17, 768, 16500)])
def test_matmul_silu_gate_one_launch_with_four_and_eight_waves(waves, b, s, hidden, product_route):
    """The one-launch form (w1 and w3 rows of the same outputs in one work-group, gate in the epilogue) with work-groups of four
    and of eight waves, whichever the library would pick for the shape: row counts that leave the last work-group and the last
    wave partly empty, few and many columns."""
    _lib.check(_lib.lib().gh_gemm_set_gate_waves(waves))
    try:
        check_matmul_silu_gate(torch.float16, b, s, hidden, product_route)
    finally:
        _lib.check(_lib.lib().gh_gemm_set_gate_waves(0))


def check_matmul_silu_gate(dt, b, s, hidden, product_route):
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((b, s), generator=g, device="cuda").to(dt)
    w13 = (torch.randn((2 * hidden, s), generator=g, device="cuda") / s ** 0.5).to(dt)
    hb = ops.matmul(x, w13[:hidden].contiguous())
    hb2 = ops.matmul(x, w13[hidden:].contiguous())
    ops.silu(hb, hb2)
    got = ops.matmul_silu_gate(x, w13)
    # the fused call multiplies one (2*hidden, s) matrix and may split K differently from the two
    # separate calls, so the fp32 sums can differ in the last bit before rounding
    tol = 2e-3 if dt == torch.float16 else 2e-6
    assert torch.allclose(got.float(), hb.float(), rtol=tol, atol=tol)
    if b * hidden * s <= 64 * 512 * 16384:
        xh, wh = x.float().cpu().numpy(), w13.float().cpu().numpy()
        want = O.matmul(xh, np.ascontiguousarray(wh[:hidden]))
        O.silu(want, O.matmul(xh, np.ascontiguousarray(wh[hidden:])))
        assert_close(got.float().cpu().numpy(), want, what="fused w1, w3, silu")
    # some hundred rows and a wide [w1; w3]: one product of the vendor library, then the gate over the two halves of each row
    wide = dt == torch.float16 and 128 <= b < product_route.ROWS and 2 * hidden >= 16384 and s % 8 == 0 and hidden % 8 == 0
    plain = 2 if dt == torch.float16 and product_route.wanted(b, s, hidden) else 0        # the two separate products above
    product_route.check(plain + (1 if wide else 0))


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [Shape(dim=32, n_layers=1, n_heads=4, n_kv_heads=2, hidden_dim=48, seq_len=16),
                                   Shape(dim=288, n_layers=1, n_heads=6, n_kv_heads=6, hidden_dim=768, seq_len=256),
                                   Shape(dim=1024, n_layers=1, n_heads=8, n_kv_heads=2, hidden_dim=64, seq_len=320)],
                         ids=["tiny", "stories15m", "gqa4"])
def test_matmul_qkv_rope_append(dt, shape):
    batch = 5
    arena_a = Arena(shape, batch, dt, seed=3)
    arena_b = Arena(shape, batch, dt, seed=3)
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn((batch, shape.dim), generator=g, device="cuda").to(dt)
    wqkv = (torch.randn((shape.dim + 2 * shape.kv_dim, shape.dim), generator=g, device="cuda") / shape.dim ** 0.5).to(dt)
    re32, im32 = O.rope_tables(shape.seq_len, shape.head_size)
    re, im = torch.from_numpy(re32).cuda().to(dt), torch.from_numpy(im32).cuda().to(dt)
    pos = [0, 3, shape.seq_len - 1, 7, 1]
    present = [True, True, True, False, True]
    dpos = torch.tensor(pos, dtype=torch.int32, device="cuda")
    rows_a = ops.row_table([arena_a.row_ptr(i, pos[i]) if present[i] else 0 for i in range(batch)])
    rows_b = ops.row_table([arena_b.row_ptr(i, pos[i]) if present[i] else 0 for i in range(batch)])
    # separate ops: matmul q, matmul kv, append, rope
    q = ops.matmul(x, wqkv[: shape.dim].contiguous())
    kv = ops.matmul(x, wqkv[shape.dim:].contiguous())
    ops.kv_append(rows_a, kv, shape.kv_dim)
    ops.rope(dpos, re, im, q, rows_a, shape)
    # fused
    q2, kv2 = ops.matmul_qkv_rope_append(x, wqkv, dpos, re, im, rows_b, shape, want_kv=True)
    # one (dim + 2 kv_dim, dim) product vs two separate ones: K may be split differently, so equality
    # holds to the last bit of the fp32 sums only
    tol = 2e-3 if dt == torch.float16 else 2e-6
    assert torch.allclose(q2.float(), q.float(), rtol=tol, atol=tol)
    assert torch.allclose(kv2.float(), kv.float(), rtol=tol, atol=tol)
    assert torch.allclose(arena_b.dev.float(), arena_a.dev.float(), rtol=tol, atol=tol)
    for i in range(batch):
        if present[i]:
            # the appended V half is exactly the (unrotated) matmul result the call reports
            assert torch.equal(arena_b.dev[i, pos[i], shape.kv_dim:], kv2[i, shape.kv_dim:])
        else:
            assert torch.equal(q2[i], kv2.new_tensor(q2[i]))      # finite, untouched by RoPE (checked via the oracle below)
    # rows other than the appended ones are untouched bit for bit
    before = torch.from_numpy(arena_b.host).cuda()
    mask = torch.ones(before.shape[:2], dtype=torch.bool, device="cuda")
    for i in range(batch):
        if present[i]:
            mask[i, pos[i]] = False
    assert torch.equal(arena_b.dev[mask], before[mask])


@pytest.mark.parametrize("name,dtype", [("test-gqa4", "f16"), ("stories15m", "f32"), ("test-tiny", "f32")])
def test_stage_with_and_without_fused_projections(name, dtype):
    cfg = SHAPES[name]
    np_dt = np.float16 if dtype == "f16" else np.float32
    wcls = name != "stories15m"
    layers, base = make_weights(cfg, np_dt, seed=31, wcls=wcls)
    batch = 4
    a = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True, fused_projections=True)
    b = S.Stage(name, dtype, 0, cfg.n_layers, batch, batch, with_cls=True, fused_projections=False)
    ref = OracleModel(cfg, layers, base)
    ref16 = OracleModel(cfg, layers, base, np.float16) if dtype == "f16" else None
    for st in (a, b):
        load_weights(st, cfg, layers, base, wcls)
        st.new_state(batch)
        for i in range(batch):
            st.set_prompt(i, i, 3 + i, 0)
    tokens = [3 + i for i in range(batch)]
    for step in range(8):
        want = ref.step(tokens, list(range(batch)), [step] * batch)
        assert a.forward() and b.forward()
        la = d2h(a.scratch_ptr("logits"), (batch, cfg.vocab_size), np_dt).astype(np.float32)
        lb = d2h(b.scratch_ptr("logits"), (batch, cfg.vocab_size), np_dt).astype(np.float32)
        # the two differ in reduction order only: the rmsnorm sum, and the K split of a concatenated
        # projection against the split of its parts (an fp16 rounding can flip and travel through the layers)
        tol = 8e-3 if dtype == "f16" else 2e-5
        np.testing.assert_allclose(la, lb, rtol=tol, atol=tol)
        if dtype == "f16":
            want16 = ref16.step(tokens, list(range(batch)), [step] * batch)
            assert_half_parity(la, want16, want, what=f"{name} fused-projection logits step {step}")
            assert_half_parity(lb, want16, want, what=f"{name} separate-projection logits step {step}")
        else:
            assert_close(la, want, mean_rel=1e-3, what=f"{name} fused-projection logits step {step}")
        tokens = [a.row(i)["token"] for i in range(batch)]
        for i in range(batch):                         # keep both stages on the same token stream
            b.set_prompt(i, i, tokens[i], step + 1)
            a.set_prompt(i, i, tokens[i], step + 1)
    a.close()
    b.close()
