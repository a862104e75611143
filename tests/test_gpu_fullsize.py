"""The headline configuration at its real size -- Llama2-70B GQA shape, decode batch 64, 4096 keys
per context -- against the CPU oracle on the same inputs (the oracle's attention takes well under a
second per layer at this size) and against properties that do not depend on size."""
import numpy as np
import pytest
import torch

import oracle as O
from glinthawk_amd import Shape, ops, stage as S
from glinthawk_amd._lib import GH_ATTN_GENERIC, GH_ATTN_MFMA, GH_ATTN_VALU
from helpers import assert_close, assert_half_parity, errors, oracle_cfg

pytestmark = pytest.mark.gpu

SHAPE = Shape(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096)
BATCH = 64


@pytest.fixture(scope="module")
def arena():
    ops.init(0)
    cache = torch.empty((BATCH, SHAPE.seq_len, 2 * SHAPE.kv_dim), dtype=torch.float16, device="cuda")
    ops.fill_normal(cache, 0.0, 1.0, 5)
    row_bytes = 2 * SHAPE.kv_dim * 2
    layers = ops.row_table([cache.data_ptr() + i * SHAPE.seq_len * row_bytes for i in range(BATCH)])
    return cache, layers, row_bytes


def test_attention_op_at_full_size_against_the_oracle(arena):
    cache, layers, row_bytes = arena
    rng = np.random.default_rng(6)
    # ragged: most contexts at the last position, some short, one at position 0
    pos = np.full(BATCH, SHAPE.seq_len - 1)
    pos[:8] = [0, 1, 15, 16, 255, 1023, 2048, 4000]
    q = rng.standard_normal((BATCH, SHAPE.dim)).astype(np.float16)
    kv = rng.standard_normal((BATCH, 2 * SHAPE.kv_dim)).astype(np.float16)
    re, im = O.rope_tables(SHAPE.seq_len, SHAPE.head_size)
    re16, im16 = re.astype(np.float16), im.astype(np.float16)

    dq = torch.from_numpy(q).cuda()
    dpos = torch.from_numpy(pos.astype(np.int32)).cuda()
    token_rows = ops.row_table([cache.data_ptr() + (i * SHAPE.seq_len + int(pos[i])) * row_bytes for i in range(BATCH)])
    ops.kv_append(token_rows, torch.from_numpy(kv).cuda(), SHAPE.kv_dim)
    ops.rope(dpos, torch.from_numpy(re16).cuda(), torch.from_numpy(im16).cuda(), dq, token_rows, SHAPE)
    xb = torch.zeros_like(dq)
    ws = torch.empty(ops.attn_decode_workspace(BATCH, SHAPE.seq_len - 1, SHAPE), dtype=torch.uint8, device="cuda")
    ops.attn_decode(dq, layers, dpos, xb, int(pos.max()), SHAPE, workspace=ws)
    got = xb.float().cpu().numpy()

    # oracle on fp32 copies of the very same rows (the appended row included, K not yet rotated)
    host = cache.cpu().numpy()
    cfg = oracle_cfg(SHAPE)
    ctx_layers = []
    for i in range(BATCH):
        rows = host[i].astype(np.float32)
        rows[int(pos[i]), :SHAPE.kv_dim] = kv[i, :SHAPE.kv_dim].astype(np.float32)     # un-rotated K, as the oracle rotates itself
        ctx_layers.append(np.ascontiguousarray(rows))
    del host
    want = O.attention_ops(cfg, pos.tolist(), re16.astype(np.float32), im16.astype(np.float32), q.astype(np.float32), ctx_layers)
    assert_close(got, want, what="decode attention, 64 x 4096 keys, GQA 8")
    # position 0 attends a single key: the output is that key's V row for every head of the group
    v0 = kv[0, SHAPE.kv_dim:].astype(np.float32).reshape(SHAPE.n_kv_heads, 1, SHAPE.head_size)
    assert np.array_equal(got[0].reshape(SHAPE.n_kv_heads, SHAPE.gqa_size, SHAPE.head_size), np.broadcast_to(v0, (SHAPE.n_kv_heads, SHAPE.gqa_size, SHAPE.head_size)))

    # the three kernels agree with each other at this size
    for variant in (GH_ATTN_GENERIC, GH_ATTN_VALU):
        other = torch.zeros_like(dq)
        ops.attn_decode(dq, layers, dpos, other, int(pos.max()), SHAPE, workspace=ws, variant=variant)
        a, r = errors(other.float().cpu().numpy(), got)
        assert a < 4e-3 and r < 1e-3, (variant, a, r)


def test_uniform_values_pass_through_at_full_size(arena):
    cache, layers, row_bytes = arena
    # every V row of a context equal to one vector: any convex combination returns that vector
    rng = np.random.default_rng(7)
    v = torch.from_numpy(rng.standard_normal((BATCH, 1, SHAPE.kv_dim)).astype(np.float16)).cuda()
    saved = cache[:, :, SHAPE.kv_dim:].clone()
    cache[:, :, SHAPE.kv_dim:] = v
    q = torch.randn((BATCH, SHAPE.dim), dtype=torch.float16, device="cuda")
    pos = torch.full((BATCH,), SHAPE.seq_len - 1, dtype=torch.int32, device="cuda")
    xb = torch.zeros_like(q)
    ws = torch.empty(ops.attn_decode_workspace(BATCH, SHAPE.seq_len - 1, SHAPE), dtype=torch.uint8, device="cuda")
    ops.attn_decode(q, layers, pos, xb, SHAPE.seq_len - 1, SHAPE, workspace=ws, variant=GH_ATTN_MFMA)
    want = v.reshape(BATCH, SHAPE.n_kv_heads, 1, SHAPE.head_size).expand(-1, -1, SHAPE.gqa_size, -1).reshape(BATCH, SHAPE.dim)
    assert (xb.float() - want.float()).abs().max().item() < 2e-3
    cache[:, :, SHAPE.kv_dim:] = saved


@pytest.mark.parametrize("BATCH,limit", [(64, 64), (17, 64)])
def test_one_full_layer_of_the_stage_against_the_oracle(BATCH, limit):
    """One hosted layer of the 70B shape, every context at position 4095: the C++ stage driver (fused
    projections, fused attention) against the oracle's layer on the same weights and cache rows.  Once with
    a full batch and once with 17 rows on a stage whose concurrency limit is 64: the smaller batch is cut
    into more splits per context and needs more split partials than the full one, out of a workspace
    that was sized when the stage was built."""
    cfg = oracle_cfg(SHAPE)
    layer = 40
    st = S.Stage("llama2-70b-4k", "f16", layer, 1, limit, BATCH)
    rng = np.random.default_rng(8)
    block = rng.standard_normal(1 << 22).astype(np.float32)

    def tiled(shape, scale, shift=0.0):
        n = int(np.prod(shape))
        reps = (n + block.size - 1) // block.size + 1
        off = int(rng.integers(0, block.size))
        return (np.tile(block, reps)[off:off + n] * np.float32(scale) + np.float32(shift)).astype(np.float16).reshape(shape)

    s_in = 1.0 / np.sqrt(SHAPE.dim)
    w16 = {
        "rms_att_weight": tiled((SHAPE.dim,), 0.1, 1.0), "wq": tiled((SHAPE.dim, SHAPE.dim), s_in),
        "wkv": tiled((2 * SHAPE.kv_dim, SHAPE.dim), s_in), "wo": tiled((SHAPE.dim, SHAPE.dim), s_in),
        "rms_ffn_weight": tiled((SHAPE.dim,), 0.1, 1.0), "w1": tiled((SHAPE.hidden_dim, SHAPE.dim), s_in),
        "w2": tiled((SHAPE.dim, SHAPE.hidden_dim), 1.0 / np.sqrt(SHAPE.hidden_dim)), "w3": tiled((SHAPE.hidden_dim, SHAPE.dim), s_in),
    }
    for name, arr in w16.items():
        st.set_layer_tensor(layer, name, arr)
    re, im = O.rope_tables(SHAPE.seq_len, SHAPE.head_size)
    re16, im16 = re.astype(np.float16), im.astype(np.float16)
    st.set_base_tensor("freq_cis_real", re16)
    st.set_base_tensor("freq_cis_imag", im16)

    pos = SHAPE.seq_len - 1
    st.new_state(BATCH, next_layer=layer)
    for i in range(BATCH):
        st.set_prompt(i, 300 + i, 1, pos)
    assert st.acquire_contexts()
    from glinthawk_amd import _lib
    L = _lib.lib()
    n_rows_elems = SHAPE.seq_len * 2 * SHAPE.kv_dim
    for i in range(BATCH):
        _lib.check(L.gh_fill_normal(st.context_layer_ptr(i, layer), n_rows_elems, 0.0, 1.0, 900 + i, _lib.GH_F16, None))
    ops.sync()
    ctx_layers = []
    for i in range(BATCH):
        rows = np.empty((SHAPE.seq_len, 2 * SHAPE.kv_dim), np.float16)
        _lib.check(L.gh_memcpy(rows.ctypes.data, st.context_layer_ptr(i, layer), rows.nbytes, _lib.GH_D2H, 0, None))
        ctx_layers.append(rows.astype(np.float32))
    x = rng.standard_normal((BATCH, SHAPE.dim)).astype(np.float16)
    st.activations(allocate=True)[:] = x.reshape(-1)
    assert st.forward()
    got = st.activations().reshape(BATCH, SHAPE.dim).astype(np.float32)

    w32 = {k: v.astype(np.float32) for k, v in w16.items()}
    x32 = x.astype(np.float32)
    x16 = x.copy()
    half_layers = [rows.astype(np.float16) for rows in ctx_layers]        # exact: the rows came from the device as fp16
    O.layer_forward(cfg, w32, re16.astype(np.float32), im16.astype(np.float32), x32, ctx_layers, [pos] * BATCH)
    O.layer_forward(cfg, w16, re16, im16, x16, half_layers, [pos] * BATCH)
    # residual stream after one layer against the CPU path in both storage types
    # a single layer is shallow enough for the comparison with the fp16 oracle to be tight as well (measured 1.9e-4)
    assert_half_parity(got, x16, x32, what=f"70B layer, B={BATCH} of {limit}, position 4095", tol16=3e-4)
    # the appended rows (K rotated, V raw) landed where the oracle put them
    row = np.empty(2 * SHAPE.kv_dim, np.float16)
    for i in (0, BATCH // 2, BATCH - 1):
        _lib.check(L.gh_memcpy(row.ctypes.data, st.context_layer_ptr(i, layer) + pos * row.nbytes, row.nbytes, _lib.GH_D2H, 0, None))
        a, r = errors(row.astype(np.float32), ctx_layers[i][pos])
        assert a < 2e-2 and r < 2e-3, (i, a, r)
    st.close()
