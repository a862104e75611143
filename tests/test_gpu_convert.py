"""convert_and_copy (arch/amd64/llama2/ops.hh:354-368, arch/cuda/llama2/ops.cuh:455-492) through the
C-ABI, bit for bit against the oracle's element-wise casts for every copy kind, and the use the
reference makes of it: an attention stage whose storage type differs from the type the state
travels in (models/llama2/model.hh:632-690,699-720)."""
import numpy as np
import pytest
import torch

import oracle as O
from glinthawk_amd import ops, stage as S, wire
from glinthawk_amd._lib import GH_D2D, GH_D2H, GH_H2D, GH_H2H, GlintError
from helpers import assert_close
from test_gpu_stage import SHAPES, load_weights, make_weights
from test_gpu_wire import prompts_for

pytestmark = pytest.mark.gpu

TORCH = {np.float16: torch.float16, np.float32: torch.float32}


def cast_inputs(n, src_dt, seed):
    """Values that exercise the cast: ordinary numbers, halfway cases between neighbouring halves, the
    overflow threshold, subnormals, signed zeros, infinities and a NaN."""
    r = np.random.default_rng(seed)
    x = (r.standard_normal(n) * 10.0 ** r.integers(-8, 5, n)).astype(np.float32)
    halves = np.arange(0, 65536, 97, dtype=np.uint16).view(np.float16).astype(np.float32)
    halves = halves[np.isfinite(halves)]
    mids = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    edge = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14,
                     np.inf, -np.inf, np.nan], dtype=np.float32)
    x = np.concatenate([edge, mids, x])[:n]          # a short array gets the first few special values only
    if src_dt == np.float16:
        with np.errstate(over="ignore"):
            return x.astype(np.float16)
    return x


def same_bits(got, want):
    nan = np.isnan(want.astype(np.float32))
    assert np.array_equal(np.isnan(got.astype(np.float32)), nan)
    u = np.uint16 if want.dtype == np.float16 else np.uint32
    assert np.array_equal(got.view(u)[~nan], want.view(u)[~nan])


@pytest.mark.parametrize("src_dt,dst_dt", [(np.float32, np.float16), (np.float16, np.float32), (np.float16, np.float16), (np.float32, np.float32)])
@pytest.mark.parametrize("n", [1, 7, 4096 + 3, 300001])
def test_convert_and_copy_every_kind_is_bit_exact(src_dt, dst_dt, n):
    ops.init(0)
    src = cast_inputs(n, src_dt, seed=n)
    want = O.convert(src, dst_dt)

    # host -> device
    d_dst = torch.zeros(n + 8, dtype=TORCH[dst_dt], device="cuda")
    ops.convert_and_copy(d_dst, src, n, GH_H2D)
    same_bits(d_dst[:n].cpu().numpy(), want)
    assert float(d_dst[n:].abs().sum()) == 0.0                     # nothing written past n

    # device -> host
    d_src = torch.from_numpy(src).cuda()
    h_dst = np.zeros(n + 8, dtype=dst_dt)
    ops.convert_and_copy(h_dst, d_src, n, GH_D2H)
    same_bits(h_dst[:n], want)
    assert not h_dst[n:].any()

    # device -> device, synchronous and asynchronous forms
    d_dst.zero_()
    ops.convert_and_copy(d_dst, d_src, n, GH_D2D)
    same_bits(d_dst[:n].cpu().numpy(), want)
    d_dst.zero_()
    ops.convert(d_dst, d_src, n)
    ops.sync()
    same_bits(d_dst[:n].cpu().numpy(), want)
    assert float(d_dst[n:].abs().sum()) == 0.0

    # host -> host: a plain copy when the types agree; a device target refuses a converting one
    h_dst = np.zeros(n, dtype=dst_dt)
    if src_dt == dst_dt:
        ops.convert_and_copy(h_dst, src, n, GH_H2H)
        same_bits(h_dst, want)
    else:
        with pytest.raises(GlintError, match="device side"):
            ops.convert_and_copy(h_dst, src, n, GH_H2H)


def test_convert_and_copy_refuses_bad_arguments():
    ops.init(0)
    d = torch.zeros(4, dtype=torch.float16, device="cuda")
    h = np.zeros(4, dtype=np.float32)
    with pytest.raises(GlintError):
        ops.convert_and_copy(d, h, 4, 9)
    ops.convert_and_copy(d, h, 0, GH_H2D)                          # nothing to do is not an error


def attention_state(dtype_name, batch, layer, cids, pos, q, kv):
    meta = dict(id=9, dtype=wire.DTYPE_CODE[dtype_name], next_layer=layer, next_stage=S.STAGE_ATT)
    return wire.pack_state(meta, prompts_for(batch, cids, [1] * batch, pos), queries=q, kvs=kv)


@pytest.mark.parametrize("fused", [True, False])
def test_attention_stage_takes_a_state_of_the_other_type(fused):
    """An fp16 attention stage fed queries and K/V rows as fp32 (the wire type of an fp32 neighbour):
    the import rounds them like the oracle's cast, the cache and the output are then exactly those of the
    same stage fed the rounded values as fp16, and the output leaves converted back to fp32."""
    name = "test-gqa4"
    cfg = SHAPES[name]
    layers, base = make_weights(cfg, np.float16, seed=91, wcls=True)
    batch, layer = 4, 1
    a = S.Stage(name, "f16", 0, cfg.n_layers, batch, batch, fused=fused)
    b = S.Stage(name, "f16", 0, cfg.n_layers, batch, batch, fused=fused)
    for st in (a, b):
        load_weights(st, cfg, layers, base, True, with_cls=False)
    rng = np.random.default_rng(92)
    cids = [5, 6, 7, 8]
    cache32 = [np.zeros((cfg.seq_len, 2 * cfg.kv_dim), np.float32) for _ in range(batch)]
    re = base["freq_cis_real"].astype(np.float32)
    im = base["freq_cis_imag"].astype(np.float32)
    ocfg = cfg
    for step in range(6):
        pos = [step] * batch
        q32 = rng.standard_normal((batch, cfg.dim)).astype(np.float32)              # not representable in fp16
        kv32 = rng.standard_normal((batch, 2 * cfg.kv_dim)).astype(np.float32)
        q16, kv16 = O.convert(q32, np.float16), O.convert(kv32, np.float16)
        a.set_state_bytes(attention_state("f16", batch, layer, cids, pos, q16, kv16))
        assert a.forward(S.FWD_ATT)
        b.set_state_bytes(attention_state("f32", batch, layer, cids, pos, q32, kv32))
        assert b.forward(S.FWD_ATT)
        ma, _, _, out_a, _ = wire.unpack_state(a.get_state_bytes(), cfg.dim, cfg.kv_dim)
        mb, _, _, out_b, _ = wire.unpack_state(b.get_state_bytes(), cfg.dim, cfg.kv_dim)
        assert int(ma["dtype"]) == wire.DTYPE_CODE["f16"] and int(mb["dtype"]) == wire.DTYPE_CODE["f32"]
        assert int(mb["next_stage"]) == S.STAGE_POST and int(mb["has_queries"]) == 1
        assert out_a.dtype == np.float16 and out_b.dtype == np.float32
        assert np.array_equal(out_b, out_a.astype(np.float32))                        # export: fp16 -> fp32 is exact
        # against the oracle's attention on the rounded inputs
        kv_rounded = kv16.astype(np.float32)
        O.copy_kv_cache(ocfg, [cache32[i][step] for i in range(batch)], kv_rounded)
        want = O.attention_ops(ocfg, pos, re, im, q16.astype(np.float32), cache32)
        assert_close(out_b, want, what=f"attention from an fp32 state, step {step}")
    a.close()
    b.close()


def test_convert_and_copy_of_void_is_a_byte_copy():
    """The instantiation the reference's concept names, convert_and_copy<void, void>
    (models/llama2/ops/concept.hh:36): its element is a byte (arch/amd64/llama2/ops.hh:361-362 with
    sizeof(void) == 1), so `size` bytes travel unchanged, whatever their number, in every direction."""
    st = S.Stage("test-tiny", "f16", 0, 1, 2, 2)
    rng = np.random.default_rng(5)
    for n in (1, 7, 4099):                                           # odd counts: no element type divides them
        src = rng.integers(0, 256, n, dtype=np.uint8)
        dev = torch.zeros(n + 2, dtype=torch.uint8, device="cuda")
        dev2 = torch.zeros(n + 2, dtype=torch.uint8, device="cuda")
        back = np.zeros(n + 2, dtype=np.uint8)
        st.copy_bytes(dev.data_ptr(), src.ctypes.data, n, GH_H2D)
        st.copy_bytes(dev2.data_ptr(), dev.data_ptr(), n, GH_D2D)
        st.copy_bytes(back.ctypes.data, dev2.data_ptr(), n, GH_D2H)
        assert np.array_equal(back[:n], src) and not back[n:].any()   # nothing beyond `size` bytes
        again = np.zeros(n, dtype=np.uint8)
        st.copy_bytes(again.ctypes.data, src.ctypes.data, n, GH_H2H)
        assert np.array_equal(again, src)
    st.close()
