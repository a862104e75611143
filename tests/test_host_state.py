"""Wire format and batch surgery of BatchedInferenceState (reference: models/common/state.hh:17-50
packed records, :512-594 serialize/parse, :596-648 set_prompt/check_finished/discard, :696-752
replenish_from, :760-1050 split/merge), against byte strings written out by hand with `struct`,
the numpy record types of glinthawk_amd.wire, and list/slice models.  Host only, no GPU."""
import struct

import numpy as np
import pytest

from glinthawk_amd import wire
from glinthawk_amd._lib import GlintError
from glinthawk_amd.wire import HostState

DIM, KV = HostState.DIM, HostState.KV_DIM


def test_known_bytes():
    s = HostState(2, "f16", route_id=0x01020304, model_id=0x0A0B0C0D)
    s.set_meta(id=0x1122334455667788, next_layer=7, next_stage=2, next_tier=-1, next_rank=3, is_sharded=True)
    pid = bytes(range(32))
    s.set_prompt(0, pid, context_id=0xCAFEBABE, token=31999, token_pos=12, temperature=0.5, prompt_length=9,
                 max_completion_length=100, kv_tier=1, kv_rank=200)
    # row 1 stays default: inactive, kv_tier -1
    kv = s.buffer(2, allocate=True)
    kv[:] = np.arange(kv.size, dtype=np.uint8)
    want = struct.pack("<QIBIIIBbB4B", 0x1122334455667788, 2, 0, 0x01020304, 0x0A0B0C0D, 7, 2, -1, 3, 0, 0, 1, 1)
    assert len(want) == 32
    want += struct.pack("<B32sIIIBIIBbB", 1, pid, 0xCAFEBABE, 31999, 12, 127, 9, 100, 0, 1, 200)
    want += struct.pack("<B32sIIIBIIBbB", 0, b"\0" * 32, 0, 0, 0, 0, 0, 0, 0, -1, 0)
    assert len(want) == 32 + 2 * 57
    want += bytes(range(2 * 2 * KV * 2))          # 2 rows x (K|V) x fp16
    assert s.serialize() == want
    # and back
    t = HostState.parse(want)
    assert t.serialize() == want and t.batch_size() == 2 and t.free_slots() == 1 and not t.all_assigned_to_nodes()


@pytest.mark.parametrize("t,code", [(0.0, 0), (0.5, 127), (1.0, 255), (0.999, 254), (1 / 255, 1), (0.2, 51)])
def test_temperature_is_truncated_to_a_byte(t, code):
    s = HostState(1, "f32")
    s.set_prompt(0, b"", 1, 2, 3, t, 0, 0, 0, 0)
    _, p, *_ = wire.unpack_state(s.serialize(), DIM, KV)
    assert p[0]["temperature"] == int(np.float32(t) * np.float32(255.0)) == code


def random_state(rng, batch, dtype):
    code = wire.DTYPE_CODE[dtype]
    np_dt = np.float16 if dtype == "f16" else np.float32
    p = wire.new_prompts(batch)
    for name in ("context_id", "token", "token_pos", "prompt_length", "max_completion_length"):
        p[name] = rng.integers(0, 2**32, batch, dtype=np.uint64)
    p["active"] = rng.integers(0, 2, batch)
    p["finished"] = rng.integers(0, 2, batch)
    p["temperature"] = rng.integers(0, 256, batch)
    p["kv_tier"] = rng.integers(-1, 4, batch)
    p["kv_rank"] = rng.integers(0, 256, batch)
    p["prompt_id"] = rng.integers(0, 256, (batch, 32))
    have = rng.integers(0, 2, 3).astype(bool)
    bufs = [rng.standard_normal((batch, n)).astype(np_dt) if h else None for h, n in zip(have, (DIM, DIM, 2 * KV))]
    meta = dict(id=int(rng.integers(0, 2**63)), dtype=code, route_id=int(rng.integers(0, 2**32)), model_id=int(rng.integers(0, 2**32)),
                next_layer=int(rng.integers(0, 80)), next_stage=int(rng.integers(0, 4)), next_tier=int(rng.integers(-1, 3)),
                next_rank=int(rng.integers(0, 256)), is_sharded=int(rng.integers(0, 2)))
    return meta, p, bufs


def test_round_trips_between_numpy_and_the_host_layer():
    rng = np.random.default_rng(70)
    for trial in range(60):
        batch = int(rng.integers(0, 9))
        dtype = ("f16", "f32")[trial % 2]
        meta, p, bufs = random_state(rng, batch, dtype)
        raw = wire.pack_state(meta, p, *bufs)
        s = HostState.parse(raw)
        assert s.serialize() == raw                                   # parse then serialize: identity on bytes
        m2, p2, a2, q2, k2 = wire.unpack_state(raw, DIM, KV)
        assert int(m2["batch_size"]) == batch and all(m2[k] == v for k, v in meta.items())
        assert np.array_equal(p2, p)
        for got, want in zip((a2, q2, k2), bufs):
            assert (got is None) == (want is None) and (got is None or np.array_equal(got, want))
        assert s.free_slots() == int((p["active"] == 0).sum())
        assert s.all_assigned_to_nodes() == bool((p["kv_tier"] != -1).all())


def test_parse_refuses_malformed_input():
    rng = np.random.default_rng(71)
    meta, p, bufs = random_state(rng, 3, "f16")
    bufs = [np.zeros((3, DIM), np.float16), None, np.zeros((3, 2 * KV), np.float16)]
    raw = wire.pack_state(meta, p, *bufs)
    HostState.parse(raw)
    for cut in (0, 5, 31):
        with pytest.raises(GlintError, match="too small to contain metadata"):
            HostState.parse(raw[:cut])
    for cut in (32, 32 + 57, 32 + 3 * 57, len(raw) - 1):
        with pytest.raises(GlintError, match="too small for its batch size"):
            HostState.parse(raw[:cut])
    with pytest.raises(GlintError, match="more data than expected"):
        HostState.parse(raw + b"\0")
    bad = bytearray(raw)
    bad[12] = 9                                                       # dtype byte
    with pytest.raises(GlintError, match="unknown data type"):
        HostState.parse(bytes(bad))
    bad = bytearray(raw)
    bad[25] = 4                                                       # next_stage byte: __COUNT__ is not a stage
    with pytest.raises(GlintError, match="unknown next stage"):
        HostState.parse(bytes(bad))
    bad = bytearray(raw)
    bad[29] = 1                                                       # claims queries that are not there
    with pytest.raises(GlintError, match="too small for its batch size"):
        HostState.parse(bytes(bad))


def test_discard_keeps_the_slot_identity():
    s = HostState(2, "f16")
    s.set_prompt(1, b"x" * 32, 77, 5, 6, 1.0, 7, 8, 2, 9)
    s.set_finished(1)
    s.discard(1)
    _, p, *_ = wire.unpack_state(s.serialize(), DIM, KV)
    want = wire.new_prompts(1)[0]
    want["context_id"], want["kv_tier"], want["kv_rank"] = 77, 2, 9
    assert p[1] == want


@pytest.mark.parametrize("token,pos,plen,mcl,want", [
    (2, 3, 1, 0, True),            # EOS with no completion cap
    (1, 3, 1, 0, False),           # BOS is not an end token (Llama2: EOS = EOT = 2, models/llama2/variants.hh:40-42)
    (2, 3, 1, 10, False),          # EOS is ignored while a completion length is set
    (5, 15, 1, 0, False), (5, 16, 1, 0, True),        # out of sequence at seq_len = 16
    (5, 10, 4, 6, True), (5, 9, 4, 6, False),         # prompt + completion cap reached
])
def test_check_finished(token, pos, plen, mcl, want):
    s = HostState(1, "f16")
    s.set_prompt(0, b"", 1, token, pos, 0.0, plen, mcl, 0, 0)
    assert s.check_finished(0) == want


def test_positions_beyond_the_window_are_refused_before_any_launch():
    """A position parsed from the wire is not trusted: the stage driver's forward entry points check
    every row that owns a context slot against seq_len on the host (rows past the window would address
    cache rows and RoPE table entries outside their allocations).  Inactive rows hold the shared empty
    context, which every op skips, so their positions do not matter."""
    seq = HostState.SEQ_LEN
    s = HostState(3, "f16")
    s.set_prompt(0, b"a" * 32, 1, 5, 0, 0.0, 1, 0, 0, 0)
    s.set_prompt(1, b"b" * 32, 2, 5, seq - 1, 0.0, 1, 0, 0, 0)
    assert s.positions_fit(seq)
    s.set_prompt(2, b"c" * 32, 3, 5, seq, 0.0, 1, 0, 0, 0)
    assert not s.positions_fit(seq)
    assert s.positions_fit(seq + 1)
    # the same through the wire: parse() accepts the bytes, the check refuses the state
    back = HostState.parse(s.serialize())
    assert not back.positions_fit(seq)
    s.discard(2)                                   # an inactive row is never addressed
    assert s.positions_fit(seq)
    huge = HostState(1, "f16")
    huge.set_prompt(0, b"d" * 32, 1, 5, 0xFFFFFFFF, 0.0, 1, 0, 0, 0)
    assert not huge.positions_fit(seq)


def fill(state: HostState, prompts: np.ndarray, rng, which=(0, 2)):
    for i, r in enumerate(prompts):
        if r["active"]:
            state.set_prompt(i, bytes(r["prompt_id"]), int(r["context_id"]), int(r["token"]), int(r["token_pos"]),
                             float(r["temperature"]) / 255.0 + 1e-4, int(r["prompt_length"]), int(r["max_completion_length"]),
                             int(r["kv_tier"]), int(r["kv_rank"]))
        else:
            state.set_prompt(i, b"", int(r["context_id"]), 0, 0, 0.0, 0, 0, int(r["kv_tier"]), int(r["kv_rank"]))
            state.discard(i)
    for w in which:
        b = state.buffer(w, allocate=True)
        b[:] = rng.integers(0, 256, b.size, dtype=np.uint8)


def view(state: HostState):
    """Unpacked state with the buffers as raw integer words (random bytes may spell NaNs)."""
    m, p, *bufs = wire.unpack_state(state.serialize(), DIM, KV)
    bits = [None if b is None else b.view(np.uint16 if b.itemsize == 2 else np.uint32) for b in bufs]
    return (m, p, *bits)


def test_replenish_from_against_a_list_model():
    rng = np.random.default_rng(72)
    for trial in range(40):
        batch = int(rng.integers(1, 10))
        _, mine, _ = random_state(rng, batch, "f16")
        _, theirs, _ = random_state(rng, batch, "f16")
        mine["context_id"] = rng.integers(1, 1000, batch)       # slots own a context
        theirs["context_id"] = 0                                  # fresh prompts carry none
        a, b = HostState(batch, "f16"), HostState(batch, "f16")
        fill(a, mine, rng)
        fill(b, theirs, rng)
        _, pa, aa, _, ka = view(a)
        _, pb, ab, _, kb = view(b)
        # model: walk my inactive rows, take their active rows in order
        donors = [j for j in range(batch) if pb[j]["active"]]
        want_p, want_a, want_k, left = pa.copy(), aa.copy(), ka.copy(), pb.copy()
        ok = True
        for i in range(batch):
            if want_p[i]["active"]:
                continue
            if not donors:
                ok = False
                break
            j = donors.pop(0)
            ctx = want_p[i]["context_id"]
            want_p[i] = pb[j]
            want_p[i]["context_id"] = ctx
            want_a[i], want_k[i] = ab[j], kb[j]
            left[j] = wire.new_prompts(1)[0]
        assert a.replenish_from(b) == ok
        _, pa2, aa2, _, ka2 = view(a)
        _, pb2, *_ = view(b)
        assert np.array_equal(pa2, want_p) and np.array_equal(aa2, want_a) and np.array_equal(ka2, want_k)
        assert np.array_equal(pb2, left)


def test_split_and_merge_are_inverse():
    rng = np.random.default_rng(73)
    for trial in range(30):
        batch = int(rng.integers(2, 12))
        _, prompts, _ = random_state(rng, batch, "f32")
        prompts["active"] = 1
        s = HostState(batch, "f32", 3, 4)
        s.set_meta(id=99, next_layer=5, next_stage=1, next_tier=1, next_rank=2)
        fill(s, prompts, rng, which=(0, 1, 2))
        raw = s.serialize()
        m, p, a, q, k = view(s)
        n = int(rng.integers(1, batch))
        x, y = s.split(n)
        assert s.serialize() == raw                                  # split leaves the source alone
        mx, px, ax, qx, kx = view(x)
        my, py, ay, qy, ky = view(y)
        assert int(mx["batch_size"]) == n and int(my["batch_size"]) == batch - n
        for name in m.dtype.names:
            if name != "batch_size":
                assert mx[name] == m[name] == my[name]
        assert np.array_equal(px, p[:n]) and np.array_equal(py, p[n:])
        assert np.array_equal(ax, a[:n]) and np.array_equal(qy, q[n:]) and np.array_equal(ky, k[n:])
        x.merge(y)
        assert x.serialize() == raw and y.batch_size() == 0
        empty = HostState()
        empty.merge(x)                                               # merging into an empty state adopts the other
        assert empty.serialize() == raw


def test_split_on_kv_cuts_at_placement_changes():
    rng = np.random.default_rng(74)
    for trial in range(30):
        batch = int(rng.integers(1, 14))
        _, prompts, _ = random_state(rng, batch, "f16")
        prompts["active"] = 1
        prompts["kv_tier"] = rng.integers(0, 2, batch)
        prompts["kv_rank"] = rng.integers(0, 2, batch)
        s = HostState(batch, "f16")
        fill(s, prompts, rng, which=(1,))
        raw = s.serialize()
        _, p, _, q, _ = view(s)
        cuts = [0] + [i for i in range(1, batch) if (p[i]["kv_tier"], p[i]["kv_rank"]) != (p[i - 1]["kv_tier"], p[i - 1]["kv_rank"])] + [batch]
        pieces = s.split_on_kv()
        assert len(pieces) == len(cuts) - 1
        assert s.batch_size() == 0                                   # the source is consumed
        for piece, lo, hi in zip(pieces, cuts[:-1], cuts[1:]):
            _, pp, _, qq, _ = view(piece)
            assert np.array_equal(pp, p[lo:hi]) and np.array_equal(qq, q[lo:hi])
            assert len({(int(r["kv_tier"]), int(r["kv_rank"])) for r in pp}) == 1
        whole = pieces[0]
        for piece in pieces[1:]:
            whole.merge(piece)
        assert whole.serialize() == raw
