"""Pins the oracle's integer bookkeeping (KV addressing, paging, slot manager, finish rule)
against brute-force models written independently in Python."""
import collections
import itertools

import numpy as np
import pytest

import oracle as O

CFG = O.Config(dim=32, n_layers=5, n_heads=4, n_kv_heads=2, hidden_dim=48, seq_len=16, vocab_size=64)


def test_context_addressing_brute_force():
    cfg = CFG
    hosted = [1, 0, 1, 1, 0]
    # brute-force model: lay rows out by enumerating (hosted layer, token, K/V, head, elem) in order
    offset = 0
    table = {}
    for layer in range(cfg.n_layers):
        if not hosted[layer]:
            continue
        for pos in range(cfg.seq_len):
            for part in ("k", "v"):
                for h in range(cfg.n_kv_heads):
                    table[(layer, pos, part, h)] = offset
                    offset += cfg.head_size
    assert offset * 4 == O.ctx_max_size_bytes(cfg, sum(hosted), 4)
    for layer, pos, h in itertools.product(range(cfg.n_layers), range(cfg.seq_len), range(cfg.n_kv_heads)):
        k = O.ctx_key_head_offset(cfg, hosted, layer, pos, h)
        v = O.ctx_value_head_offset(cfg, hosted, layer, pos, h)
        if hosted[layer]:
            assert k == table[(layer, pos, "k", h)] and v == table[(layer, pos, "v", h)]
        else:
            assert k is None and v is None
    assert O.ctx_layer_offset(cfg, hosted, 2) == cfg.seq_len * 2 * cfg.kv_dim
    assert O.ctx_layer_offset(cfg, hosted, 1) is None


def test_context_size_headline_shape():
    cfg70 = O.Config(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096)
    assert cfg70.kv_dim == 1024 and cfg70.gqa_size == 8 and cfg70.head_size == 128
    assert O.ctx_max_size_bytes(cfg70, 10, 2) == 10 * 16 * 2 ** 20       # 160 MiB per context
    assert O.ctx_max_size_bytes(cfg70, 1, 2) // 4096 == 4096              # 4 KiB rows


@pytest.mark.parametrize("commit_all", [False, True])
def test_dynamic_context_paging_model(commit_all):
    # shape with 4 KiB rows so a 2 MiB block holds 512 rows
    cfg = O.Config(dim=8192, n_layers=3, n_heads=64, n_kv_heads=8, hidden_dim=64, seq_len=4096)
    elem = 2
    row = 2 * cfg.kv_dim * elem
    block = 2 * 2 ** 20
    allocated = np.zeros(cfg.n_layers, np.uint64)
    model = [0] * cfg.n_layers
    rng = np.random.default_rng(5)
    pos = 0
    for step in range(3000):
        layer = step % cfg.n_layers
        if layer == 0:
            pos = 0 if rng.random() < 0.002 else min(pos + 1, cfg.seq_len - 1)
        can_release = pos == 0 and layer == 0
        n, cleared = O.dynctx_prepare(cfg, elem, allocated, layer, pos, can_release, commit_all)
        if can_release:
            model = [0] * cfg.n_layers
        need = (pos + 1) * row
        want_n = 0
        if commit_all:
            while need > model[layer]:
                model[layer] += block
                want_n += 1
        elif need > model[layer]:
            model[layer] += block
            want_n = 1
        assert (n, cleared) == (want_n, can_release)
        assert allocated.tolist() == model
        # sequential growth: the row is always backed after prepare, in both modes
        assert model[layer] >= need
    # a jump straight to a far position: the reference rule commits one block only
    allocated[:] = 0
    n, _ = O.dynctx_prepare(cfg, elem, allocated, 1, 2000, False, commit_all)
    assert n == (4 if commit_all else 1)


def test_context_manager_vs_model():
    rng = np.random.default_rng(11)
    for trial in range(30):
        cap = int(rng.integers(1, 9))
        m = O.ContextManager(cap)
        free = collections.deque(range(cap))
        alloc = {}
        for _ in range(60):
            op = rng.random()
            if op < 0.7:
                bs = int(rng.integers(1, 7))
                active = rng.random(bs) < 0.8
                ids = rng.integers(0, 12, bs).astype(np.uint32)
                start = int(rng.integers(0, bs))
                end = int(rng.integers(start, bs + 1))
                got = m.get_contexts(active, ids, start, end)
                missing = sum(1 for i in range(start, end) if active[i] and int(ids[i]) not in alloc)
                if missing > len(free):
                    assert got is None
                else:
                    want = []
                    for i in range(start, end):
                        if not active[i]:
                            want.append(-1)
                        else:
                            cid = int(ids[i])
                            if cid not in alloc:
                                alloc[cid] = free.popleft()
                            want.append(alloc[cid])
                    assert got == want
            elif op < 0.85:
                cid = int(rng.integers(0, 12))
                got = m.get_context(cid)
                if cid in alloc:
                    assert got == alloc[cid]
                elif not free:
                    assert got == -1
                else:
                    alloc[cid] = free.popleft()
                    assert got == alloc[cid]
            else:
                cid = int(rng.integers(0, 12))
                got = m.release(cid)
                assert got == (cid in alloc)
                if cid in alloc:
                    free.append(alloc.pop(cid))
            assert m.free() == len(free) and m.allocated() == len(alloc)
            assert m.free() + m.allocated() == cap


def test_context_manager_documented_cases():
    m = O.ContextManager(2)
    # duplicate unseen ids in one batch are counted twice in the admission pass, so this is refused
    # although one slot would do; nothing is allocated by a refused call
    assert m.get_contexts([1, 1, 1], [7, 7, 8]) is None
    assert m.free() == 2
    assert m.get_contexts([1, 0, 1], [7, 9, 8]) == [0, -1, 1]
    assert m.get_contexts([1, 1], [8, 7]) == [1, 0]            # sticky ids
    assert m.get_contexts([1], [5]) is None                     # exhausted
    assert m.get_contexts([0], [5]) == [-1]                     # inactive rows never need a slot
    assert m.release(7) and m.get_contexts([1], [5]) == [0]     # FIFO reuse of the released slot


# (token, token_pos, prompt_length, max_completion_length, seq_len, eos, eot) -> finished, each case worked out by hand from the
# three clauses of models/common/state.hh:621-631: an end token only counts while no completion length is set; the position
# bound is `>=`; the completion bound is `>= max_completion_length + prompt_length` and only exists when a length is set.
CHECK_FINISHED_CASES = [
    ((5, 3, 2, 0, 16, 2, 9), False),     # ordinary token, inside the window, no length limit
    ((2, 3, 2, 0, 16, 2, 9), True),      # end of sentence, no length limit
    ((9, 3, 2, 0, 16, 2, 9), True),      # end of turn (a different id than eos), no length limit
    ((2, 3, 2, 7, 16, 2, 9), False),     # eos is ignored once a completion length is set ...
    ((9, 3, 2, 7, 16, 2, 9), False),     # ... and so is eot
    ((5, 15, 2, 0, 16, 2, 9), False),    # last position of the window
    ((5, 16, 2, 0, 16, 2, 9), True),     # position == seq_len
    ((5, 17, 2, 0, 16, 2, 9), True),     # beyond it
    ((5, 8, 2, 7, 16, 2, 9), False),     # 8 < 7 + 2
    ((5, 9, 2, 7, 16, 2, 9), True),      # 9 >= 7 + 2
    ((5, 10, 2, 7, 16, 2, 9), True),
    ((5, 6, 0, 7, 16, 2, 9), False),     # no prompt: the limit is the completion length alone
    ((5, 7, 0, 7, 16, 2, 9), True),
    ((5, 0, 0, 0, 16, 2, 9), False),     # a length of 0 means "no limit", not "finished at once"
    ((2, 16, 2, 7, 16, 2, 9), True),     # out of the window wins although eos is ignored
    ((5, 15, 10, 7, 16, 2, 9), False),   # 15 < 17 and 15 < 16
    ((0, 0, 0, 0, 1, 2, 9), False),      # a window of one position: position 0 is inside
    ((0, 1, 0, 0, 1, 2, 9), True),
    ((9, 3, 2, 0, 16, 2, 2), False),     # token 9 is no end token when eot == eos == 2 (the Llama2 configs)
]


def test_check_finished_hand_derived_cases():
    for (token, pos, plen, mcl, seq, eos, eot), want in CHECK_FINISHED_CASES:
        assert O.check_finished(token, pos, plen, mcl, seq, token_eos=eos, token_eot=eot) == want, (token, pos, plen, mcl, seq, eos, eot)


def test_temperature_codec():
    for t in [0.0, 0.1, 0.5, 0.999, 1.0]:
        e = O.encode_temperature(t)
        assert e == int(np.float32(t) * np.float32(255.0))      # truncation, not rounding
        assert abs(O.decode_temperature(e) - e / 255.0) < 1e-7
    assert O.encode_temperature(0.5) == 127
