"""The C++ host layer's integer bookkeeping against the oracle, without a GPU: slot manager
(bit-exact slot indices on random op sequences), paged-context block accounting, KV addressing."""
import numpy as np

import oracle as O
from glinthawk_amd import stage as S

CFG70 = O.Config(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096)


def test_slot_manager_matches_oracle_on_random_sequences():
    rng = np.random.default_rng(17)
    for trial in range(25):
        cap = int(rng.integers(1, 10))
        ours, ref = S.BookManager(cap), O.ContextManager(cap)
        for _ in range(80):
            op = rng.random()
            if op < 0.7:
                bs = int(rng.integers(1, 8))
                active = rng.random(bs) < 0.8
                ids = rng.integers(0, 14, bs).astype(np.uint32)
                start = int(rng.integers(0, bs))
                end = int(rng.integers(start, bs + 1))
                assert ours.get_contexts(active, ids, start, end) == ref.get_contexts(active, ids, start, end)
            elif op < 0.85:
                cid = int(rng.integers(0, 14))
                assert ours.get_context(cid) == ref.get_context(cid)
            else:
                cid = int(rng.integers(0, 14))
                assert ours.release(cid) == ref.release(cid)
            assert (ours.free(), ours.allocated()) == (ref.free(), ref.allocated())


def test_slot_manager_churn_like_config5():
    # 256 slots, 10% of rows finish each step and are refilled under the same context id: the
    # mapping never changes and no slot is ever taken from the free list after the first step
    rng = np.random.default_rng(5)
    man, ref = S.BookManager(256), O.ContextManager(256)
    ids = np.arange(1000, 1256, dtype=np.uint32)
    first = man.get_contexts(np.ones(256, bool), ids)
    assert first == ref.get_contexts(np.ones(256, bool), ids) == list(range(256))
    for step in range(50):
        active = rng.random(256) > 0.1            # discarded rows are inactive for a step ...
        got = man.get_contexts(active, ids)
        assert got == ref.get_contexts(active, ids)
        assert all(g == (i if a else -1) for i, (g, a) in enumerate(zip(got, active)))
        assert man.free() == 0 and man.allocated() == 256
    assert man.get_contexts([1], [7]) is None     # a new id cannot be served: all slots are owned


def test_paged_context_block_accounting():
    n_hosted = 3
    ctx = S.BookPagedContext(n_hosted)
    allocated = np.zeros(CFG70.n_layers, np.uint64)
    rng = np.random.default_rng(9)
    pos, blocks, clears = 0, 0, 0
    for step in range(4000):
        layer = step % n_hosted
        if layer == 0:
            pos = 0 if (step == 0 or rng.random() < 0.003) else min(pos + 1, CFG70.seq_len - 1)
        can_release = pos == 0 and layer == 0
        n, cleared = O.dynctx_prepare(CFG70, 2, allocated, layer, pos, can_release, commit_all=True)
        blocks += n
        clears += int(cleared)
        got_alloc, got_blocks, got_clears = ctx.prepare(layer, pos, can_release)
        assert (got_alloc, got_blocks, got_clears) == (int(allocated[layer]), blocks, clears)
    # a jump to a far position commits every missing block (superset of the reference's one block)
    ctx2 = S.BookPagedContext(1)
    assert ctx2.prepare(0, 2000, False) == (4 * 2 * 2 ** 20, 4, 0)
    assert ctx2.prepare(0, 0, True) == (2 * 2 ** 20, 5, 1)


def test_addressing_matches_oracle():
    rng = np.random.default_rng(3)
    hosted = np.zeros(80, np.uint8)
    hosted[[2, 3, 7, 40, 79]] = 1
    for _ in range(300):
        layer = int(rng.integers(0, 80))
        pos = int(rng.integers(0, 4096))
        head = int(rng.integers(0, 8))
        assert S.book_head_offset(hosted, layer, pos, head, False) == O.ctx_key_head_offset(CFG70, hosted, layer, pos, head)
        assert S.book_head_offset(hosted, layer, pos, head, True) == O.ctx_value_head_offset(CFG70, hosted, layer, pos, head)
    assert S.book_head_offset(hosted, 3, 0, 0, False) == 4096 * 2048      # second hosted layer starts one layer span in
    assert S.book_head_offset(hosted, 5, 0, 0, False) is None
