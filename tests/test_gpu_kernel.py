"""The compute kernel around the real model: states pushed as wire bytes come back, in order, with
the same tokens a synchronously driven stage produces from the same weights."""
import numpy as np
import pytest

from glinthawk_amd import stage as S, wire
from glinthawk_amd.kernel import ComputeKernel

pytestmark = pytest.mark.gpu


def test_kernel_equals_synchronous_stage():
    name, dtype, batch, dim, kv_dim = "test-gqa4", "f16", 4, 1024, 256
    n_layers = 3
    kernel = ComputeKernel(name, dtype, 0, n_layers, batch, 2 * batch, with_cls=True, seed=17)
    stage = S.Stage(name, dtype, 0, n_layers, batch, 2 * batch, with_cls=True, seed=17)      # same seed, same weights
    meta = dict(dtype=wire.DTYPE_CODE[dtype], next_layer=0, next_stage=S.STAGE_PRE, route_id=3)
    # two interleaved "conversations" (disjoint context ids) pushed back to back, several rounds deep
    convs = {0: dict(cids=[10, 11, 12, 13], tokens=[1, 2, 3, 4]), 1: dict(cids=[20, 21, 22, 23], tokens=[50, 60, 70, 80])}
    expected = {0: [], 1: []}
    rounds = 4
    for c, conv in convs.items():
        toks = list(conv["tokens"])
        for pos in range(rounds):
            stage.new_state(batch)
            for i in range(batch):
                stage.set_prompt(i, conv["cids"][i], toks[i], pos, 0.0, 64, 0)
            assert stage.forward()
            toks = [stage.row(i)["token"] for i in range(batch)]
            expected[c].append(list(toks))
    toks = {c: list(conv["tokens"]) for c, conv in convs.items()}
    for pos in range(rounds):
        for c, conv in convs.items():
            p = wire.new_prompts(batch)
            p["active"], p["kv_tier"] = 1, 0
            p["context_id"], p["token"], p["token_pos"] = conv["cids"], toks[c], pos
            p["prompt_length"] = 64
            kernel.push(wire.pack_state(dict(meta, id=100 * c + pos), p))
        got = []
        while len(got) < 2:
            assert kernel.wait(30.0)
            kernel.read_event()
            while (raw := kernel.pop()) is not None:
                got.append(raw)
        for c, raw in zip(convs, got):                          # comes back in push order
            m, p, *_ = wire.unpack_state(raw, dim, kv_dim)
            assert int(m["id"]) == 100 * c + pos and int(m["route_id"]) == 3
            assert [int(t) for t in p["token"]] == expected[c][pos]
            assert [int(t) for t in p["token_pos"]] == [pos + 1] * batch
            toks[c] = [int(t) for t in p["token"]]
    assert kernel.slot_counts() == dict(free=0, allocated=8, total=8)
    kernel.close()
    stage.close()
