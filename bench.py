#!/usr/bin/env python3
"""Benchmark of the per-stage Llama2 KV-cache path on one MI355X.

One "step" is one pass of the hot path over one batch: the C++ stage driver's forward() for a
pipeline stage of 10 layers of the Llama2-70B GQA shape (pre-attention, KV append, RoPE, fused
decode attention, post-attention for every layer) with decode batch 64 and every context
pre-filled so that the current token attends 4096 keys.  Inputs are synthetic (weights N(0,0.02),
K/V rows N(0,1), activations N(0,1), all seeded) and resident in HBM before the timed region.

Prints ONE JSON line:
  value        decode-attention algorithmic bytes / time of the attention op (split-K kernel + merge)
  roofline     the dominant kernel (split-K attention) against the 8 TB/s HBM peak, from HIP events
               recorded on the launch stream around every attention launch of K stage steps
  stage_*      whole stage step: tokens/s and the fraction of the bandwidth roofline, timed over K
               steps with no event between the kernels (ms_per_step); the K steps that carry the
               events run right after them and are reported as ms_per_step_with_attn_events
  cpu_baseline the CPU oracle (a port of the reference's fp32 OpenMP path) timed on a bounded sample
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch of the dominant kernel, from the FETCH_SIZE / WRITE_SIZE counter passes
# summarised in profiles/attn_decode_mfma_llama2-70b-gqa-b64-ctx4096_hbm_counters.md (each counter
# scaled by what it reads for a 1 GiB copy).  Only valid for the workload it was measured on.
MEASURED_TRAFFIC = {"llama2-70b-gqa-b64-ctx4096": 1086915785}

# the decode configurations that fit one GPU as a single stage (the first is the headline)
WORKLOADS = {
    # name: (stage config, first layer, hosted layers, batch, keys attended, description)
    "llama2-70b-gqa-b64-ctx4096": ("llama2-70b-4k", 10, 10, 64, 4096,
                                   "Llama2-70B GQA shape, one stage of 10 layers, fp16, decode batch 64, 4096 keys per context"),
    "llama2-7b-b32-ctx1024": ("llama2-7b", 8, 8, 32, 1024,
                              "Llama2-7B MHA shape, one stage of 8 layers, fp16, decode batch 32, 1024 keys per context"),
}
SHAPES = {
    "llama2-70b-4k": dict(dim=8192, n_heads=64, n_kv_heads=8, hidden_dim=28672, seq_len=4096, n_layers=80),
    "llama2-7b": dict(dim=4096, n_heads=32, n_kv_heads=32, hidden_dim=11008, seq_len=2048, n_layers=32),
    "llama2-13b-4k": dict(dim=5120, n_heads=40, n_kv_heads=40, hidden_dim=13824, seq_len=4096, n_layers=40),
}
# the prefill-heavy and the slot-churn configuration: not the headline, different step definitions
OTHER_WORKLOADS = {
    "llama2-13b-prefill-8x2048": "Llama2-13B MHA shape (seq 4096), one stage of 10 layers, fp16: batched prefill of 8 prompts x 2048 "
                                 "tokens per step, then 64 decode steps",
    "llama2-70b-churn-256": "Llama2-70B GQA shape, one stage of 10 layers, fp16: 256 context slots with lengths U[16,4096]; every "
                            "step decodes all slots, then 10 % of them finish and are refilled in place with 128-token prefills",
}
MFMA_PEAK_TFLOPS = 2500.0


def attention_bytes(shape, batch, keys, elem=2):
    """Algorithmic bytes of one layer's decode attention: every cached K and V element once, plus
    q read, output write and the appended row."""
    kv_dim = shape["dim"] // (shape["n_heads"] // shape["n_kv_heads"])
    return batch * keys * 2 * kv_dim * elem + batch * (2 * shape["dim"] + 2 * kv_dim) * elem


def layer_weight_bytes(shape, elem=2):
    d, h = shape["dim"], shape["hidden_dim"]
    kv_dim = d // (shape["n_heads"] // shape["n_kv_heads"])
    return (2 * d + 2 * d * d + 2 * d * kv_dim + 3 * d * h) * elem


def calibration_copy(n_bytes):
    """A plain device-to-device copy of known size, so that hardware byte counters read under a
    profiler can be scaled (the copy reads n_bytes and writes n_bytes)."""
    from glinthawk_amd import _lib, ops

    L = _lib.lib()
    src, dst = C.c_void_p(), C.c_void_p()
    _lib.check(L.gh_malloc(C.byref(src), n_bytes))
    _lib.check(L.gh_malloc(C.byref(dst), n_bytes))
    _lib.check(L.gh_memset_zero(src, n_bytes, None))
    for _ in range(3):
        _lib.check(L.gh_memcpy(dst, src, n_bytes, _lib.GH_D2D, 0, None))
    ops.sync()
    _lib.check(L.gh_free(src))
    _lib.check(L.gh_free(dst))


def gpu_bench(workload, steps, warmup):
    import numpy as np
    import torch

    from glinthawk_amd import _lib, ops, stage as S

    cfg_name, first, n_hosted, batch, keys, _ = WORKLOADS[workload]
    shape = SHAPES[cfg_name]
    pos = keys - 1
    ops.init(0)
    L = _lib.lib()

    st = S.Stage(cfg_name, "f16", first, n_hosted, batch, batch, fused=True, seed=4, weight_std=0.02)
    st.new_state(batch, next_layer=first)
    for i in range(batch):
        st.set_prompt(i, 1000 + i, 1, pos)
    assert st.acquire_contexts()
    # pre-fill: every slot gets N(0,1) rows for every hosted layer
    kv_dim = shape["dim"] // (shape["n_heads"] // shape["n_kv_heads"])
    layer_elems = shape["seq_len"] * 2 * kv_dim
    for i in range(batch):
        for l in range(first, first + n_hosted):
            _lib.check(L.gh_fill_normal(st.context_layer_ptr(i, l), layer_elems, 0.0, 1.0, 77 + i * 131 + l, _lib.GH_F16, None))
    ops.sync()

    rng = np.random.default_rng(0)
    acts = rng.standard_normal((batch, shape["dim"])).astype(np.float16)

    def one_step():
        st.set_next(first)
        st.activations(allocate=True)[:] = acts.reshape(-1)
        ok = st.forward()
        assert ok

    for _ in range(warmup):
        one_step()
    ops.sync()
    torch.cuda.synchronize()
    # pass 1: the stage step as it runs in production, nothing recorded between its kernels
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    ops.sync()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    # pass 2: the same steps with HIP events around every attention launch (an event record holds
    # the next kernel back by a few microseconds, so this pass is not the one the step is timed on)
    L.gh_attn_timing_enable(1)
    L.gh_attn_timing_reset()
    t2 = time.perf_counter()
    for _ in range(steps):
        one_step()
    ops.sync()
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    k_ms, m_ms, n = C.c_double(0), C.c_double(0), C.c_uint64(0)
    _lib.check(L.gh_attn_timing_read(C.byref(k_ms), C.byref(m_ms), C.byref(n)))
    L.gh_attn_timing_enable(0)

    out = st.activations().astype(np.float32)
    assert np.all(np.isfinite(out)), "stage output is not finite"

    # what a plain device-to-device copy reaches on this box (bytes read + bytes written per second):
    # the practical ceiling beside the published peak
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").zero_()
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    copy_gbps = 10 * 2 * src.numel() / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst

    ms_per_step = (t1 - t0) * 1e3 / steps
    launches = max(1, n.value)
    kernel_ms = k_ms.value / launches
    merge_ms = m_ms.value / launches
    a_bytes = attention_bytes(shape, batch, keys)
    stage_bytes = n_hosted * (a_bytes + layer_weight_bytes(shape))
    res = dict(
        ms_per_step=ms_per_step,
        ms_per_step_with_events=(t3 - t2) * 1e3 / steps,
        attn_kernel_ms=kernel_ms,
        attn_merge_ms=merge_ms,
        attn_launches=int(n.value),
        attn_bytes=a_bytes,
        stage_bytes=stage_bytes,
        batch=batch,
        device=ops.device_name(),
        copy_gbps=copy_gbps,
    )
    st.close()
    return res


def layer_matmul_flops(shape, tokens):
    d, h = shape["dim"], shape["hidden_dim"]
    kv_dim = d // (shape["n_heads"] // shape["n_kv_heads"])
    return 2 * tokens * (2 * d * d + 2 * d * kv_dim + 3 * d * h)


def prefill_bench(steps, warmup):
    """The prefill-heavy configuration.  One step = one batched prefill of 8 x 2048 prompt tokens through 10 layers
    (activations in and out over the boundary, like forward()); afterwards 64 decode steps on the same contexts."""
    import numpy as np

    from glinthawk_amd import ops, stage as S

    name, first, n_hosted, batch, T = "llama2-13b-4k", 10, 10, 8, 2048
    shape = SHAPES[name]
    ops.init(0)
    st = S.Stage(name, "f16", first, n_hosted, batch, batch, seed=3)
    rng = np.random.default_rng(3)
    # the boundary's host buffers, page-locked like the states' own buffers
    x = ops.pinned_empty((batch * T, shape["dim"]), np.float16)
    x[:] = rng.standard_normal(x.shape).astype(np.float16)
    y = ops.pinned_empty((batch * T, shape["dim"]), np.float16)
    ids = [100 + i for i in range(batch)]

    def one_step():
        res = st.prefill(ids, [0] * batch, T, first, activations=x, out=y)
        assert res is not None
        return res[0]

    for _ in range(warmup):
        one_step()
    ops.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = one_step()
    ops.sync()
    t1 = time.perf_counter()
    assert np.isfinite(out.astype(np.float32)).all()
    ms = (t1 - t0) * 1e3 / steps
    decode_steps = 64
    acts = x[:batch].copy()
    t0 = time.perf_counter()
    for k in range(decode_steps):
        st.new_state(batch, next_layer=first)
        for i in range(batch):
            st.set_prompt(i, ids[i], 1, T + k)
        st.activations(allocate=True)[:] = acts.reshape(-1)
        assert st.forward()
    ops.sync()
    t1 = time.perf_counter()
    decode_ms = (t1 - t0) * 1e3 / decode_steps
    flops = n_hosted * (layer_matmul_flops(shape, batch * T) + batch * 4 * shape["dim"] * T * (T + 1) // 2)
    dev = ops.device_name()
    st.close()
    return {
        "metric": "prefill prompt tokens/s (+ decode ms/step), Llama2-13B shape, 8 x 2048 tokens, 10 layers",
        "value": round(batch * T / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama2-13b-prefill-8x2048", "description": OTHER_WORKLOADS["llama2-13b-prefill-8x2048"], "device": dev},
        "decode_ms_per_step": round(decode_ms, 3), "decode_tokens_per_s": round(batch / (decode_ms * 1e-3), 1),
        "roofline": {"bound": "mfma", "achieved": round(flops / (ms * 1e-3) / 1e12, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "whole prefill pass incl. host transfers (projection GEMMs + causal attention flops / step time)",
                     "algorithmic_flops_per_step": flops},
        "cpu_baseline": None,
    }


def churn_bench(steps, warmup):
    """The slot-churn configuration.  One step = decode of all 256 slots (ragged lengths), then the slots drawn
    to finish (10 %, seeded) restart in place: a 128-token batched prefill into the same slot."""
    import numpy as np

    from glinthawk_amd import _lib, ops, stage as S

    name, first, n_hosted, slots, refill = "llama2-70b-4k", 10, 10, 256, 128
    shape = SHAPES[name]
    ops.init(0)
    L = _lib.lib()
    st = S.Stage(name, "f16", first, n_hosted, slots, slots, seed=5)
    rng = np.random.default_rng(5)
    pos = rng.integers(16, 4096, slots)
    ids = [1000 + i for i in range(slots)]
    st.new_state(slots, next_layer=first)
    for i in range(slots):
        st.set_prompt(i, ids[i], 1, int(pos[i]))
    assert st.acquire_contexts()
    kv_dim = shape["dim"] // (shape["n_heads"] // shape["n_kv_heads"])
    for i in range(slots):
        for l in range(first, first + n_hosted):
            _lib.check(L.gh_fill_normal(st.context_layer_ptr(i, l), shape["seq_len"] * 2 * kv_dim, 0.0, 1.0, 7 + i * 131 + l, _lib.GH_F16, None))
    slot_of = [st.context_slot(i) for i in range(slots)]
    acts = rng.standard_normal((slots, shape["dim"])).astype(np.float16)
    prompt = ops.pinned_empty((slots * refill, shape["dim"]), np.float16)
    prompt[:] = rng.standard_normal(prompt.shape).astype(np.float16)
    decoded = prefilled = restarts = 0
    keys_read = 0
    t_decode = t_prefill = 0.0

    def one_step(count):
        nonlocal decoded, prefilled, restarts, keys_read, t_decode, t_prefill
        t0 = time.perf_counter()
        st.new_state(slots, next_layer=first)
        for i in range(slots):
            st.set_prompt(i, ids[i], 1, int(pos[i]))
        st.activations(allocate=True)[:] = acts.reshape(-1)
        assert st.forward()
        t1 = time.perf_counter()
        assert [st.context_slot(i) for i in (0, slots // 2, slots - 1)] == [slot_of[0], slot_of[slots // 2], slot_of[slots - 1]]
        if count:
            decoded += slots
            keys_read += int((pos + 1).sum())
            t_decode += t1 - t0
        pos[:] = pos + 1
        done = (rng.random(slots) < 0.10) | (pos >= shape["seq_len"] - 1)
        gone = np.nonzero(done)[0]
        if len(gone):
            t0 = time.perf_counter()
            res = st.prefill([ids[i] for i in gone], [0] * len(gone), refill, first, activations=prompt[:len(gone) * refill],
                             want_activations=False)
            assert res is not None
            st.sync()
            t1 = time.perf_counter()
            pos[gone] = refill
            if count:
                prefilled += len(gone) * refill
                restarts += len(gone)
                t_prefill += t1 - t0

    for _ in range(warmup):
        one_step(False)
    ops.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step(True)
    ops.sync()
    t1 = time.perf_counter()
    counts = st.slot_counts()
    assert counts == dict(free=0, allocated=slots, total=slots), counts
    ms = (t1 - t0) * 1e3 / steps
    dev = ops.device_name()
    st.close()
    kv_bytes = keys_read * 2 * kv_dim * 2 * n_hosted
    return {
        "metric": "tokens/s (decode + refill prefill), ragged slot churn, Llama2-70B GQA shape, 256 slots, 10 layers",
        "value": round((decoded + prefilled) / (t1 - t0), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama2-70b-churn-256", "description": OTHER_WORKLOADS["llama2-70b-churn-256"], "device": dev},
        "decode_tokens_per_s": round(decoded / t_decode, 1), "decode_ms_per_step": round(t_decode * 1e3 / steps, 3),
        "prefill_tokens_per_s": round(prefilled / max(t_prefill, 1e-9), 1), "prefill_ms_per_step": round(t_prefill * 1e3 / steps, 3),
        "restarts": restarts, "mean_keys_per_slot": round(keys_read / max(decoded, 1), 1),
        "roofline": {"bound": "hbm", "achieved": round((kv_bytes + steps * n_hosted * layer_weight_bytes(shape)) / t_decode / 1e9, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round((kv_bytes + steps * n_hosted * layer_weight_bytes(shape)) / t_decode / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": None, "kernel": "whole decode step (cached K/V read once + weights once) / decode time"},
        "cpu_baseline": None,
    }


def cpu_baseline(workload):
    """The oracle (port of the reference's fp32 amd64/OpenMP path) on ONE layer of the workload,
    fp32 weights and fp32 K/V like the reference's CPU build, median of 3 after one warm-up; the
    stage figure scales that layer time by the number of hosted layers."""
    import numpy as np

    import oracle as O

    cfg_name, first, n_hosted, batch, keys, _ = WORKLOADS[workload]
    s = SHAPES[cfg_name]
    cfg = O.Config(dim=s["dim"], n_layers=s["n_layers"], n_heads=s["n_heads"], n_kv_heads=s["n_kv_heads"],
                   hidden_dim=s["hidden_dim"], seq_len=s["seq_len"])
    rng = np.random.default_rng(1)
    block = rng.standard_normal(1 << 22).astype(np.float32)

    def tiled(shape, scale):
        n = int(np.prod(shape))
        reps = (n + block.size - 1) // block.size
        return (np.tile(block, reps)[:n] * np.float32(scale)).reshape(shape)

    w = {
        "rms_att_weight": tiled((cfg.dim,), 0.02), "wq": tiled((cfg.dim, cfg.dim), 0.02),
        "wkv": tiled((2 * cfg.kv_dim, cfg.dim), 0.02), "wo": tiled((cfg.dim, cfg.dim), 0.02),
        "rms_ffn_weight": tiled((cfg.dim,), 0.02), "w1": tiled((cfg.hidden_dim, cfg.dim), 0.02),
        "w2": tiled((cfg.dim, cfg.hidden_dim), 0.02), "w3": tiled((cfg.hidden_dim, cfg.dim), 0.02),
    }
    re, im = O.rope_tables(cfg.seq_len, cfg.head_size)
    cache = tiled((batch, cfg.seq_len, 2 * cfg.kv_dim), 1.0)
    layers = [cache[i] for i in range(batch)]
    pos = [keys - 1] * batch
    scratch = {}
    att_times, layer_times = [], []
    for rep in range(4):
        x = tiled((batch, cfg.dim), 1.0).copy()
        t0 = time.perf_counter()
        scratch = O.layer_forward(cfg, w, re, im, x, layers, pos, scratch)
        t1 = time.perf_counter()
        q = scratch["q"].copy()
        O.attention_ops(cfg, pos, re, im, q, layers, att=scratch["att"])
        t2 = time.perf_counter()
        if rep:
            layer_times.append(t1 - t0)
            att_times.append(t2 - t1)
    layer_s = float(np.median(layer_times))
    att_s = float(np.median(att_times))
    a_bytes32 = attention_bytes(s, batch, keys, elem=4)
    return {
        "value": batch / (layer_s * n_hosted),
        "unit": "tokens/s",
        "cores": O.num_threads(),
        "kind": "port",
        "sample": f"1 of {n_hosted} layers (B={batch}, {keys} keys, fp32 weights and K/V as in the reference's CPU build), "
                  f"median of 3 after 1 warm-up; layer time {layer_s * 1e3:.0f} ms scaled x{n_hosted}",
        "attn_GBps": a_bytes32 / att_s / 1e9,
        "attn_ms_per_layer": att_s * 1e3,
        "layer_ms": layer_s * 1e3,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama2-70b-gqa-b64-ctx4096", choices=sorted(WORKLOADS) + sorted(OTHER_WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--attn-variant", default="auto", choices=["auto", "generic", "valu", "mfma"],
                    help="decode attention kernel the stage uses (measurement of the alternatives; auto = the library's choice)")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run a plain D2D copy of this many MiB (reference point for profiler byte counters)")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build runs one pipeline stage on ONE GPU; --gpus must be 1 "
              "(the path shards by context, slot -> GPU, with no collective; only the one-GPU share is built)", file=sys.stderr)
        sys.exit(2)

    if args.calibration_copy_mib > 0:
        from glinthawk_amd import ops
        ops.init(0)
        calibration_copy(args.calibration_copy_mib << 20)
    if args.attn_variant != "auto":
        from glinthawk_amd import _lib, ops
        ops.init(0)
        _lib.check(_lib.lib().gh_attn_set_auto_variant({"generic": 1, "valu": 2, "mfma": 3}[args.attn_variant]))
    if args.workload == "llama2-13b-prefill-8x2048":
        print(json.dumps(prefill_bench(args.steps, args.warmup)))
        return
    if args.workload == "llama2-70b-churn-256":
        print(json.dumps(churn_bench(args.steps, args.warmup)))
        return
    g = gpu_bench(args.workload, args.steps, args.warmup)
    cfg_name, first, n_hosted, batch, keys, desc = WORKLOADS[args.workload]

    attn_op_ms = g["attn_kernel_ms"] + g["attn_merge_ms"]
    value = g["attn_bytes"] / (attn_op_ms * 1e-3) / 1e9
    achieved = g["attn_bytes"] / (g["attn_kernel_ms"] * 1e-3) / 1e9
    tokens_per_s = batch / (g["ms_per_step"] * 1e-3)
    stage_roofline_ms = g["stage_bytes"] / (HBM_PEAK_GBPS * 1e9) * 1e3

    line = {
        "metric": "decode attn HBM GB/s (% of peak) + stage tokens/s, Llama2-70B GQA, B=64, ctx 4096",
        "value": round(value, 1),
        "unit": "GB/s",
        "pct_of_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "copy_ceiling_gbps": round(g["copy_gbps"], 1),
        "pct_of_copy_ceiling": round(100 * value / g["copy_gbps"], 2),
        "stage_tokens_per_s": round(tokens_per_s, 1),
        "stage_roofline_frac": round(stage_roofline_ms / g["ms_per_step"], 4),
        "stage_bytes_per_step": g["stage_bytes"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(g["ms_per_step"], 4),
        "ms_per_step_with_attn_events": round(g["ms_per_step_with_events"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": desc, "stage_config": cfg_name, "first_layer": first,
                   "hosted_layers": n_hosted, "batch": batch, "keys_per_context": keys, "device": g["device"],
                   "attn_variant": args.attn_variant},
        "attn_op_ms": round(attn_op_ms, 5),
        "attn_kernel_ms": round(g["attn_kernel_ms"], 5),
        "attn_merge_ms": round(g["attn_merge_ms"], 5),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC.get(args.workload),
                     "kernel": "attn_decode (split-K fused decode attention)", "launches_timed": g["attn_launches"],
                     "algorithmic_bytes_per_launch": g["attn_bytes"]},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.workload)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
