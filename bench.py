#!/usr/bin/env python3
"""Benchmark of the per-stage Llama2 KV-cache path on one MI355X.

One "step" is one pass of the hot path over one batch.  The headline workload is the C++ stage
driver's forward() for a pipeline stage of 10 layers of the Llama2-70B GQA shape (pre-attention, KV
append, RoPE, fused decode attention, post-attention for every layer) with decode batch 64 and every
context pre-filled so that the current token attends 4096 keys.  Inputs are synthetic (weights
N(0,0.02), K/V rows N(0,1), activations N(0,1), all seeded) and resident in HBM before the timed region.

Prints ONE JSON line:
  value        decode-attention algorithmic bytes / time of the attention op (split-K kernel + merge back to back,
               one event in front of the pair and one behind, in K steps of their own)
  roofline     the dominant kernel (split-K attention) against the 8 TB/s HBM peak, from HIP events
               recorded on the launch stream around every attention launch of K stage steps
  stage_*      whole stage step: tokens/s and the fraction of the bandwidth roofline, timed over K
               steps with no event between the kernels (ms_per_step); the K steps that carry the
               events run right after them and are reported as ms_per_step_with_attn_events
  *_resident   the same step between two events, after its activations and tables are queued and before the copy
               back: what the stage costs with its inputs resident in HBM (ms_per_step goes through the host
               state buffers on both sides, as the reference's forward() does)
  cpu_baseline the CPU oracle (a port of the reference's fp32 OpenMP path) timed on a bounded sample:
               one hosted layer on the very weights, cache rows and activations the GPU stage ran on
  concept_path the same stage driven through the reference's own op sequence only (unfused attention
               ops with a score buffer, separate projections, host-side tables staged per op)
  other        short runs of the other decode / prefill / churn configurations, each with its own
               roofline and CPU sample (leave out with --skip-others)
"""
from __future__ import annotations

import argparse
import ctypes as C
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0

# HBM bytes per launch of the dominant kernel come from hardware counters (FETCH_SIZE / WRITE_SIZE under
# rocprofv3, each scaled by what it reads for a plain copy); they cannot be read from inside this program.
# The summary of that measurement names the kernel source it was taken on by its SHA-256; the figure is
# reported only while that source is unchanged, otherwise `traffic` is null.
TRAFFIC_PROFILE = {
    "llama2-70b-gqa-b64-ctx4096": ("profiles/attn_decode_mfma_llama2-70b-gqa-b64-ctx4096_hbm_counters.md",
                                   ("glinthawk_amd/csrc/gh_attn_decode.hip", "glinthawk_amd/csrc/gh_attn_tiles.h")),
}


def gemm_route(calls_before=0):
    """Which kernels ran the products of many activation rows: the tile kernels of this library ("own", the default) or,
    when a row threshold was set (--library-rows, GLINT_LIBRARY_ROWS), the vendor's GEMM library from that many rows on;
    `vendor_products` counts the products the vendor library really ran since `calls_before` (it declines silently)."""
    from glinthawk_amd import _lib
    L = _lib.lib()
    rows = int(L.gh_gemm_library_rows())
    calls = int(L.gh_gemm_library_calls()) - calls_before
    return {"route": "vendor" if rows > 0 and calls > 0 else "own", "vendor_library_from_rows": rows or None, "vendor_products": calls}


def library_calls():
    from glinthawk_amd import _lib
    return int(_lib.lib().gh_gemm_library_calls())


def kernel_source_digest(sources):
    """sha256 over the kernel's source files, in the order given."""
    h = hashlib.sha256()
    for p in sources:
        h.update(open(os.path.join(ROOT, p), "rb").read())
    return h.hexdigest()

# the decode configurations that fit one GPU as a single stage (the first is the headline)
WORKLOADS = {
    # name: (stage config, first layer, hosted layers, batch, keys attended, description)
    "llama2-70b-gqa-b64-ctx4096": ("llama2-70b-4k", 10, 10, 64, 4096,
                                   "Llama2-70B GQA shape, one stage of 10 layers, fp16, decode batch 64, 4096 keys per context"),
    "llama2-7b-b32-ctx1024": ("llama2-7b", 8, 8, 32, 1024,
                              "Llama2-7B MHA shape, one stage of 8 layers, fp16, decode batch 32, 1024 keys per context"),
}
METRICS = {
    "llama2-70b-gqa-b64-ctx4096": "decode attn HBM GB/s (% of peak) + stage tokens/s, Llama2-70B GQA, B=64, ctx 4096",
    "llama2-7b-b32-ctx1024": "decode attn HBM GB/s (% of peak) + stage tokens/s, Llama2-7B MHA, B=32, ctx 1024",
    "llama2-13b-prefill-8x2048": "prefill prompt tokens/s (+ decode ms/step), Llama2-13B shape, 8 x 2048 tokens, 10 layers",
    "llama2-70b-churn-256": "tokens/s (decode + refill prefill), ragged slot churn, Llama2-70B GQA shape, 256 slots, 10 layers",
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
LAYER_TENSORS = ("rms_att_weight", "wq", "wkv", "wo", "rms_ffn_weight", "w1", "w2", "w3")


def kv_dim_of(shape):
    return shape["dim"] // (shape["n_heads"] // shape["n_kv_heads"])


def attention_bytes(shape, batch, keys, elem=2):
    """Algorithmic bytes of one layer's decode attention: every cached K and V element once, plus
    q read, output write and the appended row."""
    kv_dim = kv_dim_of(shape)
    return batch * keys * 2 * kv_dim * elem + batch * (2 * shape["dim"] + 2 * kv_dim) * elem


def layer_weight_bytes(shape, elem=2):
    d, h = shape["dim"], shape["hidden_dim"]
    return (2 * d + 2 * d * d + 2 * d * kv_dim_of(shape) + 3 * d * h) * elem


def layer_matmul_flops(shape, tokens):
    d, h = shape["dim"], shape["hidden_dim"]
    return 2 * tokens * (2 * d * d + 2 * d * kv_dim_of(shape) + 3 * d * h)


def measured_traffic(workload):
    """(bytes per launch or None, note): the counter figure of the committed profile summary, if it was taken on
    the kernel source as it is now."""
    if workload not in TRAFFIC_PROFILE:
        return None, "no counter profile for this workload"
    summary, sources = TRAFFIC_PROFILE[workload]
    summary = os.path.join(ROOT, summary)
    try:
        text = open(summary).read()
        digest = kernel_source_digest(sources)
    except OSError:
        return None, "counter profile summary not present"
    m_bytes = re.search(r"traffic_bytes_per_launch:\s*(\d+)", text)
    m_hash = re.search(r"kernel_source_sha256:\s*([0-9a-f]{64})", text)
    if not m_bytes or not m_hash:
        return None, "counter profile summary carries no figure"
    if m_hash.group(1) != digest:
        return None, "kernel source changed since the counters were read"
    return int(m_bytes.group(1)), os.path.relpath(summary, ROOT)


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


def download(ptr, n_elems, dtype):
    import numpy as np

    from glinthawk_amd import _lib
    out = np.empty(n_elems, dtype=dtype)
    _lib.check(_lib.lib().gh_memcpy(out.ctypes.data, ptr, out.nbytes, _lib.GH_D2H, 0, None), "gh_memcpy")
    return out


def layer_inputs_f32(st, shape, layer):
    """The weights of one hosted layer and the RoPE tables as the GPU stage holds them, as fp32 for the CPU path."""
    import numpy as np
    d, h, kv = shape["dim"], shape["hidden_dim"], kv_dim_of(shape)
    shapes = {"rms_att_weight": (d,), "wq": (d, d), "wkv": (2 * kv, d), "wo": (d, d), "rms_ffn_weight": (d,), "w1": (h, d), "w2": (d, h), "w3": (h, d)}
    w = {name: st.get_layer_tensor(layer, name).astype(np.float32).reshape(shapes[name]) for name in LAYER_TENSORS}
    hs = d // shape["n_heads"]
    re = st.get_base_tensor("freq_cis_real").astype(np.float32).reshape(shape["seq_len"], hs // 2)
    im = st.get_base_tensor("freq_cis_imag").astype(np.float32).reshape(shape["seq_len"], hs // 2)
    return w, re, im


def oracle_config(shape):
    import oracle as O
    return O.Config(dim=shape["dim"], n_layers=shape["n_layers"], n_heads=shape["n_heads"], n_kv_heads=shape["n_kv_heads"],
                    hidden_dim=shape["hidden_dim"], seq_len=shape["seq_len"])


def cpu_decode_layer(shape, w, re, im, layers, x, pos, reps=3):
    """Median seconds of the oracle's layer (and of its attention ops alone) over `reps` runs after one warm-up."""
    import numpy as np

    import oracle as O
    cfg = oracle_config(shape)
    scratch = {}
    layer_times, att_times = [], []
    for rep in range(reps + 1):
        xx = np.ascontiguousarray(x, dtype=np.float32).copy()
        t0 = time.perf_counter()
        scratch = O.layer_forward(cfg, w, re, im, xx, layers, pos, scratch)
        t1 = time.perf_counter()
        q = scratch["q"].copy()
        O.attention_ops(cfg, pos, re, im, q, layers, att=scratch["att"])
        t2 = time.perf_counter()
        if rep:
            layer_times.append(t1 - t0)
            att_times.append(t2 - t1)
    return float(np.median(layer_times)), float(np.median(att_times)), O.num_threads()


def decode_bench(workload, steps, warmup, fused=True, cpu=True, events=True, advance=False):
    """A decode workload: K stage steps timed plain, K more with events around the attention launches, a plain
    copy as the practical bandwidth ceiling, and (cpu) the oracle on the first hosted layer's own inputs."""
    import numpy as np
    import torch

    from glinthawk_amd import _lib, ops, stage as S

    cfg_name, first, n_hosted, batch, keys, _ = WORKLOADS[workload]
    shape = SHAPES[cfg_name]
    pos = keys - 1
    ops.init(0)
    L = _lib.lib()
    calls0 = library_calls()

    st = S.Stage(cfg_name, "f16", first, n_hosted, batch, batch, fused=fused, seed=4, weight_std=0.02)
    st.new_state(batch, next_layer=first)
    for i in range(batch):
        st.set_prompt(i, 1000 + i, 1, pos)
    assert st.acquire_contexts()
    # pre-fill: every slot gets N(0,1) rows for every hosted layer
    kv_dim = kv_dim_of(shape)
    layer_elems = shape["seq_len"] * 2 * kv_dim
    for i in range(batch):
        for l in range(first, first + n_hosted):
            _lib.check(L.gh_fill_normal(st.context_layer_ptr(i, l), layer_elems, 0.0, 1.0, 77 + i * 131 + l, _lib.GH_F16, None))
    ops.sync()

    rng = np.random.default_rng(0)
    acts = rng.standard_normal((batch, shape["dim"])).astype(np.float16)

    ids = [1000 + i for i in range(batch)]
    ones = np.ones(batch, np.uint32)

    def one_step(at=None):
        if at is None:
            st.set_next(first)
        else:                                   # the next token of every context: a new state at the next position
            st.new_state(batch, next_layer=first)
            st.set_prompts(ids, ones, np.full(batch, at, np.uint32))
        st.activations(allocate=True)[:] = acts.reshape(-1)
        ok = st.forward()
        assert ok

    for _ in range(warmup):
        one_step()
    ops.sync()
    torch.cuda.synchronize()
    # pass 1: the stage step as it runs in production, nothing recorded between its kernels
    t0 = time.perf_counter()
    for k in range(steps):
        one_step(pos + k if advance else None)
    ops.sync()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    res = dict(ms_per_step=(t1 - t0) * 1e3 / steps, batch=batch, device=ops.device_name())
    a_bytes = attention_bytes(shape, batch, keys)
    res.update(attn_bytes=a_bytes, stage_bytes=n_hosted * (a_bytes + layer_weight_bytes(shape)))
    if advance:                                 # keys grow by one per step: the bytes of the run are the sum over its steps
        res["stage_bytes"] = sum(n_hosted * (attention_bytes(shape, batch, keys + k) + layer_weight_bytes(shape)) for k in range(steps)) // steps
        res["gemm_route"] = gemm_route(calls0)
        st.close()
        return res
    if events and fused:
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
        launches = max(1, n.value)
        # waves per work-group when the splits of a context are added up inside the attention kernel's work-groups: then there is
        # no merge kernel, and what lies between the second and the third event is the events' own cost
        from glinthawk_amd import Shape
        join = ops.attn_decode_join_waves(batch, keys - 1, Shape(**{k: shape[k] for k in ("dim", "n_layers", "n_heads", "n_kv_heads", "hidden_dim", "seq_len")}))
        res.update(ms_per_step_with_events=(t3 - t2) * 1e3 / steps, attn_kernel_ms=k_ms.value / launches,
                   attn_merge_ms=None if join else m_ms.value / launches, attn_launches=int(n.value), attn_split_join=join)
        # the attention op as it runs in production, its two kernels back to back: one event in front of the pair, one behind
        L.gh_attn_timing_enable(2)
        L.gh_attn_timing_reset()
        for _ in range(steps):
            one_step()
        ops.sync()
        _lib.check(L.gh_attn_timing_read(C.byref(k_ms), C.byref(m_ms), C.byref(n)))
        L.gh_attn_timing_enable(0)
        res.update(attn_op_ms=k_ms.value / max(1, n.value))

    # pass 3: the same steps once more with two events per step, after the activations and tables are queued and before
    # the copy back: the stage step with its inputs resident in HBM, without the host boundary on either side
    st.time_device_spans(True)
    for _ in range(steps):
        one_step()
    span_ms, spans = st.device_spans()
    st.time_device_spans(False)
    res.update(ms_per_step_resident=span_ms / max(1, spans))
    out = st.activations().astype(np.float32)
    assert np.all(np.isfinite(out)), "stage output is not finite"

    if cpu:
        # the CPU path on the first hosted layer: the same weights, the same cache rows, the same activations
        w, re, im = layer_inputs_f32(st, shape, first)
        layers = [download(st.context_layer_ptr(i, first), layer_elems, np.float16).astype(np.float32).reshape(shape["seq_len"], 2 * kv_dim)
                  for i in range(batch)]
        layer_s, att_s, cores = cpu_decode_layer(shape, w, re, im, layers, acts, [pos] * batch)
        res["cpu_baseline"] = {
            "value": batch / (layer_s * n_hosted), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"1 of {n_hosted} layers (B={batch}, {keys} keys) on the weights, cache rows and activations of the GPU run's first "
                      f"hosted layer, held as fp32 like the reference's CPU build; median of 3 after 1 warm-up; layer time "
                      f"{layer_s * 1e3:.0f} ms scaled x{n_hosted}",
            "attn_GBps": attention_bytes(shape, batch, keys, elem=4) / att_s / 1e9,
            "attn_ms_per_layer": att_s * 1e3, "layer_ms": layer_s * 1e3,
        }
        del w, layers
    res["gemm_route"] = gemm_route(calls0)
    st.close()
    return res


def copy_ceiling_gbps():
    """What a plain device-to-device copy reaches on this box (bytes read + bytes written per second): the
    practical ceiling beside the published peak."""
    import torch
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
    return 10 * 2 * src.numel() / (e0.elapsed_time(e1) * 1e-3) / 1e9


def decode_line(workload, steps, warmup, attn_variant="auto", cpu=True):
    """The JSON line of a decode workload."""
    g = decode_bench(workload, steps, warmup, cpu=cpu)
    cfg_name, first, n_hosted, batch, keys, desc = WORKLOADS[workload]
    copy_gbps = copy_ceiling_gbps()
    attn_op_ms = g["attn_op_ms"]
    value = g["attn_bytes"] / (attn_op_ms * 1e-3) / 1e9
    achieved = g["attn_bytes"] / (g["attn_kernel_ms"] * 1e-3) / 1e9
    tokens_per_s = batch / (g["ms_per_step"] * 1e-3)
    stage_roofline_ms = g["stage_bytes"] / (HBM_PEAK_GBPS * 1e9) * 1e3
    traffic, traffic_note = measured_traffic(workload)
    return {
        "metric": METRICS[workload],
        "value": round(value, 1),
        "unit": "GB/s",
        "pct_of_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "copy_ceiling_gbps": round(copy_gbps, 1),
        "pct_of_copy_ceiling": round(100 * value / copy_gbps, 2),
        "stage_tokens_per_s": round(tokens_per_s, 1),
        "stage_roofline_frac": round(stage_roofline_ms / g["ms_per_step"], 4),
        "stage_bytes_per_step": g["stage_bytes"],
        "ms_per_step_resident": round(g["ms_per_step_resident"], 4),
        "stage_tokens_per_s_resident": round(batch / (g["ms_per_step_resident"] * 1e-3), 1),
        "stage_roofline_frac_resident": round(stage_roofline_ms / g["ms_per_step_resident"], 4),
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(g["ms_per_step"], 4),
        "ms_per_step_with_attn_events": round(g["ms_per_step_with_events"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": workload, "description": desc, "stage_config": cfg_name, "first_layer": first,
                   "hosted_layers": n_hosted, "batch": batch, "keys_per_context": keys, "device": g["device"],
                   "attn_variant": attn_variant},
        "attn_op_ms": round(attn_op_ms, 5),
        "attn_kernel_ms": round(g["attn_kernel_ms"], 5),
        "attn_merge_ms": None if g["attn_merge_ms"] is None else round(g["attn_merge_ms"], 5),
        "attn_split_join_waves": g["attn_split_join"],
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_note,
                     "kernel": "attn_decode (split-K fused decode attention)", "launches_timed": g["attn_launches"],
                     "algorithmic_bytes_per_launch": g["attn_bytes"]},
        "cpu_baseline": g.get("cpu_baseline"),
        "gemm_route": g["gemm_route"],
    }


def concept_path(workload, steps, warmup):
    """The same stage driven only through the methods of the reference's operations interface, in the order its model
    driver issues them (models/llama2/model.hh:326-427): separate projections, copy_kv_cache, apply_rope,
    attention_0_gemm, attention_softmax, attention_2_gemm with the (batch, n_heads, seq_len) score buffer, and the
    host-side context tables staged by every op.  What an unmodified model driver would execute on this backend."""
    g = decode_bench(workload, steps, warmup, fused=False, cpu=False, events=False)
    return {"ms_per_step": round(g["ms_per_step"], 4), "stage_tokens_per_s": round(g["batch"] / (g["ms_per_step"] * 1e-3), 1),
            "stage_roofline_frac": round(g["stage_bytes"] / (HBM_PEAK_GBPS * 1e9) * 1e3 / g["ms_per_step"], 4),
            "gemm_route": g["gemm_route"],
            "note": "unfused attention ops + score buffer, separate projection / element-wise ops, per-op host tables"}


def prefill_bench(steps, warmup, cpu=True):
    """The prefill-heavy configuration.  One step = one batched prefill of 8 x 2048 prompt tokens through 10 layers
    (activations in and out over the boundary, like forward()); afterwards 64 decode steps on the same contexts."""
    import numpy as np

    from glinthawk_amd import ops, stage as S

    name, first, n_hosted, batch, T = "llama2-13b-4k", 10, 10, 8, 2048
    shape = SHAPES[name]
    ops.init(0)
    calls0 = library_calls()
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

    cpu_res = None
    if cpu:
        # The reference's CPU path feeds a prompt one token per forward (frontend/infer.cc:124-125): a step of all 8
        # prompts at prompt position p costs one batch-8 layer pass over p + 1 keys.  Sampled at three positions on the
        # first hosted layer, with the weights, the cache rows the GPU prefill wrote and the prompt's own input rows.
        kv_dim = kv_dim_of(shape)
        w, re, im = layer_inputs_f32(st, shape, first)
        layers = [download(st.context_layer_ptr(i, first), T * 2 * kv_dim, np.float16).astype(np.float32).reshape(T, 2 * kv_dim) for i in range(batch)]
        xin = x.reshape(batch, T, shape["dim"])
        times = []
        for p in (0, T // 2 - 1, T - 1):
            layer_s, _, cores = cpu_decode_layer(shape, w, re, im, layers, xin[:, p], [p] * batch, reps=2)
            times.append(layer_s)
        mean_s = float(np.mean(times))
        cpu_res = {"value": batch / (mean_s * n_hosted), "unit": "tokens/s", "cores": cores, "kind": "port",
                   "sample": f"token-by-token prompt processing as the reference does it: 1 of {n_hosted} layers, the 8 prompts at positions "
                             f"0, {T // 2 - 1} and {T - 1} (median of 2 after 1 warm-up each) on the GPU run's weights, cache rows and inputs held as "
                             f"fp32; mean layer pass {mean_s * 1e3:.0f} ms scaled x{n_hosted}"}
        del w, layers

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
        "metric": METRICS["llama2-13b-prefill-8x2048"],
        "value": round(batch * T / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama2-13b-prefill-8x2048", "description": OTHER_WORKLOADS["llama2-13b-prefill-8x2048"], "device": dev},
        "decode_ms_per_step": round(decode_ms, 3), "decode_tokens_per_s": round(batch / (decode_ms * 1e-3), 1),
        "roofline": {"bound": "mfma", "achieved": round(flops / (ms * 1e-3) / 1e12, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "whole prefill pass incl. host transfers (projection GEMMs + causal attention flops / step time)",
                     "algorithmic_flops_per_step": flops},
        "cpu_baseline": cpu_res,
        "gemm_route": gemm_route(calls0),
    }


def churn_bench(steps, warmup, cpu=True):
    """The slot-churn configuration.  One step = decode of all 256 slots (ragged lengths), then the slots drawn
    to finish (10 %, seeded) restart in place: a 128-token batched prefill into the same slot.  The timed steps
    start from the configuration's own length distribution U[16, 4096): the warm-up steps run first and the
    positions are then set back (every row of every slot holds N(0,1) values, so any length is valid)."""
    import numpy as np

    from glinthawk_amd import _lib, ops, stage as S

    name, first, n_hosted, slots, refill = "llama2-70b-4k", 10, 10, 256, 128
    shape = SHAPES[name]
    ops.init(0)
    L = _lib.lib()
    calls0 = library_calls()
    st = S.Stage(name, "f16", first, n_hosted, slots, slots, seed=5)
    rng = np.random.default_rng(5)
    start_pos = rng.integers(16, 4096, slots)
    pos = start_pos.copy()
    ids = [1000 + i for i in range(slots)]
    ones = np.ones(slots, np.uint32)
    st.new_state(slots, next_layer=first)
    for i in range(slots):
        st.set_prompt(i, ids[i], 1, int(pos[i]))
    assert st.acquire_contexts()
    kv_dim = kv_dim_of(shape)
    for i in range(slots):
        for l in range(first, first + n_hosted):
            _lib.check(L.gh_fill_normal(st.context_layer_ptr(i, l), shape["seq_len"] * 2 * kv_dim, 0.0, 1.0, 7 + i * 131 + l, _lib.GH_F16, None))
    slot_of = [st.context_slot(i) for i in range(slots)]
    first_layer_rows = [st.context_layer_ptr(i, first) for i in range(slots)]       # slots never move
    acts = rng.standard_normal((slots, shape["dim"])).astype(np.float16)
    prompt = ops.pinned_empty((slots * refill, shape["dim"]), np.float16)
    prompt[:] = rng.standard_normal(prompt.shape).astype(np.float16)
    decoded = prefilled = restarts = 0
    keys_read = 0
    t_decode = t_prefill = 0.0
    per_step = []

    def one_step(count):
        nonlocal decoded, prefilled, restarts, keys_read, t_decode, t_prefill
        t0 = time.perf_counter()
        st.new_state(slots, next_layer=first)
        st.set_prompts(ids, ones, pos)
        st.activations(allocate=True)[:] = acts.reshape(-1)
        assert st.forward()
        t1 = time.perf_counter()
        assert [st.context_slot(i) for i in (0, slots // 2, slots - 1)] == [slot_of[0], slot_of[slots // 2], slot_of[slots - 1]]
        if count:
            decoded += slots
            keys_read += int((pos + 1).sum())
            t_decode += t1 - t0
            per_step.append((float((pos + 1).mean()), (t1 - t0) * 1e3))
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
    pos[:] = start_pos
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step(True)
    ops.sync()
    t1 = time.perf_counter()
    counts = st.slot_counts()
    assert counts == dict(free=0, allocated=slots, total=slots), counts
    ms = (t1 - t0) * 1e3 / steps

    cpu_res = None
    if cpu:
        # one decode step of all 256 slots at the starting lengths on the first hosted layer (the refill prefills are not in the sample)
        w, re, im = layer_inputs_f32(st, shape, first)
        layers = [download(first_layer_rows[i], (int(start_pos[i]) + 1) * 2 * kv_dim, np.float16).astype(np.float32)
                  .reshape(int(start_pos[i]) + 1, 2 * kv_dim) for i in range(slots)]
        layer_s, _, cores = cpu_decode_layer(shape, w, re, im, layers, acts, [int(p) for p in start_pos], reps=2)
        cpu_res = {"value": slots / (layer_s * n_hosted), "unit": "tokens/s", "cores": cores, "kind": "port",
                   "sample": f"decode part only: 1 of {n_hosted} layers, all 256 slots at their starting lengths (mean {float((start_pos + 1).mean()):.0f} keys) on "
                             f"the GPU run's weights, cache rows and activations held as fp32; median of 2 after 1 warm-up; layer time "
                             f"{layer_s * 1e3:.0f} ms scaled x{n_hosted}"}
        del w, layers
    dev = ops.device_name()
    st.close()
    kv_bytes = keys_read * 2 * kv_dim * 2 * n_hosted
    decode_bytes = kv_bytes + steps * n_hosted * layer_weight_bytes(shape)
    return {
        "metric": METRICS["llama2-70b-churn-256"],
        "value": round((decoded + prefilled) / (t1 - t0), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama2-70b-churn-256", "description": OTHER_WORKLOADS["llama2-70b-churn-256"], "device": dev},
        "decode_tokens_per_s": round(decoded / t_decode, 1), "decode_ms_per_step": round(t_decode * 1e3 / steps, 3),
        "prefill_tokens_per_s": round(prefilled / max(t_prefill, 1e-9), 1), "prefill_ms_per_step": round(t_prefill * 1e3 / steps, 3),
        "restarts": restarts, "mean_keys_per_slot": round(keys_read / max(decoded, 1), 1),
        "decode_ms_by_mean_keys": [[round(k), round(m, 2)] for k, m in per_step],
        "roofline": {"bound": "hbm", "achieved": round(decode_bytes / t_decode / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(decode_bytes / t_decode / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": None, "kernel": "whole decode step (cached K/V read once + weights once) / decode time"},
        "cpu_baseline": cpu_res,
        "gemm_route": gemm_route(calls0),
    }


def with_own_kernels(others):
    """When a run was asked to send products to the vendor's GEMM library, the same prefill and churn steps once more on
    the kernels of this library, so that the line carries both (`ms_per_step_own_kernels`)."""
    from glinthawk_amd import _lib
    L = _lib.lib()
    rows = int(L.gh_gemm_library_rows())
    if rows == 0:
        return
    _lib.check(L.gh_gemm_set_library_rows(0))
    try:
        for key, again in (("cfg3", lambda: prefill_bench(3, 1, False)), ("cfg5", lambda: churn_bench(16, 3, False))):
            if key in others and others[key]["gemm_route"]["route"] == "vendor":
                others[key]["ms_per_step_own_kernels"] = again()["ms_per_step"]
    finally:
        _lib.check(L.gh_gemm_set_library_rows(rows))


def full_configs(cpu):
    """The configurations other than the headline at the run lengths they are stated with (the default run keeps them short)."""
    g = decode_bench("llama2-7b-b32-ctx1024", 128, 3, cpu=False, events=False, advance=True)
    cfg2 = {"workload": "llama2-7b-b32-ctx1024", "steps": 128, "keys_per_context": "1024..1151, one more per step",
            "ms_per_step": round(g["ms_per_step"], 4), "stage_tokens_per_s": round(g["batch"] / (g["ms_per_step"] * 1e-3), 1),
            "stage_roofline_frac": round(g["stage_bytes"] / (HBM_PEAK_GBPS * 1e9) * 1e3 / g["ms_per_step"], 4), "gemm_route": g["gemm_route"]}
    cfg3 = brief(prefill_bench(3, 1, cpu))
    cfg3["decode_steps"] = 64
    cfg5 = brief(churn_bench(512, 3, cpu))
    by_keys = cfg5.pop("decode_ms_by_mean_keys")
    cfg5["decode_ms_by_mean_keys_every_32nd_step"] = by_keys[::32]
    return {"full_configs": {"cfg2": cfg2, "cfg3": cfg3, "cfg5": cfg5}, "n_gpus": 1, "data": "synthetic", "dtype": "f16"}


def brief(line):
    """What the headline line keeps of another configuration's line."""
    keep = ("value", "unit", "ms_per_step", "steps", "warmup", "stage_tokens_per_s", "stage_roofline_frac", "attn_kernel_ms", "decode_ms_per_step",
            "decode_tokens_per_s", "prefill_ms_per_step", "prefill_tokens_per_s", "mean_keys_per_slot", "decode_ms_by_mean_keys", "gemm_route",
            "ms_per_step_own_kernels")
    out = {"workload": line["config"]["workload"], "metric": line["metric"]}
    out.update({k: line[k] for k in keep if k in line})
    r = line["roofline"]
    out["roofline"] = {k: r[k] for k in ("bound", "achieved", "peak", "unit", "frac", "kernel")}
    c = line.get("cpu_baseline")
    out["cpu_baseline"] = None if c is None else {k: (round(c[k], 2) if k == "value" else c[k]) for k in ("value", "unit", "cores", "kind", "sample")}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama2-70b-gqa-b64-ctx4096", choices=sorted(WORKLOADS) + sorted(OTHER_WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--skip-others", action="store_true",
                    help="only the named workload: no concept-path run and no short runs of the other configurations")
    ap.add_argument("--attn-variant", default="auto", choices=["auto", "generic", "valu", "mfma"],
                    help="decode attention kernel the stage uses (measurement of the alternatives; auto = the library's choice)")
    ap.add_argument("--attn-split-join", type=int, default=1, choices=[0, 1, 4, 8],
                    help="measurement hook: how the splits of a context are added up in the decode attention (1: the library's choice; 0: always partial "
                         "sums and the merge kernel; 4, 8: inside work-groups of that many waves where the plan has 2 or 4 splits)")
    ap.add_argument("--gate-waves", type=int, default=0, choices=[0, 4, 8],
                    help="measurement hook: waves per work-group of the decode product that computes w1 and w3 in one launch (0: the library's choice)")
    ap.add_argument("--attn-chunk", type=int, default=0,
                    help="measurement hook: keys per split of the decode attention (0: the library's plan)")
    ap.add_argument("--concept-path", action="store_true", help="time the named decode workload through the reference's op sequence only")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run a plain D2D copy of this many MiB (reference point for profiler byte counters)")
    ap.add_argument("--library-rows", type=int, default=-1,
                    help="measurement hook: rows from which plain products go to the vendor's GEMM library (0: never; default: the library's own setting, "
                         "which is never unless GLINT_LIBRARY_ROWS says otherwise)")
    ap.add_argument("--full-configs", action="store_true",
                    help="the other configurations at their stated run lengths instead of the headline line: 128 decode steps at 1024..1151 keys "
                         "(7B shape), the 8 x 2048 prefill with its 64 decode steps (13B shape), 512 churn steps (70B shape); takes some minutes")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build runs one pipeline stage on ONE GPU; --gpus must be 1 "
              "(the path shards by context, slot -> GPU, with no collective; only the one-GPU share is built)", file=sys.stderr)
        sys.exit(2)

    cpu = not args.no_cpu_baseline
    if args.calibration_copy_mib > 0:
        from glinthawk_amd import ops
        ops.init(0)
        calibration_copy(args.calibration_copy_mib << 20)
    if args.library_rows >= 0:
        from glinthawk_amd import _lib, ops
        ops.init(0)
        _lib.check(_lib.lib().gh_gemm_set_library_rows(args.library_rows))
    if args.attn_split_join != 1:
        from glinthawk_amd import _lib, ops
        ops.init(0)
        _lib.check(_lib.lib().gh_attn_set_split_join(args.attn_split_join))
    if args.attn_chunk > 0:
        from glinthawk_amd import ops
        ops.init(0)
        ops.attn_set_chunk(args.attn_chunk)
    if args.gate_waves:
        from glinthawk_amd import _lib, ops
        ops.init(0)
        _lib.check(_lib.lib().gh_gemm_set_gate_waves(args.gate_waves))
    if args.attn_variant != "auto":
        from glinthawk_amd import _lib, ops
        ops.init(0)
        _lib.check(_lib.lib().gh_attn_set_auto_variant({"generic": 1, "valu": 2, "mfma": 3}[args.attn_variant]))
    if args.full_configs:
        print(json.dumps(full_configs(cpu)))
        return
    if args.workload == "llama2-13b-prefill-8x2048":
        print(json.dumps(prefill_bench(args.steps, args.warmup, cpu)))
        return
    if args.workload == "llama2-70b-churn-256":
        print(json.dumps(churn_bench(args.steps, args.warmup, cpu)))
        return
    if args.concept_path:
        print(json.dumps({"workload": args.workload, "concept_path": concept_path(args.workload, args.steps, args.warmup)}))
        return

    line = decode_line(args.workload, args.steps, args.warmup, args.attn_variant, cpu)
    if not args.skip_others and args.workload == "llama2-70b-gqa-b64-ctx4096":
        # bounded runs of everything else the configurations name, in the same process and the same line
        line["concept_path_ms_per_step"] = None
        cp = concept_path(args.workload, min(args.steps, 10), 2)
        line["concept_path_ms_per_step"] = cp["ms_per_step"]
        line["concept_path"] = cp
        others = {
            "cfg2": decode_line("llama2-7b-b32-ctx1024", min(args.steps, 20), 3, "auto", cpu),
            "cfg3": prefill_bench(3, 1, cpu),
            "cfg5": churn_bench(16, 3, cpu),
        }
        with_own_kernels(others)
        line["other"] = {k: brief(v) for k, v in others.items()}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
