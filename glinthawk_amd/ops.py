"""Thin torch-tensor front-end over the C-ABI, for the tests and the benchmark.

torch is used for device memory and the current stream only; every function below ends in exactly
one call into libglint_hip.so.  Names follow the reference's op names
(models/common/ops/concept.hh, models/llama2/ops/concept.hh).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import GH_ATTN_AUTO, GH_F16, GH_F32, Shape, check, lib


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return GH_F16
    if t.dtype == torch.float32:
        return GH_F32
    raise TypeError(f"unsupported dtype {t.dtype}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    assert t.is_contiguous()
    return t.data_ptr()


def init(device: int = 0) -> None:
    check(lib().gh_init(device), "gh_init")


def device_name() -> str:
    buf = C.create_string_buffer(128)
    check(lib().gh_device_name(buf, 128), "gh_device_name")
    return buf.value.decode()


# ---- tables -------------------------------------------------------------------------------------
def row_table(ptrs: Sequence[int], device="cuda") -> torch.Tensor:
    """Device-resident table of row / layer base addresses (0 = empty context)."""
    return torch.tensor([int(p) for p in ptrs], dtype=torch.int64, device=device)


def host_ptr_array(ptrs: Sequence[int]):
    arr = (C.c_void_p * max(1, len(ptrs)))()
    for i, p in enumerate(ptrs):
        arr[i] = p if p else None
    return arr


def host_u32_array(vals: Sequence[int]):
    arr = (C.c_uint32 * max(1, len(vals)))()
    for i, v in enumerate(vals):
        arr[i] = int(v)
    return arr


# ---- common ops ---------------------------------------------------------------------------------
def accum(a: torch.Tensor, b: torch.Tensor) -> None:
    batch, size = a.shape
    check(lib().gh_accum(_p(a), _p(b), size, batch, _dt(a), _stream()), "gh_accum")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    batch, size = x.shape
    out = torch.empty_like(x) if out is None else out
    check(lib().gh_rmsnorm(_p(out), _p(x), _p(weight), size, batch, _dt(x), _stream()), "gh_rmsnorm")
    return out


def silu(hb: torch.Tensor, hb2: torch.Tensor) -> None:
    batch, hidden = hb.shape
    check(lib().gh_silu(_p(hb), _p(hb2), hidden, batch, _dt(hb), _stream()), "gh_silu")


def argmax(v: torch.Tensor, to_host: bool = True):
    batch, n = v.shape
    out_dev = torch.empty(batch, dtype=torch.int32, device=v.device)
    host = (C.c_uint32 * batch)() if to_host else None
    check(lib().gh_argmax(host, _p(out_dev), _p(v), n, batch, _dt(v), _stream()), "gh_argmax")
    return list(host) if to_host else out_dev


def matmul(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    b, s = x.shape
    r, s2 = w.shape
    assert s == s2
    out = torch.empty((b, r), dtype=x.dtype, device=x.device) if out is None else out
    check(lib().gh_matmul(_p(out), _p(x), _p(w), s, r, b, _dt(x), _stream()), "gh_matmul")
    return out


def matmul_pair(x: torch.Tensor, w: torch.Tensor, rows_first: int):
    """(x @ w[:rows_first].T, x @ w[rows_first:].T): two products that share their activations."""
    b, s = x.shape
    r, s2 = w.shape
    assert s == s2 and 0 < rows_first < r and w.is_contiguous()
    out_a = torch.empty((b, rows_first), dtype=x.dtype, device=x.device)
    out_b = torch.empty((b, r - rows_first), dtype=x.dtype, device=x.device)
    check(lib().gh_matmul_pair(_p(out_a), _p(out_b), _p(x), _p(w), s, rows_first, r - rows_first, b, _dt(x), _stream()),
          "gh_matmul_pair")
    return out_a, out_b


def matmul_accum(residual: torch.Tensor, x: torch.Tensor, w: torch.Tensor, norm_weight: Optional[torch.Tensor] = None):
    """residual += x @ w.T; returns rmsnorm(residual) * norm_weight when a weight is given."""
    b, s = x.shape
    r = w.shape[0]
    norm_out = torch.empty_like(residual) if norm_weight is not None else None
    check(lib().gh_matmul_accum(_p(residual), _p(x), _p(w), s, r, b, _p(norm_out), _p(norm_weight), _dt(x), _stream()),
          "gh_matmul_accum")
    return norm_out


def matmul_silu_gate(x: torch.Tensor, w13: torch.Tensor) -> torch.Tensor:
    b, s = x.shape
    hidden = w13.shape[0] // 2
    hb = torch.empty((b, hidden), dtype=x.dtype, device=x.device)
    check(lib().gh_matmul_silu_gate(_p(hb), _p(x), _p(w13), s, hidden, b, _dt(x), _stream()), "gh_matmul_silu_gate")
    return hb


def matmul_qkv_rope_append(x: torch.Tensor, wqkv: torch.Tensor, pos: torch.Tensor, freq_real, freq_imag,
                           token_rows: torch.Tensor, shape: Shape, want_kv: bool = False):
    b, s = x.shape
    q = torch.empty((b, shape.dim), dtype=x.dtype, device=x.device)
    kv = torch.empty((b, 2 * shape.kv_dim), dtype=x.dtype, device=x.device) if want_kv else None
    check(lib().gh_matmul_qkv_rope_append(_p(q), _p(kv), _p(x), _p(wqkv), s, b, _p(pos), _p(freq_real), _p(freq_imag),
                                          _p(token_rows), shape.n_kv_heads, shape.gqa_size, shape.head_size, _dt(x),
                                          _stream()), "gh_matmul_qkv_rope_append")
    return q, kv


def soft_sample(v: torch.Tensor, temperatures: Sequence[float], seed: int = 0) -> None:
    batch, vocab = v.shape
    temps = (C.c_float * batch)(*[float(t) for t in temperatures])
    check(lib().gh_soft_sample(_p(v), temps, vocab, batch, seed, _dt(v), _stream()), "gh_soft_sample")


def fill_normal(t: torch.Tensor, mean: float, std: float, seed: int) -> None:
    check(lib().gh_fill_normal(_p(t), t.numel(), mean, std, seed, _dt(t), _stream()), "gh_fill_normal")


def fill_uniform(t: torch.Tensor, lo: float, hi: float, seed: int) -> None:
    check(lib().gh_fill_uniform(_p(t), t.numel(), lo, hi, seed, _dt(t), _stream()), "gh_fill_uniform")


# ---- llama2 ops ---------------------------------------------------------------------------------
def kv_append(token_rows: torch.Tensor, state_kv: torch.Tensor, kv_dim: int) -> None:
    """token_rows: int64 device table of row addresses."""
    batch = token_rows.numel()
    check(lib().gh_kv_append(_p(token_rows), _p(state_kv), batch, kv_dim, _dt(state_kv), _stream()), "gh_kv_append")


def kv_append_host(token_rows: Sequence[int], state_kv: torch.Tensor, kv_dim: int) -> None:
    arr = host_ptr_array(token_rows)
    check(lib().gh_kv_append_host(arr, _p(state_kv), len(token_rows), kv_dim, _dt(state_kv), _stream()),
          "gh_kv_append_host")


def rope(pos: torch.Tensor, freq_real: torch.Tensor, freq_imag: torch.Tensor, q: torch.Tensor,
         token_rows: torch.Tensor, shape: Shape) -> None:
    batch = token_rows.numel()
    check(lib().gh_rope(batch, _p(pos), _p(freq_real), _p(freq_imag), _p(q), _p(token_rows),
                        shape.n_kv_heads, shape.gqa_size, shape.head_size, _dt(q), _stream()), "gh_rope")


def rope_host(pos: Sequence[int], freq_real: torch.Tensor, freq_imag: torch.Tensor, q: torch.Tensor,
              token_rows: Sequence[int], shape: Shape) -> None:
    check(lib().gh_rope_host(len(token_rows), host_u32_array(pos), _p(freq_real), _p(freq_imag), _p(q),
                             host_ptr_array(token_rows), shape.n_kv_heads, shape.gqa_size, shape.head_size,
                             _dt(q), _stream()), "gh_rope_host")


def attn_scores(q, layer_rows: torch.Tensor, att, pos: torch.Tensor, shape: Shape) -> None:
    s = shape.c()
    check(lib().gh_attn_scores(_p(q), _p(layer_rows), _p(att), layer_rows.numel(), _p(pos), C.byref(s), _dt(q),
                               _stream()), "gh_attn_scores")


def attn_softmax(att, pos: torch.Tensor, shape: Shape) -> None:
    s = shape.c()
    check(lib().gh_attn_softmax(_p(att), _p(pos), pos.numel(), C.byref(s), _dt(att), _stream()), "gh_attn_softmax")


def attn_pv(att, layer_rows: torch.Tensor, xb, pos: torch.Tensor, shape: Shape) -> None:
    s = shape.c()
    check(lib().gh_attn_pv(_p(att), _p(layer_rows), _p(xb), layer_rows.numel(), _p(pos), C.byref(s), _dt(att),
                           _stream()), "gh_attn_pv")


def attn_scores_host(q, layer_rows: Sequence[int], att, pos: Sequence[int], shape: Shape) -> None:
    s = shape.c()
    check(lib().gh_attn_scores_host(_p(q), host_ptr_array(layer_rows), _p(att), len(layer_rows), host_u32_array(pos),
                                    C.byref(s), _dt(q), _stream()), "gh_attn_scores_host")


def attn_softmax_host(att, pos: Sequence[int], shape: Shape) -> None:
    s = shape.c()
    check(lib().gh_attn_softmax_host(_p(att), host_u32_array(pos), len(pos), C.byref(s), _dt(att), _stream()),
          "gh_attn_softmax_host")


def attn_pv_host(att, layer_rows: Sequence[int], xb, pos: Sequence[int], shape: Shape) -> None:
    s = shape.c()
    check(lib().gh_attn_pv_host(_p(att), host_ptr_array(layer_rows), _p(xb), len(layer_rows), host_u32_array(pos),
                                C.byref(s), _dt(att), _stream()), "gh_attn_pv_host")


def attn_decode_workspace(batch: int, max_pos: int, shape: Shape) -> int:
    s = shape.c()
    return int(lib().gh_attn_decode_workspace(batch, max_pos, C.byref(s)))


def attn_decode_join_waves(batch: int, max_pos: int, shape: Shape, dt: int = GH_F16, variant: int = GH_ATTN_AUTO) -> int:
    """Waves per work-group if the call's splits are added up inside the work-groups, 0 if partial sums and the merge kernel are used."""
    s = shape.c()
    return int(lib().gh_attn_decode_join_waves(batch, max_pos, C.byref(s), dt, variant))


def attn_decode(q, layer_rows: torch.Tensor, pos: torch.Tensor, xb, max_pos: int, shape: Shape,
                workspace: Optional[torch.Tensor] = None, variant: int = GH_ATTN_AUTO) -> None:
    s = shape.c()
    batch = layer_rows.numel()
    if workspace is None:
        workspace = torch.empty(attn_decode_workspace(batch, max_pos, shape), dtype=torch.uint8, device=q.device)
    check(lib().gh_attn_decode(_p(q), _p(layer_rows), _p(pos), _p(xb), batch, max_pos, C.byref(s), _dt(q),
                               _p(workspace), workspace.numel() * workspace.element_size(), variant, _stream()),
          "gh_attn_decode")


def attn_balanced_workspace(batch: int, shape: Shape) -> int:
    s = shape.c()
    return int(lib().gh_attn_balanced_workspace(batch, C.byref(s)))


def attn_balance(layer_rows: torch.Tensor, pos: torch.Tensor, max_pos: int, shape: Shape, workspace: torch.Tensor) -> None:
    """Cuts the keys of a batch into equal runs (once per step); `workspace` then serves attn_decode_balanced for every layer."""
    s = shape.c()
    check(lib().gh_attn_balance(_p(layer_rows), _p(pos), layer_rows.numel(), max_pos, C.byref(s), _p(workspace),
                                workspace.numel() * workspace.element_size(), _stream()), "gh_attn_balance")


def attn_decode_balanced(q, layer_rows: torch.Tensor, xb, max_pos: int, shape: Shape, workspace: torch.Tensor) -> None:
    s = shape.c()
    check(lib().gh_attn_decode_balanced(_p(q), _p(layer_rows), _p(xb), layer_rows.numel(), max_pos, C.byref(s), _dt(q), _p(workspace),
                                        workspace.numel() * workspace.element_size(), _stream()), "gh_attn_decode_balanced")


def attn_decode_host(q, layer_rows: Sequence[int], pos: Sequence[int], xb, shape: Shape,
                     workspace: Optional[torch.Tensor] = None, variant: int = GH_ATTN_AUTO) -> None:
    s = shape.c()
    batch = len(layer_rows)
    if workspace is None:
        workspace = torch.empty(attn_decode_workspace(batch, shape.seq_len - 1, shape), dtype=torch.uint8,
                                device=q.device)
    check(lib().gh_attn_decode_host(_p(q), host_ptr_array(layer_rows), host_u32_array(pos), _p(xb), batch,
                                    C.byref(s), _dt(q), _p(workspace), workspace.numel(), variant, _stream()),
          "gh_attn_decode_host")


def prefill_tables(layer_rows: torch.Tensor, start_pos: torch.Tensor, n_tokens: int, row_bytes: int):
    """Expanded (context, token) tables: (layer_rows, token_rows, pos), each of batch * n_tokens entries."""
    batch = layer_rows.numel()
    n = batch * n_tokens
    rows = torch.empty(n, dtype=torch.int64, device=layer_rows.device)
    trows = torch.empty(n, dtype=torch.int64, device=layer_rows.device)
    pos = torch.empty(n, dtype=torch.int32, device=layer_rows.device)
    check(lib().gh_prefill_tables(_p(layer_rows), _p(start_pos), batch, n_tokens, row_bytes, _p(rows), _p(trows), _p(pos),
                                  _stream()), "gh_prefill_tables")
    return rows, trows, pos


def attn_prefill(q, layer_rows: torch.Tensor, start_pos: torch.Tensor, xb, n_tokens: int, max_start_pos: int, shape: Shape,
                 variant: int = GH_ATTN_AUTO) -> None:
    s = shape.c()
    batch = layer_rows.numel()
    ws = torch.empty(int(lib().gh_attn_prefill_workspace(batch, n_tokens, C.byref(s))), dtype=torch.uint8, device=q.device)
    check(lib().gh_attn_prefill(_p(q), _p(layer_rows), _p(start_pos), _p(xb), batch, n_tokens, max_start_pos, C.byref(s),
                                _dt(q), _p(ws), ws.numel(), variant, _stream()), "gh_attn_prefill")


def attn_set_chunk(tokens: int) -> None:
    check(lib().gh_attn_set_chunk(tokens), "gh_attn_set_chunk")


def attn_set_split_join(mode) -> None:
    """0 / False: partial sums + merge kernel; 1 / True: the library's choice; 4, 8: joined with that many waves per work-group."""
    check(lib().gh_attn_set_split_join(int(mode)), "gh_attn_set_split_join")


def pinned_empty(shape, dtype):
    """A numpy array in page-locked host memory (gh_host_malloc): transfers to and from the device need
    no staging copy.  The memory is released when the array and every view of it are gone."""
    import ctypes as C
    import weakref

    import numpy as np

    dt = np.dtype(dtype)
    n = int(np.prod(shape)) * dt.itemsize
    ptr = C.c_void_p()
    check(lib().gh_host_malloc(C.byref(ptr), max(n, 1)), "gh_host_malloc")
    buf = (C.c_uint8 * max(n, 1)).from_address(ptr.value)
    arr = np.frombuffer(buf, dtype=dt, count=int(np.prod(shape))).reshape(shape)
    weakref.finalize(buf, lambda p=ptr.value: lib().gh_host_free(C.c_void_p(p)))
    return arr


def _addr(buf) -> int:
    """Address of a torch tensor (device or host) or of a numpy array."""
    if isinstance(buf, torch.Tensor):
        assert buf.is_contiguous()
        return buf.data_ptr()
    assert buf.flags["C_CONTIGUOUS"]
    return buf.ctypes.data


def _dt_any(buf) -> int:
    name = str(buf.dtype).replace("torch.", "")
    if name == "float16":
        return GH_F16
    if name == "float32":
        return GH_F32
    raise TypeError(f"unsupported dtype {buf.dtype}")


def convert_and_copy(dst, src, n: int, kind: int) -> None:
    """LlamaOperations::convert_and_copy: `n` elements from `src` to `dst` (torch device tensors or numpy host
    arrays, as `kind` says), converted element by element when the two types differ."""
    check(lib().gh_convert_and_copy(_addr(dst), _dt_any(dst), _addr(src), _dt_any(src), n, kind, _stream()), "gh_convert_and_copy")


def convert(dst: torch.Tensor, src: torch.Tensor, n: int) -> None:
    check(lib().gh_convert(_p(dst), _dt(dst), _p(src), _dt(src), n, _stream()), "gh_convert")


def sync() -> None:
    check(lib().gh_sync(None), "gh_sync")
