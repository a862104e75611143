"""Writer for the reference's on-disk model directory (the output format of its converter,
tools/bin2glint.py:28-86): CONFIG, BASEWEIGHTS_<FP16|FP32>, LAYER<i>_<FP16|FP32>.  For exporting
synthetic or converted weights to a directory that `Stage.load()` -- and the reference -- read."""
from __future__ import annotations

import os
import struct
from typing import Dict, Sequence

import numpy as np


def dtype_text(np_dtype) -> str:
    return "FP16" if np.dtype(np_dtype) == np.float16 else "FP32"


def write_config(dest_dir: str, dim: int, hidden_dim: int, n_layers: int, n_heads: int, n_kv_heads: int,
                 vocab_size: int, seq_len: int, wcls_present: bool) -> None:
    """Seven native int32; a negative vocabulary size marks a separate classifier matrix."""
    os.makedirs(dest_dir, exist_ok=True)
    with open(os.path.join(dest_dir, "CONFIG"), "wb") as f:
        f.write(struct.pack("=iiiiiii", dim, hidden_dim, n_layers, n_heads, n_kv_heads,
                            -vocab_size if wcls_present else vocab_size, seq_len))


def write_model_dir(dest_dir: str, cfg, layers: Sequence[Dict[str, np.ndarray]], base: Dict[str, np.ndarray],
                    np_dtype, wcls_present: bool, only_layers=None, write_base: bool = True) -> None:
    """`cfg` has dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len.  `layers[i]` maps
    rms_att_weight, wq, wkv (wk rows then wv rows), wo, rms_ffn_weight, w1, w2, w3 to arrays; `base`
    maps token_embedding_table, rms_final_weight, freq_cis_real, freq_cis_imag and (if present) wcls."""
    dt = np.dtype(np_dtype)
    text = dtype_text(dt)
    write_config(dest_dir, cfg.dim, cfg.hidden_dim, cfg.n_layers, cfg.n_heads, cfg.n_kv_heads, cfg.vocab_size,
                 cfg.seq_len, wcls_present)
    if write_base:
        with open(os.path.join(dest_dir, f"BASEWEIGHTS_{text}"), "wb") as f:
            names = ["token_embedding_table", "rms_final_weight", "freq_cis_real", "freq_cis_imag"]
            if wcls_present:
                names.append("wcls")
            for n in names:
                f.write(np.ascontiguousarray(base[n], dtype=dt).tobytes())
    for i in (range(cfg.n_layers) if only_layers is None else only_layers):
        with open(os.path.join(dest_dir, f"LAYER{i}_{text}"), "wb") as f:
            # the converter writes wk then wv; together they are the (2 kv_dim, dim) matrix wkv
            for n in ("rms_att_weight", "wq", "wkv", "wo", "rms_ffn_weight", "w1", "w2", "w3"):
                f.write(np.ascontiguousarray(layers[i][n], dtype=dt).tobytes())
