"""On-disk formats and the store writer's preprocessing.

Follows bergson/builder.py:14-32 (`_preprocess`), bergson/data.py:37-137 and
:380-445 and :492-519 (gradient store), bergson/score/score_writer.py:16-58
(score-store record layout).
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from torch import Tensor

EPS_SQ = torch.finfo(torch.float32).eps ** 2


def preprocess(mod_grads: dict[str, Tensor], grad_sizes: dict[str, int], unit_normalize: bool) -> Tensor:
    """Concatenate modules in grad_sizes order, optionally unit-normalise rows (builder.py:17-32)."""
    grads = torch.cat([mod_grads[m] for m in grad_sizes.keys()], dim=-1)
    if unit_normalize:
        inv = grads.pow(2).sum(dim=-1).clamp_min_(EPS_SQ).rsqrt().unsqueeze(1)
        grads = grads * inv
    return grads


def num_token_grads(lengths) -> np.ndarray:
    """max(length - 1, 0) rows per document (data.py:37-62)."""
    return np.maximum(np.asarray(lengths, dtype=np.int64) - 1, 0)


def token_offsets(lengths) -> np.ndarray:
    """int64 [num_items + 1] cumulative row offsets (data.py:99-101)."""
    n = num_token_grads(lengths)
    off = np.zeros(len(n) + 1, dtype=np.int64)
    np.cumsum(n, out=off[1:])
    return off


def column_offsets(grad_sizes: dict[str, int]) -> dict[str, tuple[int, int]]:
    """data.py:380-389."""
    out, start = {}, 0
    for name, size in grad_sizes.items():
        out[name] = (start, start + size)
        start += size
    return out


def index_info(num_items: int, num_grads: int, grad_sizes: dict[str, int], base_dtype: str,
               attribute_tokens: bool) -> dict:
    """The info.json record (data.py:114-125, :421-432)."""
    return {
        "attribute_tokens": attribute_tokens,
        "num_items": num_items,
        "num_grads": num_grads,
        "grad_sizes": grad_sizes,
        "base_dtype": base_dtype,
    }


def read_store_bytes(root: Path) -> tuple[dict, np.ndarray]:
    """info.json plus gradients.bin as raw bytes reshaped to [num_grads, row_bytes] (data.py:492-519)."""
    root = Path(root)
    info = json.loads((root / "info.json").read_text())
    itemsize = {"float16": 2, "bfloat16": 2, "float32": 4, "float64": 8}[info["base_dtype"]]
    width = sum(info["grad_sizes"].values()) * itemsize
    raw = np.fromfile(root / "gradients.bin", dtype=np.uint8)
    return info, raw.reshape(info["num_grads"], width)


def score_struct_dtype(num_scores: int, score_itemsize: int, score_format: str) -> dict:
    """Interleaved (score_i, written_i) record (score_writer.py:16-58)."""
    pair = score_itemsize + 1
    aligned = 1 << (pair - 1).bit_length()
    names, formats, offsets = [], [], []
    for i in range(num_scores):
        names += [f"score_{i}", f"written_{i}"]
        formats += [score_format, "bool"]
        offsets += [i * aligned, i * aligned + score_itemsize]
    total = num_scores * aligned
    return {"names": names, "formats": formats, "offsets": offsets, "itemsize": ((total + 7) // 8) * 8}
