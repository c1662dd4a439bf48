"""Scores a batch of index gradients against the query gradients (bergson/score/scorer.py).

The reference loops over modules with one small GEMM and one sum of squares
each; here the batch's rows and the queries are each one [., D] matrix and a
single `bgx_scan` launch produces scores, row norms and the per-row maximum.
"""
from __future__ import annotations

from collections.abc import Callable

import torch
from torch import Tensor

from . import ops
from .builder import RowBlock
from .score_writer import ScoreWriter


def _identity(x):
    return x


class Scorer:
    """Same constructor and call protocol as the reference's Scorer (scorer.py:21-90)."""

    def __init__(self, query_grads: dict[str, Tensor], modules: list[str], writer: ScoreWriter,
                 device: torch.device, dtype: torch.dtype, *, unit_normalize: bool = False,
                 score_mode: str = "individual", attribute_tokens: bool = False,
                 index_transform: Callable[[dict[str, Tensor]], dict[str, Tensor]] = _identity,
                 query_offset: int = 0):
        self.device = torch.device(device)
        self.dtype = dtype
        self.modules = list(modules)
        self.unit_normalize = unit_normalize
        self.score_mode = score_mode
        self.attribute_tokens = attribute_tokens
        self.writer = writer
        self.index_transform = index_transform
        self.query_offset = query_offset
        if self.device.type != "cuda":
            raise RuntimeError("bergson_amd has no CPU path: Scorer needs a GPU device")
        if dtype not in ops.DTYPE_CODE:
            raise TypeError(f"Scorer dtype {dtype} is not supported by the scan kernels")
        # queries as one [Q, D] matrix in module order
        self.queries = torch.cat([query_grads[m].to(device=self.device, dtype=self.dtype) for m in self.modules],
                                 dim=1).contiguous()
        # kept for callers that read the reference's attribute
        self.query_grads_t = {m: query_grads[m].to(device=self.device, dtype=self.dtype).T for m in self.modules}

    def __call__(self, indices: list[int], mod_grads: dict[str, Tensor]):
        scores = self.score(mod_grads)
        self.writer(indices, scores, query_offset=self.query_offset)

    @torch.inference_mode()
    def score(self, index_grads: dict[str, Tensor]) -> Tensor:
        """[rows, Q] scores, or [rows, 1] row maxima with score_mode='nearest' (scorer.py:89-115)."""
        transformed = self.index_transform(index_grads)
        rows = None
        if isinstance(transformed, RowBlock) and transformed.rows is not None and list(transformed.keys()) == self.modules:
            rows = transformed.rows
        if rows is None:
            rows = torch.cat([transformed[m].to(self.device, non_blocking=True) for m in self.modules], dim=1)
        rows = rows.to(device=self.device, dtype=self.dtype)
        if rows.stride(-1) != 1:
            rows = rows.contiguous()
        if rows.shape[0] == 0:
            width = 1 if self.score_mode == "nearest" else self.queries.shape[0]
            return torch.zeros((0, width), dtype=torch.float32, device=self.device)
        nearest = self.score_mode == "nearest"
        res = ops.scan(rows, self.queries, unit_norm=self.unit_normalize, want_scores=not nearest,
                       want_row_max=nearest)
        if nearest:
            return res.row_max.unsqueeze(1)
        return res.scores
