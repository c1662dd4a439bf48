"""Query an existing gradient store (bergson/query/attributor.py).

The store stays in HBM in its on-disk dtype (e.g. 24.6 GB for 10^6 fp16 rows of
12288); `search` streams it once through `bgx_scan`, which folds the row
normalisation (attributor.py:137-167), the GEMM against the queries and the
per-query top-k (attributor.py:229-235) into one pass.
"""
from __future__ import annotations

import math
from contextlib import contextmanager
from pathlib import Path
from typing import Generator

import numpy as np
import torch
import torch.nn as nn
from torch import Tensor

from . import ops
from .data import column_offsets, load_gradients, load_info, store_base_dtype
from .gradient_collectors import TraceCollector
from .gradients import GradientProcessor
from .utils import numpy_to_tensor, torch_dtype_from_name


class TraceResult:
    """Holds the top-k of a `trace()` block once it has exited (attributor.py:22-44)."""

    def __init__(self):
        self._indices: Tensor | None = None
        self._scores: Tensor | None = None

    @property
    def indices(self) -> Tensor:
        if self._indices is None:
            raise ValueError("No indices available. Exit the context manager first.")
        return self._indices

    @property
    def scores(self) -> Tensor:
        if self._scores is None:
            raise ValueError("No scores available. Exit the context manager first.")
        return self._scores


def upload_store(mmap: np.ndarray, base_dtype: str, device: torch.device, chunk_bytes: int = 1 << 30) -> Tensor:
    """Copies a mapped store to the device in row chunks, keeping its dtype and bits."""
    n, D = mmap.shape
    out = torch.empty((n, D), dtype=torch_dtype_from_name(base_dtype), device=device)
    step = max(1, chunk_bytes // max(1, D * mmap.dtype.itemsize))
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        out[lo:hi].copy_(numpy_to_tensor(mmap[lo:hi], base_dtype), non_blocking=False)
    return out


class Attributor:
    """`Attributor(index_path, device, dtype, unit_norm).search(queries, k)` (attributor.py:47-235)."""

    def __init__(self, index_path: str | Path, device: str = "cuda", dtype: torch.dtype = torch.float32,
                 unit_norm: bool = False, faiss_cfg=None, inversion_cfg=None, hessian_path: str | Path | None = None,
                 ev_correction: bool = False, device_store_bytes: int | None = None):
        if faiss_cfg is not None:
            raise NotImplementedError("FAISS search is outside this package; the exact scan replaces the Flat index")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("bergson_amd has no CPU path: Attributor needs a GPU device")
        self.dtype = dtype
        self.unit_norm = unit_norm
        # `hessian_path` enables preconditioning: H^-1 on the queries, or -- with unit_norm -- H^-1/2 on the
        # index rows as well as on the queries (attributor.py:73-89)
        if hessian_path is None:
            self.precondition = "none"
            self.preconditioner = None
        else:
            from .hessians import load_preconditioner

            self.precondition = "two-sided" if unit_norm else "one-sided"
            self.preconditioner = load_preconditioner(hessian_path, inversion_cfg=inversion_cfg,
                                                      power=-0.5 if unit_norm else -1.0, ev_correction=ev_correction,
                                                      device=self.device)
        self.faiss_index = None
        index_path = Path(index_path)
        self.processor = GradientProcessor.load(index_path, map_location=device)
        info = load_info(index_path)
        self.grad_sizes: dict[str, int] = info["grad_sizes"]
        self.ordered_modules = list(self.grad_sizes)
        self._columns = column_offsets(self.grad_sizes)
        base = store_base_dtype(info)
        if base == "float64":
            raise TypeError("float64 stores are not supported by the scan kernels")
        self._row_sumsq: Tensor | None = None
        self._row_sumsq_of: tuple | None = None
        mapped = load_gradients(index_path)
        self.N = mapped.shape[0]
        # The store lives in HBM when it fits (`device_store_bytes`, default four fifths of the free memory).  A
        # larger one stays mapped on the host and every search streams it through the device in slabs of rows,
        # each scanned like a store of its own (`row_base` = its first row) and merged into the running top-k.
        free, _ = torch.cuda.mem_get_info(self.device)
        budget = int(free * 0.8) if device_store_bytes is None else int(device_store_bytes)
        self._base = base
        self._mapped = None
        self._slab_rows = 0
        self._slab_sumsq: dict[int, Tensor] = {}
        split = self.preconditioner is not None and unit_norm
        if mapped.size * mapped.dtype.itemsize <= budget:
            self.store = upload_store(mapped, base, self.device)
            if split:
                # split mode: the index rows are transformed once, before the scan normalises them.  The
                # transformed store is fp32 (what g.float() @ H gives) when a second, fp32 copy fits in half of the
                # free memory, else it keeps the store's dtype.
                free, _ = torch.cuda.mem_get_info(self.device)
                out_dtype = torch.float32 if self.store.numel() * 4 <= free // 2 else self.store.dtype
                self.store = self.preconditioner.apply_rows(self.store, self.grad_sizes, out_dtype=out_dtype)
            if unit_norm:
                self.row_sumsq()  # the reference normalises the index when it loads it (attributor.py:137-167)
        else:
            self.store = None
            self._mapped = mapped
            row_bytes = mapped.shape[1] * mapped.dtype.itemsize * (2 if split else 1)  # split mode: slab + its transform
            self._slab_rows = max(1, budget // row_bytes)

    def _slabs(self):
        """(first row, device rows, their sums of squares or None) for every slab of a store that is streamed."""
        for lo in range(0, self.N, self._slab_rows):
            hi = min(self.N, lo + self._slab_rows)
            rows = upload_store(self._mapped[lo:hi], self._base, self.device)
            if self.preconditioner is not None and self.unit_norm:
                rows = self.preconditioner.apply_rows(rows, self.grad_sizes, out_dtype=rows.dtype)
            norms = None
            if self.unit_norm:
                if lo not in self._slab_sumsq:  # 4 bytes per row: kept for the next search
                    self._slab_sumsq[lo] = ops.row_sumsq(rows)
                norms = self._slab_sumsq[lo]
            yield lo, rows, norms

    def row_sumsq(self) -> Tensor:
        """Sums of squares of the store's rows (one HBM-bound pass), kept for every search: the index-side
        normalisation the reference applies once at load time (attributor.py:137-167), here as the row
        multipliers the scan takes instead of summing the squares of every row again.  Recomputed when `store`
        has been replaced or written to since (its storage, shape or version counter changed)."""
        store = self.store
        if store is None:
            raise RuntimeError("this store is streamed from the host in slabs; its row sums are kept per slab")
        state = (store.data_ptr(), tuple(store.shape), store.dtype, store._version)
        if self._row_sumsq is None or self._row_sumsq_of != state:
            self._row_sumsq = ops.row_sumsq(store)
            self._row_sumsq_of = state
        return self._row_sumsq

    @property
    def grads(self) -> dict[str, Tensor]:
        """Per-module column views of the device store (raw rows; normalisation happens inside the scan)."""
        if self.store is None:
            raise RuntimeError("this store is streamed from the host in slabs and has no device-resident views")
        return {name: self.store[:, lo:hi] for name, (lo, hi) in self._columns.items()}

    def search(self, queries: dict[str, Tensor], k: int | None, modules: set[str] | None = None,
               reverse: bool = False):
        """Top-k rows per query by inner product (cosine when unit_norm); returns (values, indices) [..., k]."""
        q = torch.cat([queries[name].to(self.device, torch.float32) for name in self.ordered_modules], dim=1)
        if self.preconditioner is not None:
            q = self.preconditioner.apply_rows(q.contiguous(), self.grad_sizes)
        if self.unit_norm:
            norm = q.norm(dim=1, keepdim=True)
            q = q / (norm + torch.finfo(norm.dtype).eps)
        if modules:
            for name, (lo, hi) in self._columns.items():
                if name not in modules:
                    q[:, lo:hi] = 0
        if reverse:
            q = -q
        k = min(k or self.N, self.N)
        # a power-of-two rescale keeps small query entries clear of the fp16 subnormal range
        qmax = float(q.abs().max().item())
        shift = 0 if qmax == 0 or not math.isfinite(qmax) else -math.frexp(qmax)[1]
        if self.store is not None:
            norms = self.row_sumsq() if self.unit_norm else None
            values, indices = self._search_rows(self.store, 0, norms, q, shift, k)
        else:
            values = indices = None
            for lo, rows, norms in self._slabs():
                v, i = self._search_rows(rows, lo, norms, q, shift, min(k, rows.shape[0]))
                if values is not None:  # the running top-k and the slab's, merged
                    v, i = torch.cat([values, v], dim=1), torch.cat([indices, i], dim=1)
                    v, pick = torch.topk(v, min(k, v.shape[1]), dim=1)
                    i = torch.gather(i, 1, pick)
                values, indices = v, i
                del rows
        if reverse:
            values = -values
        return torch.return_types.topk((values.to(self.dtype), indices))

    def _search_rows(self, rows: Tensor, row_base: int, norms: Tensor | None, q: Tensor, shift: int, k: int):
        """Top-k of `rows` (store rows `row_base` onwards) for fp32 queries `q`: (values, store row numbers)."""
        qd = (q * (2.0 ** shift)).to(rows.dtype)
        scale = 2.0 ** (-shift)
        if k <= ops.SCAN_KMAX:
            res = ops.scan(rows, qd, unit_norm=self.unit_norm, k=k, query_scale=scale, row_base=row_base,
                           row_sumsq=norms)
            return res.topk_values, res.topk_indices
        # beyond the fused selection's capacity of 65 536 (k = None asks for a full ranking of the store): the
        # scan writes every score, in slices of queries so that [n, Q'] fp32 stays near 4 GB, and the
        # ranking is the library's
        step = max(1, (1 << 30) // max(1, rows.shape[0]))
        vals, idxs = [], []
        for lo in range(0, qd.shape[0], step):
            res = ops.scan(rows, qd[lo:lo + step].contiguous(), unit_norm=self.unit_norm, query_scale=scale,
                           want_scores=True, row_sumsq=norms)
            v, i = torch.topk(res.scores.T, k, dim=1)
            vals.append(v)
            idxs.append(i + row_base)
        return torch.cat(vals), torch.cat(idxs)

    @contextmanager
    def trace(self, module: nn.Module, k: int | None, *, modules: set[str] | None = None, reverse: bool = False
              ) -> Generator[TraceResult, None, None]:
        """Collects the gradients of whatever is back-propagated through `module` inside the block and
        searches the store with them (attributor.py:237-282)."""
        result = TraceResult()
        collector = TraceCollector(model=module, processor=self.processor, target_modules=modules,
                                   device=self.device, dtype=self.dtype)
        mod_grads = collector.mod_grads
        with collector:
            yield result
        if not mod_grads:
            raise ValueError("No grads collected. Did you forget to call backward?")
        queries = {name: torch.cat(mod_grads[name], dim=1) for name in self.ordered_modules if name in mod_grads}
        if any(q.isnan().any() for q in queries.values()):
            raise ValueError("NaN found in queries.")
        for name in self.ordered_modules:  # modules that were not traced contribute nothing
            if name not in queries:
                rows = next(iter(queries.values())).shape[0]
                queries[name] = torch.zeros((rows, self.grad_sizes[name]), device=self.device, dtype=self.dtype)
        result._scores, result._indices = self.search(queries, k, modules, reverse)
