"""Concrete collectors (bergson/collector/gradient_collectors.py).

`GradientCollector` (:19-164) builds an on-disk store or feeds a scorer;
`TraceCollector` (:167-203) keeps query gradients on the device;
`StreamingGradientCollector` (:206-240) exposes each step's gradients to a
training callback.

`GradientCollector` defers: its backward hook queues each module's (a, g) and
`process_batch` issues ONE fused launch for the whole batch, writing rows in
the store dtype directly into the builder's device store (or into a [N, D]
batch buffer that the scorer / the builder's normalisation consume).
"""
from __future__ import annotations

import math
from collections import defaultdict
from dataclasses import dataclass, field

import torch
import torch.distributed as dist
import torch.nn as nn
from torch import Tensor

from .builder import Builder, RowBlock
from .collector import HookCollectorBase
from .config import IndexConfig, PreprocessConfig
from .data import column_offsets
from .utils import DeviceIndexRing, get_gradient_dtype


class _DeferredBatchMixin:
    """Shared batch logic of the collectors that write rows of all modules in one launch."""

    def _prepare_collection(self, save_dtype: torch.dtype | None = None) -> dict[str, int]:
        """What a row-writing collector fixes before its first batch: per-token or per-sequence rows, the dtype the
        rows are saved in with its clamp range (`save_dtype`, default the model's gradient dtype), and the
        per-document loss vector; returns the column width of every stored block, in store order."""
        device = self.model.device
        if not isinstance(device, torch.device):
            raise AssertionError("Model device is not set correctly")
        self.attribute_tokens = bool(self.cfg.attribute_tokens)
        if self.attribute_tokens and self.preprocess_cfg.aggregation != "none":
            raise AssertionError("attribute_tokens is incompatible with reduce mode.")
        self.save_dtype = save_dtype or get_gradient_dtype(self.model)
        limits = torch.finfo(self.save_dtype)
        self.lo, self.hi = limits.min, limits.max
        self.per_doc_losses = torch.zeros(len(self.data), dtype=torch.float32, device=device)
        return {name: math.prod(shape) for name, shape in self.shapes().items()}

    def _column_of(self, name: str) -> int:
        cols = getattr(self, "_columns", None)
        if cols is None:
            sizes = {n: math.prod(s) for n, s in self.shapes().items()}
            cols = self._columns = {n: lo for n, (lo, _) in column_offsets(sizes).items()}
            self._row_width = sum(sizes.values())
            self._grad_sizes = sizes
        if self.processor.projection_target == "global":
            return 0  # every module adds into the single "gradients" block
        return cols[name]

    def _indices_dev(self, indices: list[int], device) -> Tensor:
        ring = getattr(self, "_index_ring", None)
        if ring is None:
            ring = self._index_ring = DeviceIndexRing()
        return ring.get(indices, torch.device(device))

    def _record_losses(self, indices: list[int], losses: Tensor) -> None:
        """per_doc_losses[indices] = losses, with the indices taken to the device without a host stall."""
        idx = self._indices_dev(indices, self.per_doc_losses.device)
        self.per_doc_losses.index_copy_(0, idx, losses.detach().to(self.per_doc_losses.dtype))

    def _launch_batch(self, indices: list[int], builder: Builder | None, need_rows: bool) -> RowBlock:
        """Runs the deferred launch.  Rows go straight into the builder's device store when it accepts
        them and nobody else needs them; otherwise into a fresh batch buffer whose column views are
        returned as mod_grads."""
        block = RowBlock()
        queued = self._deferred or self._deferred_adam or self._deferred_full
        if not queued:
            return block
        g0 = queued[0][-1]
        dev = g0.device
        block.indices_dev = self._indices_dev(indices, dev)
        N = g0.shape[0]
        assert N == len(indices), f"batch of {N} sequences but {len(indices)} indices"
        lengths = self._batch_lengths(dev) if (self.attribute_tokens or self.skip_padding) else None
        direct = builder is not None and builder.direct and not need_rows
        if self.attribute_tokens:
            assert lengths is not None, "attribute_tokens needs a collection mask (with_batch)"
            if direct:
                self.launch_deferred(builder.device_rows, lengths=lengths,
                                     row_offsets=builder.token_row_offsets(block.indices_dev))
                block.committed = True
                return block
            counts = (lengths.to(torch.int64) - 1).clamp_min_(0)
            offsets = torch.cumsum(counts, 0) - counts
            total = self._token_total(counts)
            rows = torch.zeros((total, self._row_width), dtype=self.save_dtype, device=dev)
            if total:
                self.launch_deferred(rows, lengths=lengths, row_offsets=offsets)
            else:
                self._deferred.clear()
                self._deferred_adam.clear()
                self._deferred_full.clear()
        elif direct:
            self.launch_deferred(builder.device_rows, lengths=lengths, out_rows=block.indices_dev)
            block.committed = True
            return block
        else:
            rows = torch.empty((N, self._row_width), dtype=self.save_dtype, device=dev)
            self.launch_deferred(rows, lengths=lengths)
        block.rows = rows
        for name, (lo, hi) in column_offsets(self._grad_sizes).items():
            block[name] = rows[:, lo:hi]
        return block


@dataclass(kw_only=True)
class GradientCollector(_DeferredBatchMixin, HookCollectorBase):
    """Collects per-sample (or per-token) projected gradients and writes them to a store, or scores them."""

    persistent_hooks = True

    data: object
    cfg: IndexConfig
    mod_grads: dict = field(default_factory=dict)
    preprocess_cfg: PreprocessConfig = field(default_factory=PreprocessConfig)
    builder: Builder | None = None
    scorer: object | None = None
    skip_index: bool = False
    skip_padding: bool = False
    """Per-sequence mode only: do not read positions past each document's last label.  Exact for causal
    models with right padding (their output gradient is zero there); off by default because the
    reference reads every position."""
    device_store_bytes: int | None = None
    """HBM budget for keeping the whole store on the device (default: a quarter of the free memory)."""
    store_dtype: torch.dtype | None = None
    """Store dtype; None = the model's gradient dtype as in the reference.  (The reference's fp16 stores
    come from its training callback, bergson/huggingface.py:41.)"""

    def setup(self) -> None:
        grad_sizes = self._prepare_collection(self.store_dtype)
        self.save_index = self.scorer is None and not self.skip_index
        self.builder = None
        if self.save_index:
            self.builder = Builder(self.data, grad_sizes, self.save_dtype, self.preprocess_cfg,
                                   attribute_tokens=self.attribute_tokens,
                                   path=self.cfg.partial_run_path if self.cfg.run_path else None,
                                   device=self.model.device, device_store_bytes=self.device_store_bytes)

    @HookCollectorBase.split_attention_heads
    def backward_hook(self, module: nn.Module, g: Tensor):
        """Queues the module for the batch's fused launch."""
        name: str = module._name  # type: ignore[assignment]
        self.defer_module(module, g, self._column_of(name))

    def process_batch(self, indices: list[int], **kwargs):
        losses = kwargs.get("losses")
        assert losses is not None, "losses must be provided in kwargs"
        need_rows = self.scorer is not None or self.builder is None or self.preprocess_cfg.aggregation != "none"
        block = self._launch_batch(indices, self.builder, need_rows)
        self.mod_grads = block
        if self.builder:
            self.builder(indices, block)
        if self.scorer:
            self.scorer(indices, block)
        if self.builder or self.scorer:
            self.mod_grads = {}
        self._record_losses(indices, losses)

    def teardown(self):
        if dist.is_initialized():
            dist.reduce(self.per_doc_losses, dst=0)
        self.remove_hooks()
        if self.builder:
            self.builder.teardown()
        if self.rank == 0 and self.cfg.run_path:
            self._save_artifacts()

    def _save_artifacts(self) -> None:
        """data.hf (+ loss column) and the processor files next to the store (gradient_collectors.py:141-164)."""
        path = self.cfg.partial_run_path
        path.mkdir(parents=True, exist_ok=True)
        try:
            from datasets import Dataset, Value
        except Exception:  # pragma: no cover - datasets is optional
            Dataset = None
        if Dataset is not None:
            if self.preprocess_cfg.aggregation != "none":
                assert self.builder
                data = Dataset.from_list([{"query_index": i} for i in range(self.builder.grad_buffer.shape[0])])
            elif isinstance(self.data, Dataset):
                data = self.data
                if self.cfg.drop_columns and "input_ids" in data.column_names:
                    data = data.remove_columns(["input_ids"])
                data = data.add_column("loss", self.per_doc_losses.cpu().numpy(), feature=Value("float32"),
                                       new_fingerprint="loss")
            else:
                data = Dataset.from_dict({"loss": self.per_doc_losses.cpu().numpy()})
            data.save_to_disk(str(path / "data.hf"))
            self.data = data
        self.processor.save(path)


@dataclass(kw_only=True)
class TraceCollector(HookCollectorBase):
    """Accumulates per-sample gradients of arbitrary backward passes in lists, on `device`."""

    mod_grads: dict = field(default_factory=lambda: defaultdict(list))
    device: torch.device | str
    dtype: torch.dtype

    def setup(self) -> None:
        self.save_dtype = get_gradient_dtype(self.model)
        self.lo = torch.finfo(self.save_dtype).min
        self.hi = torch.finfo(self.save_dtype).max

    @HookCollectorBase.split_attention_heads
    def backward_hook(self, module: nn.Module, g: Tensor):
        name: str = module._name  # type: ignore[assignment]
        P = self._compute_gradient(module, g)
        self.mod_grads[name].append(P.to(self.device, self.dtype, non_blocking=True))

    def process_batch(self, indices: list[int], **kwargs):
        return

    def teardown(self):
        return


@dataclass(kw_only=True)
class StreamingGradientCollector(HookCollectorBase):
    """Per-step gradients in `mod_grads` for an external consumer (a training callback)."""

    mod_grads: dict = field(default_factory=dict)
    dtype: torch.dtype

    def setup(self) -> None:
        self.save_dtype = get_gradient_dtype(self.model)
        self.lo = torch.finfo(self.save_dtype).min
        self.hi = torch.finfo(self.save_dtype).max

    def teardown(self) -> None:
        pass

    def process_batch(self, indices: list[int], **kwargs) -> None:
        pass

    @HookCollectorBase.split_attention_heads
    def backward_hook(self, module: nn.Module, g: Tensor):
        name: str = module._name  # type: ignore[assignment]
        P = self._compute_gradient(module, g)
        self.mod_grads[name] = P.to(device="cpu", dtype=self.save_dtype, non_blocking=True)
