"""Collector that keeps the store in memory (bergson/collector/in_memory_collector.py:23-183).

Rows are written by the same fused launch as `GradientCollector`; after
`teardown()` the per-module tensors are in `.gradients` and, with a scorer,
the scores in `.scores`.  With `skip_hessians=False` every batch's rows are also
added into the per-module autocorrelation Grams `P^T P` (fp32, one fused launch
for all modules), which `teardown()` normalises and attaches to the processor.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
import torch.distributed as dist
import torch.nn as nn
from torch import Tensor

from .builder import Builder
from .collector import HookCollectorBase
from .config import IndexConfig, PreprocessConfig
from .gradient_collectors import _DeferredBatchMixin
from .utils import get_gradient_dtype, numpy_to_tensor


@dataclass(kw_only=True)
class InMemoryCollector(_DeferredBatchMixin, HookCollectorBase):
    persistent_hooks = True

    data: object
    cfg: IndexConfig
    skip_hessians: bool = True
    mod_grads: dict = field(default_factory=dict)
    preprocess_cfg: PreprocessConfig = field(default_factory=PreprocessConfig)
    builder: Builder | None = None
    scorer: object | None = None
    gradients: dict[str, Tensor] = field(default_factory=dict)
    scores: object | None = None
    skip_padding: bool = False

    def __post_init__(self):
        if self.filter_modules is None:
            self.filter_modules = self.cfg.filter_modules
        super().__post_init__()

    def setup(self) -> None:
        if not self.skip_hessians and self.processor.projection_target == "global":
            raise NotImplementedError("autocorrelation statistics of a global projection")
        self._gram_blocks = None
        grad_sizes = self._prepare_collection()
        self.gradients, self.scores = {}, None
        if self.builder is None and self.scorer is None:  # rows stay in memory: a Builder without a path
            self.builder = Builder(self.data, grad_sizes, self.save_dtype, self.preprocess_cfg,
                                   attribute_tokens=self.attribute_tokens, device=self.model.device)

    @HookCollectorBase.split_attention_heads
    def backward_hook(self, module: nn.Module, g: Tensor) -> None:
        name: str = module._name  # type: ignore[assignment]
        self.defer_module(module, g, self._column_of(name))

    def process_batch(self, indices: list[int], **kwargs) -> None:
        losses = kwargs.get("losses")
        assert losses is not None, "losses must be provided in kwargs"
        need_rows = (self.scorer is not None or self.preprocess_cfg.aggregation != "none"
                     or not self.skip_hessians)
        block = self._launch_batch(indices, self.builder, need_rows)
        if not self.skip_hessians and block.rows is not None:
            self._accumulate_grams(block.rows)
        if self.builder is not None:
            self.builder(indices, block)
        if self.scorer is not None:
            self.scorer(indices, block)
        self._record_losses(indices, losses)

    def _accumulate_grams(self, rows: Tensor) -> None:
        """hessians[name] += P.float().T @ P.float() for every module (in_memory_collector.py:149-154)."""
        from . import ops
        from .data import column_offsets

        if self._gram_blocks is None:
            sizes = {name: math.prod(s) for name, s in self.shapes().items()}
            self._gram_blocks = []
            for name, (lo, hi) in column_offsets(sizes).items():
                h = self.processor.hessians.get(name)
                if h is None or h.device != rows.device or h.dtype != torch.float32 or not h.is_contiguous():
                    h0 = torch.zeros((hi - lo, hi - lo), dtype=torch.float32, device=rows.device)
                    if h is not None:
                        h0.copy_(h)
                    h = self.processor.hessians[name] = h0
                self._gram_blocks.append((h, lo))
        ops.gram_accumulate(rows, self._gram_blocks)

    def num_rows(self) -> int:
        """Rows summed into the Grams: documents, or gradient-carrying tokens with attribute_tokens."""
        if self.cfg.attribute_tokens:
            from .data import compute_num_token_grads

            return int(compute_num_token_grads(self.data).sum())
        return len(self.data)

    def teardown(self) -> None:
        """Detaches from the model, finishes the autocorrelation statistics and exposes what was gathered:
        `gradients[name]` = the module's columns of the in-memory store, `scores` = the scorer's."""
        self.remove_hooks()
        if dist.is_initialized():
            dist.reduce(self.per_doc_losses, dst=0)
        widths = {name: math.prod(shape) for name, shape in self.shapes().items()}
        if not self.skip_hessians and self.processor.hessians:
            from .hessians import process_autocorrelation_matrices

            if dist.is_initialized() and dist.get_world_size() > 1:
                raise NotImplementedError("autocorrelation statistics across ranks")
            process_autocorrelation_matrices(self.processor, self.processor.hessians, self.num_rows(), widths)
        if self.builder is not None:
            from .data import column_offsets

            self.builder.teardown()
            rows = self.builder.grad_buffer
            self.gradients.update({name: numpy_to_tensor(rows[:, lo:hi], self.builder.base_dtype)
                                   for name, (lo, hi) in column_offsets(widths).items()})
        if self.scorer is not None:
            self.scores = self.scorer.writer.scores
