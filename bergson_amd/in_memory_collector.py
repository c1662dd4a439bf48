"""Collector that keeps the store in memory (bergson/collector/in_memory_collector.py:23-183).

Rows are written by the same fused launch as `GradientCollector`; after
`teardown()` the per-module tensors are in `.gradients` and, with a scorer,
the scores in `.scores`.  The autocorrelation statistics of the reference
(`skip_hessians=False`) belong to Hessian fitting and are not provided.
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
        assert isinstance(self.model.device, torch.device), "Model device is not set correctly"
        if not self.skip_hessians:
            raise NotImplementedError("autocorrelation statistics (skip_hessians=False) are outside this package")
        self.attribute_tokens = self.cfg.attribute_tokens
        if self.cfg.attribute_tokens:
            assert self.preprocess_cfg.aggregation == "none", "attribute_tokens is incompatible with reduce mode."
        self.save_dtype = get_gradient_dtype(self.model)
        self.lo = torch.finfo(self.save_dtype).min
        self.hi = torch.finfo(self.save_dtype).max
        self.per_doc_losses = torch.full((len(self.data),), device=self.model.device, dtype=torch.float32,
                                         fill_value=0.0)
        self.gradients = {}
        self.scores = None
        if self.builder is None and self.scorer is None:
            grad_sizes = {name: math.prod(s) for name, s in self.shapes().items()}
            self.builder = Builder(self.data, grad_sizes, self.save_dtype, self.preprocess_cfg,
                                   attribute_tokens=self.cfg.attribute_tokens, device=self.model.device)

    @HookCollectorBase.split_attention_heads
    def backward_hook(self, module: nn.Module, g: Tensor) -> None:
        name: str = module._name  # type: ignore[assignment]
        self.defer_module(module, g, self._column_of(name))

    def process_batch(self, indices: list[int], **kwargs) -> None:
        losses = kwargs.get("losses")
        assert losses is not None, "losses must be provided in kwargs"
        need_rows = self.scorer is not None or self.preprocess_cfg.aggregation != "none"
        block = self._launch_batch(indices, self.builder, need_rows)
        if self.builder is not None:
            self.builder(indices, block)
        if self.scorer is not None:
            self.scorer(indices, block)
        self.per_doc_losses[indices] = losses.detach().type_as(self.per_doc_losses)

    def teardown(self) -> None:
        self.remove_hooks()
        if dist.is_initialized():
            dist.reduce(self.per_doc_losses, dst=0)
        grad_sizes = {name: math.prod(s) for name, s in self.shapes().items()}
        if self.builder is not None:
            self.builder.teardown()
            buf = self.builder.grad_buffer
            offset = 0
            for name, dim in grad_sizes.items():
                self.gradients[name] = numpy_to_tensor(buf[:, offset:offset + dim], self.builder.base_dtype)
                offset += dim
        if self.scorer is not None:
            self.scores = self.scorer.writer.scores
