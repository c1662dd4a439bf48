"""Hook layer of gradient collection, backed by the fused HIP kernels.

Mirrors the interface of bergson/collector/collector.py: `HookCollectorBase`
(:44-768: target discovery, per-head splitting, hook registration, the
`with collector.with_batch(mask):` protocol, `shapes()`), `CollectorComputer`
(:771-923), `fwd_bwd_factory` (:926-985) and `create_projection_matrix`
(:1029-1063).

What differs from the reference is where the arithmetic happens.  The
reference's forward hook scales and projects the activations and its backward
hook scales, projects and reduces the output gradients, each as a handful of
PyTorch ops per module.  Here the forward hook only keeps a reference to the
module input; the backward hook hands (a, g) to one fused kernel launch --
either immediately (`_compute_gradient`, one module per launch, returns the
tensor the reference would) or deferred (`defer_module` + `launch_deferred`,
all modules of the batch in one launch writing straight into a row buffer).
"""
from __future__ import annotations

import functools
import hashlib
import math
import os
from abc import ABC, abstractmethod
from contextlib import ContextDecorator, nullcontext
from dataclasses import dataclass, field
from fnmatch import fnmatchcase
from typing import Callable, Literal, Mapping, Optional

import numpy as np
import torch
import torch.distributed as dist
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor
from torch.utils.hooks import RemovableHandle

from . import ops
from .config import AttentionConfig, IndexConfig
from .data import compute_num_token_grads, pad_and_tensor
from .gradients import AdafactorNormalizer, AdamNormalizer, GradientProcessor, LayerAdapter


def create_projection_matrix(identifier: str, m: int, n: int, dtype: torch.dtype, device: torch.device | str,
                             projection_type: Literal["normal", "rademacher"] = "normal",
                             projection_scale: Literal["jl", "row_norm"] = "jl") -> Tensor:
    """Deterministic [m, n] projection matrix named by `identifier` (collector.py:1029-1063).

    The seed is md5(identifier) mod 2**63-1.  `normal` draws `torch.randn` in `dtype`; the draw always
    uses the CPU generator and is uploaded afterwards, so a matrix depends on (identifier, shape, dtype)
    only and equals what the reference produces with device='cpu' on any machine.  `rademacher` uses
    numpy's PCG64 bit stream exactly as the reference does.
    """
    digest = hashlib.md5(bytes(identifier, "utf-8")).digest()
    seed = int.from_bytes(digest, byteorder="big") % (2**63 - 1)
    if projection_type == "normal":
        prng = torch.Generator("cpu").manual_seed(seed)
        A = torch.randn(m, n, dtype=dtype, generator=prng)
    elif projection_type == "rademacher":
        random_bytes = np.random.Generator(np.random.PCG64(seed)).bytes((m * n + 7) // 8)
        bits = np.unpackbits(np.frombuffer(random_bytes, dtype=np.uint8))[: m * n].reshape((m, n))
        A = torch.from_numpy(bits).to(dtype=dtype)
        A = A.add_(-0.5).mul_(2)
    else:
        raise ValueError(f"Unknown projection type: {projection_type}")
    if projection_scale == "row_norm":
        A /= A.norm(dim=1, keepdim=True)
    else:
        A /= math.sqrt(m)  # variance 1/m
    return A.to(device)


@dataclass(frozen=True)
class GradBlock:
    """One block of store columns: the gradient of a whole module, or of one attention head of it."""

    name: str  # key in shapes(), in the normalizers of a head-wise processor and in the projection cache
    module: str  # the hooked module the block belongs to
    head: int | None  # None for a whole module
    first: int  # first output feature of the block
    width: int  # number of output features
    axis: int  # dimension of g the output features lie on (heads only)
    weight_shape: torch.Size  # [O, I (+1)] of the block when nothing is projected


class HeadView:
    """Stands in for a hooked module while one of its attention heads is processed: `_name` is the head's
    name, the module's output-feature attribute reads as the head's width, everything else (the kept input,
    the bias flag, the input width, the module's type for isinstance checks) is the module's own."""

    __slots__ = ("_hv_module", "_hv_block", "_hv_width_attr")

    def __init__(self, module: nn.Module, block: GradBlock):
        object.__setattr__(self, "_hv_module", module)
        object.__setattr__(self, "_hv_block", block)
        object.__setattr__(self, "_hv_width_attr", LayerAdapter.out_attr(module))

    @property
    def __class__(self):  # isinstance(view, nn.Linear) answers for the module
        return type(self._hv_module)

    def __getattr__(self, key):
        if key == "_name":
            return self._hv_block.name
        if key == self._hv_width_attr:
            return self._hv_block.width
        return getattr(self._hv_module, key)

    def __setattr__(self, key, value):
        setattr(self._hv_module, key, value)

    def __delattr__(self, key):
        delattr(self._hv_module, key)


@dataclass
class HookCollectorBase(ContextDecorator, ABC):
    """Attaches forward and backward hooks to the supported layers of `model`.

    Activations are [N, S, I], activation gradients [N, S, O].  Subclasses implement `setup`, `teardown`,
    `backward_hook` and `process_batch` (collector.py:493-516, :745-768).
    """

    model: nn.Module
    filter_modules: str | None = None
    target_modules: set[str] | None = None
    processor: GradientProcessor = field(default_factory=GradientProcessor)
    attention_cfgs: dict[str, AttentionConfig] = field(default_factory=dict)
    attribute_tokens: bool = False
    lo: float = float("-inf")
    hi: float = float("inf")
    mod_grads: dict = field(default_factory=dict)
    save_dtype: torch.dtype = torch.float32

    persistent_hooks = False
    """When True the forward hooks stay registered between `with` blocks (they do nothing while no block is
    open) and are removed by `remove_hooks()`; saves re-registering every hook for every batch."""

    def __post_init__(self):
        self.rank = dist.get_rank() if dist.is_initialized() else 0
        self.world_size = dist.get_world_size() if dist.is_initialized() else 1
        self._fwd_hooks: list[RemovableHandle] = []
        self._bwd_hooks: list[RemovableHandle] = []
        self._current_collection_mask: Tensor | None = None
        self._current_doc_lengths: list[int] | None = None
        self._deferred: list = []
        self._prepared: dict[str, ops.PreparedModule] = {}
        self._adam_prepared: dict[str, ops.AdamPrepared] = {}
        self._deferred_adam: list = []
        self._deferred_full: list = []  # unprojected / global-projection modules: (FullGradModule, name, a, g)
        self._full_prepared: dict = {}
        self._active = False
        self._recording: BatchRecord | None = None
        self._scale_cache: dict[str, tuple[Tensor | None, Tensor | None]] = {}
        self.target_info = self.discover_targets(self.model, self.target_modules, self.processor.include_bias,
                                                 self.filter_modules)
        if unknown := set(self.attention_cfgs) - set(self.target_info):
            raise ValueError(f"attention_cfgs contains module names not found in the model: {unknown}. "
                             f"Available modules: {set(self.target_info)}")
        self.setup()

    # ---- discovery and naming (collector.py:133-241) -----------------------------------
    @staticmethod
    def discover_targets(model: nn.Module, target_modules: set[str] | None = None, include_bias: bool = False,
                         filter_modules: str | None = None) -> dict[str, tuple[torch.device, torch.Size, bool]]:
        """name -> (device, weight shape [O, I], collect_bias) for every supported layer."""
        target_info = {}
        for name, layer in model.named_modules():
            if not isinstance(layer, LayerAdapter.supported_modules):
                continue
            if target_modules is not None and name not in target_modules:
                continue
            if filter_modules and any(fnmatchcase(name, pat.strip()) for pat in filter_modules.split(",")):
                continue
            collect_bias = getattr(layer, "bias", None) is not None and include_bias
            o = getattr(layer, LayerAdapter.out_attr(layer))
            i = getattr(layer, LayerAdapter.in_attr(layer))
            target_info[name] = (layer.weight.device, torch.Size([o, i]), collect_bias)
        return target_info

    # ---- column blocks: whole modules and attention heads (collector.py:185-334) --------------------------
    @staticmethod
    def get_head_name(name: str, head_idx: int) -> str:
        return f"{name}.head_{head_idx}"

    @staticmethod
    def split_head_name(name: str) -> tuple[str, int] | None:
        """("<module>", h) for "<module>.head_<h>", None for any other name."""
        base, sep, suffix = name.rpartition(".head_")
        return (base, int(suffix)) if sep and suffix.isdigit() else None

    def _plan_blocks(self) -> dict[str, tuple["GradBlock", ...]]:
        """module name -> the column blocks its gradient is stored as, in store order: one block for an
        ordinary module; for a module listed in `attention_cfgs`, one per head, each covering `head_size`
        consecutive output features along dimension `head_dim` of g.  Every block becomes one descriptor
        of the batch's fused launch: a head's descriptor points `first` features into the rows of g and
        carries its own output column, so splitting costs no copy and no extra launch."""
        plan: dict[str, tuple[GradBlock, ...]] = {}
        for name, (_, weight_shape, with_bias) in self.target_info.items():
            dims = [int(d) for d in weight_shape]
            cfg = self.attention_cfgs.get(name)
            if cfg is None:
                heads: list[tuple[int | None, int, int]] = [(None, 0, dims[0])]
                axis = -1
            else:
                heads = [(h, h * cfg.head_size, cfg.head_size) for h in range(cfg.num_heads)]
                axis = cfg.head_dim
                dims[axis - 2] = cfg.head_size  # g is [N, S, ...]: its dimension `axis` is dimension `axis - 2` of the weight
            if with_bias:
                dims[-1] += 1
            plan[name] = tuple(GradBlock(name if h is None else self.get_head_name(name, h), name, h, first, width,
                                         axis, torch.Size(dims)) for h, first, width in heads)
        return plan

    def blocks_of(self, module_name: str) -> tuple["GradBlock", ...]:
        plan = self.__dict__.get("_blocks")
        if plan is None or module_name not in plan:
            plan = self._blocks = self._plan_blocks()
        return plan[module_name]

    @staticmethod
    def split_attention_heads(fn):
        """Decorator for `backward_hook(self, module, g)`: a module listed in `attention_cfgs` is handed to
        `fn` once per head (collector.py:191-233), as a `HeadView` of the module -- an object that answers
        `_name` with the head's name and the output-feature count with the head's width and passes every
        other attribute through -- together with the head's columns of g (a strided view).  The module
        itself is never modified, so an exception inside `fn` leaves nothing to restore."""

        @functools.wraps(fn)
        def per_block(self, module, g):
            blocks = self.blocks_of(module._name)
            if blocks[0].head is None:
                return fn(self, module, g)
            covered = sum(b.width for b in blocks)
            features = getattr(module, LayerAdapter.out_attr(module))
            if covered != features:
                raise AssertionError(f"{module._name}: {len(blocks)} heads of {blocks[0].width} features make "
                                     f"{covered}, the module has {features} output features")
            for block in blocks:
                try:
                    g_head = g.narrow(block.axis, block.first, block.width)
                except Exception:
                    cfg = self.attention_cfgs[module._name]
                    print(f"{module._name}: cannot take head {block.head} out of a gradient of shape "
                          f"{tuple(g.shape)} with {cfg}; the head configuration may be wrong.")
                    raise
                fn(self, HeadView(module, block), g_head)

        return per_block

    def normalizer_for(self, name: str):
        """The normalizer registered under `name`; for an attention head, its rows of the normalizer that is
        registered under the module's name (collector.py:243-279)."""
        registered = self.processor.normalizers
        own = registered.get(name)
        if own is not None:
            return own
        parsed = self.split_head_name(name)
        if parsed is None:
            return None
        whole = registered.get(parsed[0])
        cfg = self.attention_cfgs.get(parsed[0])
        if whole is None or cfg is None:
            return whole
        rows = slice(parsed[1] * cfg.head_size, (parsed[1] + 1) * cfg.head_size)
        cut = lambda t: None if t is None else t[rows]  # noqa: E731
        if isinstance(whole, AdafactorNormalizer):  # the column moments belong to the shared input side
            return AdafactorNormalizer(cut(whole.row), whole.col, cut(whole.bias_avg_sq))
        if isinstance(whole, AdamNormalizer):
            return AdamNormalizer(cut(whole.weight_avg_sq), cut(whole.bias_avg_sq))
        return whole

    @property
    def per_module_projection_dim(self) -> int | None:
        if self.processor.projection_target == "global":
            return None
        return self.processor.projection_dim or None

    def shapes(self) -> Mapping[str, torch.Size]:
        """Shape of every stored block, in the column order of the store (collector.py:288-334): one
        "gradients" vector in global mode, [p, p] per block when projecting per module, else the block's
        [O, I (+1)] weight shape."""
        if self.processor.projection_target == "global":
            assert self.processor.projection_dim is not None
            return {"gradients": torch.Size((self.processor.projection_dim,))}
        p = self.per_module_projection_dim
        return {block.name: block.weight_shape if p is None else torch.Size((p, p))
                for blocks in self._plan_blocks().values() for block in blocks}

    def projection(self, name: str, m: int, n: int, role: Literal["left", "right", "single"],
                   device: torch.device, dtype: torch.dtype) -> Tensor:
        """The cached `role` projection matrix [m, n] of parameter `name` (collector.py:336-362)."""
        key = (name, role, device)
        cache = self.processor._projection_matrices
        if key in cache:
            return cache[key]
        A = create_projection_matrix(f"{name}/{role}", m, n, dtype, device, self.processor.projection_type,
                                     self.processor.projection_scale)
        cache[key] = A
        return A

    def num_rows(self, data) -> int:
        if self.attribute_tokens:
            return int(compute_num_token_grads(data).sum())
        return len(data)

    # ---- batch protocol (collector.py:413-491) -------------------------------------------
    def with_batch(self, collection_mask: Tensor | None = None, doc_lengths: list[int] | None = None
                   ) -> "HookCollectorBase":
        """Sets the [N, S] mask of collected positions (every real position but each sequence's last).
        `doc_lengths`: the documents' lengths as the host knows them; with them the number of per-token rows
        of the batch needs no read-back from the device."""
        self._current_collection_mask = collection_mask
        self._current_doc_lengths = doc_lengths
        return self

    def __enter__(self):
        """Activates collection.  A forward hook on every target keeps the module input and attaches a
        tensor hook to the module output; that hook receives the gradient with respect to the output --
        what the reference's full backward hook passes as grad_output[0] (collector.py:435-472) -- without
        the extra autograd nodes a module-level backward hook inserts around every call."""
        if not self._fwd_hooks:
            for name in self.target_info:
                layer = self.model.get_submodule(name)
                layer._name = name  # type: ignore[attr-defined]
                layer._collect_bias = self.target_info[name][2]  # type: ignore[attr-defined]
                self._fwd_hooks.append(layer.register_forward_hook(self._process_input))
            self._target_layers = [self.model.get_submodule(name) for name in self.target_info]
        self._active = True
        return self

    def _process_input(self, module: nn.Module, inp: tuple, out):
        if not self._active:
            return
        x = inp[0].detach()
        assert x.ndim == 3, f"Expected input of shape [N, S, I], got {x.shape}"
        self.forward_hook(module, x)
        if isinstance(out, Tensor) and out.requires_grad:
            rec = self._recording
            if rec is not None:
                # the gradient of `out` is asked of autograd by whoever runs the backward pass
                # (`replay_backward`); no Python runs during that pass
                rec.entries.append((module, getattr(module, "_inputs", None), out))
                rec.versions.append(out._version)
            else:
                out.register_hook(functools.partial(self._on_output_grad, module))

    def _on_output_grad(self, module: nn.Module, grad: Tensor) -> None:
        if self._active:
            self._process_grad(module, None, (grad,))

    def _process_grad(self, module: nn.Module, _, grad_out):
        assert isinstance(module, LayerAdapter.supported_modules), (
            f"Expected a module of type {LayerAdapter.supported_modules}, got {type(module)}")
        g = grad_out[0].detach()
        self.backward_hook(module, g)
        if hasattr(module, "_inputs"):
            del module._inputs

    # ---- recorded batches: the backward pass without Python hooks ---------------------------------
    def begin_recording(self, collection_mask: Tensor | None = None, doc_lengths: list[int] | None = None
                        ) -> "BatchRecord":
        """Until `end_recording`, forward hooks list (module, kept input, module output) in the returned
        record instead of attaching tensor hooks.  The caller obtains the gradients of
        `record.outputs()` from autograd (e.g. `torch.autograd.grad`, possibly on another thread while the
        next batch's forward pass runs here) and hands them to `replay_backward`."""
        self._recording = BatchRecord(collection_mask, doc_lengths)
        return self._recording

    def end_recording(self) -> None:
        self._recording = None

    def replay_backward(self, record: "BatchRecord", grads) -> None:
        """Calls `backward_hook(module, g)` for every module call of `record`, last call first -- the
        order and arguments a backward pass with tensor hooks would have produced (collector.py:435-472)."""
        assert len(grads) == len(record.entries), (len(grads), len(record.entries))
        self._current_collection_mask = record.mask
        self._current_doc_lengths = record.doc_lengths
        for (module, kept, _out), g in zip(reversed(record.entries), reversed(grads)):
            if g is None:  # the loss does not depend on this call's output
                continue
            if kept is not None:
                module._inputs = kept
            self._process_grad(module, None, (g,))
        record.entries.clear()

    def invalidate_prepared(self) -> None:
        """Forget everything derived from the processor's normalizers (folded factor vectors, Adam tables):
        call after replacing `processor.normalizers`, e.g. from live optimizer state."""
        self._prepared.clear()
        self._adam_prepared.clear()
        self._full_prepared.clear()
        self._scale_cache.clear()

    def remove_hooks(self) -> None:
        """Detach from the model: remove the hooks and the attributes set on the target layers."""
        for h in self._fwd_hooks:
            h.remove()
        self._fwd_hooks.clear()
        for layer in getattr(self, "_target_layers", []):
            for attr in ("_inputs", "_name", "_collect_bias"):
                if hasattr(layer, attr):
                    delattr(layer, attr)
        self._active = False

    def __exit__(self, exc_type, exc, tb):
        self._active = False
        for layer in getattr(self, "_target_layers", []):
            if hasattr(layer, "_inputs"):
                del layer._inputs
        if not self.persistent_hooks:
            self.remove_hooks()
        if exc_type is not None:  # a failed batch leaves nothing queued; otherwise process_batch launches
            self._deferred.clear()
            self._deferred_adam.clear()
            self._deferred_full.clear()
        return False

    # ---- the hook pair -----------------------------------------------------------------------
    def forward_hook(self, module: nn.Module, a: Tensor) -> None:
        """Keeps the module input for the backward hook (collector.py:518-543).

        The reference scales and projects `a` here; the fused kernel does both when it also has g, so the
        raw input is kept alive until then.
        """
        module._inputs = a

    def _batch_lengths(self, device: torch.device) -> Tensor | None:
        """int32 [N] document lengths implied by the collection mask (mask[n, s] = s + 1 < len[n])."""
        mask = self._current_collection_mask
        if mask is None:
            return None
        cached = getattr(self, "_lengths_cache", None)
        if cached is not None and cached[0] is mask:
            return cached[1]
        lengths = (mask.sum(dim=1) + 1).to(device=device, dtype=torch.int32)
        self._lengths_cache = (mask, lengths)
        return lengths

    def _scales(self, name: str, normalizer: AdafactorNormalizer, dtype: torch.dtype, device: torch.device):
        key = f"{name}|{dtype}|{device}"
        if key not in self._scale_cache:
            self._scale_cache[key] = ops.adafactor_scales(normalizer.row.to(device), normalizer.col.to(device), dtype)
        return self._scale_cache[key]

    def module_input(self, module: nn.Module, g: Tensor, out_col: int = 0) -> ops.ModuleInput:
        """Kernel operands of `module` for the current batch: its kept input, g, the two projection matrices
        and, with an Adafactor normalizer, the two factor vectors."""
        a = module._inputs
        assert isinstance(a, Tensor), "Activation cache missing for module"
        name: str = module._name  # type: ignore[assignment]
        p = self.per_module_projection_dim
        i = getattr(module, LayerAdapter.in_attr(module))
        o = getattr(module, LayerAdapter.out_attr(module))
        normalizer = self.normalizer_for(name)
        if p is None:
            raise NotImplementedError(
                "bergson_amd collects projected gradients only: set processor.projection_dim "
                "(projection_target='per_module'); unprojected [O, I] gradients have no HIP kernel here")
        if isinstance(normalizer, AdamNormalizer):
            raise AssertionError("Adam modules go through adam_prepared()")
        if not a.is_cuda or not g.is_cuda:
            raise RuntimeError("bergson_amd has no CPU path: the model must run on the GPU")
        r_out = self.projection(name, p, o, "left", g.device, g.dtype)
        bias_col = bias_scale = None
        if module._collect_bias:
            # with a bias the right projection has I + 1 columns and is named after the (head) module
            # itself (collector.py:552-590); its last column multiplies the bias gradient
            right = self.projection(name, p, i + 1, "right", a.device, a.dtype)
            key = f"{name}|split|{a.dtype}"
            if key not in self._scale_cache:
                self._scale_cache[key] = (right[:, :i].contiguous(), right[:, i].float().contiguous())
            r_in, bias_col = self._scale_cache[key]
        else:
            # an attention head shares the parent's input and right projection (collector.py:527, :540)
            parent = self.split_head_name(name)
            right_name = parent[0] if parent is not None and parent[0] in self.attention_cfgs else name
            r_in = self.projection(right_name, p, i, "right", a.device, a.dtype)
        row_scale = col_scale = None
        if isinstance(normalizer, AdafactorNormalizer):
            row_scale, col_scale = self._scales(name, normalizer, g.dtype, g.device)
            if module._collect_bias:
                assert normalizer.bias_avg_sq is not None, f"{name}: bias collected but the normalizer has no bias_avg_sq"
                key = f"{name}|bias|{g.device}"
                if key not in self._scale_cache:
                    # rsqrt(bias_avg_sq + 1e-8), eps inside the root (gradients.py:339-349)
                    self._scale_cache[key] = (normalizer.bias_avg_sq.to(g.device, torch.float32).add(1e-8).rsqrt()
                                              .contiguous(), None)
                bias_scale = self._scale_cache[key][0]
        return ops.ModuleInput(a=a, g=g, r_in=r_in, r_out=r_out, out_col=out_col, col_scale=col_scale,
                               row_scale=row_scale, bias_col=bias_col, bias_scale=bias_scale)

    def full_prepared(self, module: nn.Module, g: Tensor, out_col: int) -> "ops.FullGradModule":
        """Normaliser vectors of `module` for the unprojected path (collector.py:609-742 with p = None)."""
        name: str = module._name  # type: ignore[assignment]
        key = f"{name}|{g.dtype}|{out_col}"
        prep = self._full_prepared.get(key)
        if prep is not None:
            return prep
        if not g.is_cuda:
            raise RuntimeError("bergson_amd has no CPU path: the model must run on the GPU")
        i = getattr(module, LayerAdapter.in_attr(module))
        o = g.shape[-1]  # an attention head sees its own slice of the output features
        normalizer = self.normalizer_for(name)
        bias = bool(module._collect_bias)
        prep = ops.FullGradModule(O=o, I=i, out_col=out_col, collect_bias=bias)
        f32 = dict(device=g.device, dtype=torch.float32)
        if isinstance(normalizer, AdamNormalizer):
            prep.adam_v = normalizer.weight_avg_sq.detach().to(**f32).contiguous()
            if bias:
                assert normalizer.bias_avg_sq is not None, f"{name}: bias collected but the normalizer has no bias_avg_sq"
                # 1 / (sqrt(bias_avg_sq) + 1e-8), eps outside the root (gradients.py:390-400)
                prep.bias_scale = (normalizer.bias_avg_sq.detach().to(**f32).sqrt() + 1e-8).reciprocal().contiguous()
        elif isinstance(normalizer, AdafactorNormalizer):
            prep.row_scale, prep.col_scale = self._scales(name, normalizer, g.dtype, g.device)
            if bias:
                assert normalizer.bias_avg_sq is not None, f"{name}: bias collected but the normalizer has no bias_avg_sq"
                # rsqrt(bias_avg_sq + 1e-8), eps inside the root (gradients.py:339-349)
                prep.bias_scale = normalizer.bias_avg_sq.detach().to(**f32).add(1e-8).rsqrt().contiguous()
        self._full_prepared[key] = prep
        return prep

    def _token_rows(self, device: torch.device):
        """(lengths, per-document token counts, offsets of each document's first row, total rows)."""
        lengths = self._batch_lengths(device)
        assert lengths is not None, "attribute_tokens needs a collection mask (with_batch)"
        counts = (lengths.to(torch.int64) - 1).clamp_min_(0)
        offsets = torch.cumsum(counts, 0) - counts
        return lengths, counts, offsets, self._token_total(counts)

    def _token_total(self, counts: Tensor) -> int:
        """Per-token rows of the current batch: from the host's document lengths when the loop supplied them
        (`with_batch(mask, doc_lengths)`), else read back from the device (one synchronisation)."""
        host = self._current_doc_lengths
        if host is not None and len(host) == counts.numel():
            return sum(max(int(n) - 1, 0) for n in host)
        return int(counts.sum().item())

    def _global_projection(self, items: list, out: Tensor, lengths: Tensor | None, out_rows: Tensor | None,
                           row_offsets: Tensor | None) -> None:
        """projection_target = "global" (collector.py:364-402): every module's clamped, flattened gradient
        times its block of the single projection matrix, summed over the modules into columns
        [0, projection_dim) of the output rows.  The sum over modules is kept in fp32 (the reference adds
        in the model dtype) and cast once."""
        pd = self.processor.projection_dim
        assert pd is not None
        g0 = items[0][3]
        N = g0.shape[0]
        if self.attribute_tokens:
            lens, counts, local, total = self._token_rows(g0.device)
            n_rows = total
        else:
            lens, counts, local, n_rows = lengths, None, None, N
        if n_rows == 0:
            return
        acc = torch.zeros((n_rows, pd), dtype=torch.float32, device=g0.device)
        for prep, name, a, g in items:
            tmp = torch.empty((n_rows, prep.width), dtype=g.dtype, device=g.device)
            ops.full_gradient(prep, a, g, tmp, per_token=self.attribute_tokens, lengths=lens,
                              rows=local if self.attribute_tokens else None, lo=self.lo, hi=self.hi)
            R = self.projection(name, pd, prep.width, "single", g.device, g.dtype)
            ops.project_rows(tmp, R, acc)
        res = acc.to(out.dtype)
        if self.attribute_tokens:
            assert row_offsets is not None and counts is not None and local is not None
            dst = torch.repeat_interleave(row_offsets.to(torch.int64) - local, counts) + torch.arange(
                n_rows, device=out.device)
            out[:, :pd].index_copy_(0, dst, res)
        elif out_rows is not None:
            out[:, :pd].index_copy_(0, out_rows, res)
        else:
            out[:n_rows, :pd].copy_(res)

    def adam_prepared(self, module: nn.Module, g: Tensor, out_col: int) -> "ops.AdamPrepared":
        """The module's Adam table and projections, built on its first batch (collector.py:609-644)."""
        name: str = module._name  # type: ignore[assignment]
        key = f"{name}|{g.dtype}|{out_col}"
        prep = self._adam_prepared.get(key)
        if prep is not None:
            return prep
        p = self.per_module_projection_dim
        if p is None:
            raise NotImplementedError("bergson_amd collects projected gradients only: set processor.projection_dim")
        if not g.is_cuda:
            raise RuntimeError("bergson_amd has no CPU path: the model must run on the GPU")
        normalizer = self.normalizer_for(name)
        assert isinstance(normalizer, AdamNormalizer)
        i = getattr(module, LayerAdapter.in_attr(module))
        o = getattr(module, LayerAdapter.out_attr(module))
        r_out = self.projection(name, p, o, "left", g.device, g.dtype)
        if module._collect_bias:
            # the projection runs on [grad | bias_grad]: I + 1 columns, named after the module itself
            # (collector.py:626-644)
            assert normalizer.bias_avg_sq is not None, f"{name}: bias collected but the normalizer has no bias_avg_sq"
            right = self.projection(name, p, i + 1, "right", g.device, g.dtype)
            prep = ops.AdamPrepared(right[:, :i].contiguous(), r_out, normalizer.weight_avg_sq, out_col,
                                    bias_col=right[:, i], bias_avg_sq=normalizer.bias_avg_sq)
        else:
            # the Adam branch projects in the backward hook, under the name the module carries there: for a
            # split attention module every head has a right projection of its own, "<module>.head_h/right"
            # (collector.py:545-550, :626-644), unlike the other branches, whose input side is projected in
            # the forward hook under the parent's name
            r_in = self.projection(name, p, i, "right", g.device, g.dtype)
            prep = ops.AdamPrepared(r_in, r_out, normalizer.weight_avg_sq, out_col)
        self._adam_prepared[key] = prep
        return prep

    def _compute_gradient(self, module: nn.Module, g: Tensor) -> Tensor:
        """Per-sample [N, p*p] (or per-token [n_valid, p*p]) projected gradient of one module, clamped to
        [lo, hi], in the model dtype (collector.py:592-743) -- one fused launch."""
        p = self.per_module_projection_dim
        N, S = g.shape[:2]
        if p is None:
            # weight-shaped gradient [O, I (+1)] per sample or per token
            fp = self.full_prepared(module, g, 0)
            a = module._inputs
            assert isinstance(a, Tensor), "Activation cache missing for module"
            if self.attribute_tokens:
                lengths, _, offsets, total = self._token_rows(g.device)
                out = torch.empty((total, fp.width), dtype=g.dtype, device=g.device)
                if total:
                    ops.full_gradient(fp, a, g, out, per_token=True, lengths=lengths, rows=offsets, lo=self.lo,
                                      hi=self.hi)
                return out
            out = torch.empty((N, fp.width), dtype=g.dtype, device=g.device)
            ops.full_gradient(fp, a, g, out, per_token=False, lengths=None, rows=None, lo=self.lo, hi=self.hi)
            return out
        if isinstance(self.normalizer_for(module._name), AdamNormalizer):
            prep = self.adam_prepared(module, g, 0)
            a = module._inputs
            if self.attribute_tokens:
                lengths = self._batch_lengths(g.device)
                assert lengths is not None, "attribute_tokens needs a collection mask (with_batch)"
                counts = (lengths.to(torch.int64) - 1).clamp_min_(0)
                offsets = torch.cumsum(counts, 0) - counts
                out = torch.empty((self._token_total(counts), p * p), dtype=g.dtype, device=g.device)
                if out.shape[0]:
                    ops.collect_adam(prep, a, g, out, per_token=True, lengths=lengths, rows=offsets, lo=self.lo,
                                     hi=self.hi)
                return out
            out = torch.empty((N, p * p), dtype=g.dtype, device=g.device)
            ops.collect_adam(prep, a, g, out, per_token=False, lengths=None, rows=None, lo=self.lo, hi=self.hi)
            return out
        mi = self.module_input(module, g, 0)
        assert p is not None
        if self.attribute_tokens:
            lengths = self._batch_lengths(g.device)
            assert lengths is not None, "attribute_tokens needs a collection mask (with_batch)"
            counts = (lengths.to(torch.int64) - 1).clamp_min_(0)
            offsets = torch.cumsum(counts, 0) - counts
            total = self._token_total(counts)
            out = torch.empty((total, p * p), dtype=g.dtype, device=g.device)
            if total:
                ops.collect_tok([mi], p, out, lengths=lengths, row_offsets=offsets, lo=self.lo, hi=self.hi)
            return out
        out = torch.empty((N, p * p), dtype=g.dtype, device=g.device)
        ops.collect_seq([mi], p, out, lo=self.lo, hi=self.hi)
        return out

    # ---- deferred (one launch per batch) -----------------------------------------------------
    def defer_module(self, module: nn.Module, g: Tensor, out_col: int) -> None:
        """Queue `module` for `launch_deferred`; keeps a and g alive until then.  Everything about the
        module that does not change between batches (projection matrices, factor vectors, output column)
        is resolved and checked on its first batch only."""
        name: str = module._name  # type: ignore[assignment]
        if self.per_module_projection_dim is None:
            a = module._inputs
            assert isinstance(a, Tensor), "Activation cache missing for module"
            self._deferred_full.append((self.full_prepared(module, g, out_col), name, a, g))
            return
        if isinstance(self.normalizer_for(name), AdamNormalizer):
            a = module._inputs
            assert isinstance(a, Tensor), "Activation cache missing for module"
            self._deferred_adam.append((self.adam_prepared(module, g, out_col), a, g))
            return
        prepared = self._prepared.get(name)
        if prepared is None or prepared.dtype != g.dtype or prepared.out_col != out_col:
            prepared = ops.PreparedModule(self.module_input(module, g, out_col), self.per_module_projection_dim)
            self._prepared[name] = prepared
        a = module._inputs
        assert isinstance(a, Tensor), "Activation cache missing for module"
        self._deferred.append((prepared, a, g))

    def launch_deferred(self, out: Tensor, *, lengths: Tensor | None = None, out_rows: Tensor | None = None,
                        row_offsets: Tensor | None = None) -> None:
        """One fused launch over every queued module (one launch sequence per module with an Adam
        normaliser), writing each module's block of `out`."""
        if not self._deferred and not self._deferred_adam and not self._deferred_full:
            return
        p = self.per_module_projection_dim
        if p is None:
            try:
                if self.processor.projection_target == "global":
                    self._global_projection(self._deferred_full, out, lengths, out_rows, row_offsets)
                else:
                    for prep, _name, a, g in self._deferred_full:
                        ops.full_gradient(prep, a, g, out, per_token=self.attribute_tokens, lengths=lengths,
                                          rows=row_offsets if self.attribute_tokens else out_rows, lo=self.lo,
                                          hi=self.hi)
            finally:
                self._deferred_full.clear()
            return
        try:
            if self.attribute_tokens:
                assert lengths is not None and row_offsets is not None
                if self._deferred:
                    ops.collect_prepared(True, self._deferred, p, out, lengths, row_offsets, self.lo, self.hi)
                for prep, a, g in self._deferred_adam:
                    ops.collect_adam(prep, a, g, out, per_token=True, lengths=lengths, rows=row_offsets, lo=self.lo,
                                     hi=self.hi)
            else:
                if self._deferred:
                    ops.collect_prepared(False, self._deferred, p, out, lengths, out_rows, self.lo, self.hi)
                for prep, a, g in self._deferred_adam:
                    ops.collect_adam(prep, a, g, out, per_token=False, lengths=lengths, rows=out_rows, lo=self.lo,
                                     hi=self.hi)
        finally:
            self._deferred.clear()
            self._deferred_adam.clear()
            self._deferred_full.clear()

    @abstractmethod
    def setup(self) -> None: ...

    @abstractmethod
    def teardown(self) -> None: ...

    @abstractmethod
    def backward_hook(self, module: nn.Module, g: Tensor) -> None: ...

    @abstractmethod
    def process_batch(self, indices: list[int], **kwargs) -> None: ...


class BatchRecord:
    """What the forward hooks saw during one recorded batch: `entries` = (module, kept input, output) per
    call of a target module, in call order; `mask` = the batch's collection mask."""

    __slots__ = ("mask", "doc_lengths", "entries", "versions")

    def __init__(self, mask: Tensor | None, doc_lengths: list[int] | None = None):
        self.mask = mask
        self.doc_lengths = doc_lengths
        self.entries: list[tuple[nn.Module, Tensor | None, Tensor]] = []
        self.versions: list[int] = []

    def outputs(self) -> list[Tensor]:
        """The recorded module outputs, for `torch.autograd.grad(loss, record.outputs())`.  A tensor hook is
        tied to the value a module returned; `autograd.grad` is tied to the tensor object, so a model that
        overwrites a module's output in place afterwards would be given the gradient of the overwritten
        value: refused here."""
        for (module, _kept, out), version in zip(self.entries, self.versions):
            if out._version != version:
                raise RuntimeError(
                    f"the output of {getattr(module, '_name', module)} was modified in place after the module "
                    "returned it; the overlapped loop cannot collect from such a model: construct "
                    "CollectorComputer with overlap_backward=False (or set BGX_OVERLAP_BACKWARD=0)")
        return [e[2] for e in self.entries]


class CollectorComputer:
    """Runs forward/backward over the batches and feeds the collector (collector.py:771-923)."""

    def __init__(self, model, data, *, collector: HookCollectorBase, batches: list[list[int]] | None = None,
                 cfg: IndexConfig, overlap_backward: bool | None = None):
        """`overlap_backward`: run each batch's backward pass beside the next batch's forward pass
        (`OverlappedSteps`); None = on for models on a GPU unless the environment has
        `BGX_OVERLAP_BACKWARD=0`.  Off gives the reference's plain loop, one batch at a time."""
        self.model = model
        self.device = torch.device(model.device)
        self.data = data
        self.batches = batches if batches is not None else [[idx] for idx in range(len(data))]
        self.forward_backward = fwd_bwd_factory(cfg)
        if overlap_backward is None:
            overlap_backward = self.device.type == "cuda" and os.environ.get("BGX_OVERLAP_BACKWARD", "1") != "0"
        self.overlap_backward = overlap_backward
        self.collector = collector
        self.cfg = cfg
        self.rank = dist.get_rank() if dist.is_initialized() else 0
        self.world_size = dist.get_world_size() if dist.is_initialized() else 1

    def run_with_collector_hooks(self, desc: Optional[str] = None):
        """For each batch: pad, forward, loss, backward (hooks fire), `collector.process_batch`; then
        `collector.teardown()`.  No host synchronisation happens inside the loop."""
        total_processed = torch.tensor(0, device=self.device)
        overlapped = OverlappedSteps(self.model, self.collector, self.cfg) if self.overlap_backward else None
        try:
            for indices in self.batches:
                batch = self.data[indices]
                x, y, _, collection_mask = pad_and_tensor(batch["input_ids"], labels=batch.get("labels"),
                                                          device=self.device, sync_max_len=False)
                total_processed += collection_mask.sum()
                if overlapped is not None:
                    overlapped.step(indices, batch, x, y, collection_mask)
                    continue
                with self.collector.with_batch(collection_mask, [len(seq) for seq in batch["input_ids"]]):
                    losses = self.forward_backward(self.model, x, y, batch)
                self.collector.process_batch(indices, losses=losses)
            if overlapped is not None:
                overlapped.drain()
        except BaseException:
            if overlapped is not None:
                overlapped.close(failed=True)
                overlapped = None
            raise
        if overlapped is not None:
            overlapped.close()
        self.collector.teardown()
        self.collector.remove_hooks()
        if dist.is_initialized():
            dist.all_reduce(total_processed, op=dist.ReduceOp.SUM)
        if self.rank == 0 and self.cfg.run_path:
            os.makedirs(self.cfg.partial_run_path, exist_ok=True)
            torch.save(total_processed, os.path.join(self.cfg.partial_run_path, "total_processed.pt"))
        self.total_processed = total_processed


def forward_loss_factory(cfg: IndexConfig) -> Callable:
    """forward_loss(model, x, y, batch) -> per-sample losses [N] with their autograd graph: the forward half
    of collector.py:926-985 (cross-entropy branch)."""
    if cfg.loss_fn != "ce":
        raise NotImplementedError("only the cross-entropy loss is supported (loss_fn='kl' needs PEFT)")

    def forward_loss(model, x: Tensor, y: Tensor, batch: dict):
        # The reference slices `logits[:, :-1]` and reshapes, which copies the [N, S-1, V] logits (400 MB for a
        # 4096-token batch of a 50k vocabulary) and, in the backward pass, zero-fills and copies them again.
        # The same losses come from the whole [N, S, V] tensor as a view, with the labels shifted left and the
        # last position ignored (-100 is cross_entropy's ignore_index: loss 0, gradient 0 -- what the slice's
        # backward pass fills in).
        logits = model(x).logits
        targets = F.pad(y[:, 1:], (0, 1), value=-100)
        masks = y[:, 1:] != -100
        denoms = masks.sum(dim=1, dtype=model.dtype) if cfg.loss_reduction == "mean" else 1.0
        if logits.is_contiguous():
            losses = F.cross_entropy(logits.view(-1, logits.size(-1)), targets.flatten(), reduction="none",
                                     label_smoothing=cfg.label_smoothing).view_as(targets)
        else:
            logits = logits[:, :-1]
            losses = F.cross_entropy(logits.reshape(-1, logits.size(-1)), y[:, 1:].flatten(), reduction="none",
                                     label_smoothing=cfg.label_smoothing).reshape_as(y[:, 1:])
        losses = losses.sum(1) / denoms
        if "advantage" in batch:
            losses *= torch.tensor(batch["advantage"], device=losses.device)
        return losses

    return forward_loss


def fwd_bwd_factory(cfg: IndexConfig) -> Callable:
    """fwd_bwd(model, x, y, batch) -> per-sample losses [N] (collector.py:926-985, cross-entropy branch)."""
    forward_loss = forward_loss_factory(cfg)
    trainable: dict[int, list] = {}

    def fwd_bwd(model, x: Tensor, y: Tensor, batch: dict):
        losses = forward_loss(model, x, y, batch)
        losses.sum().backward()
        # model.zero_grad(): only parameters that require grad can hold one; the list is built once
        params = trainable.get(id(model))
        if params is None:
            params = trainable[id(model)] = [q for q in model.parameters() if q.requires_grad]
        for q in params:
            q.grad = None
        return losses

    return fwd_bwd


_SECOND_STREAMS: dict = {}


def _second_stream(device: torch.device):
    """The one extra stream per device that `OverlappedSteps` alternates with the caller's.  Made once per
    process: which hardware queue a stream lands on depends on how many were made before it, and two
    streams that share a queue run nothing side by side."""
    key = torch.device(device)
    if key not in _SECOND_STREAMS:
        _SECOND_STREAMS[key] = torch.cuda.Stream(key)
    return _SECOND_STREAMS[key]


class OverlappedSteps:
    """The loop body of `run_with_collector_hooks` with the backward pass of a batch running beside the
    forward pass of the next one.

    Issued one batch at a time, a step of a small model leaves both sides idle in turn: the forward pass is
    Python issuing a few hundred small kernels, the backward pass is the autograd engine's own thread
    issuing as many, and most of the kernels are too small to fill the GPU.  Here the forward hooks only
    record (module, input, output); the gradients of the recorded outputs are asked of
    `torch.autograd.grad` on a helper thread, which holds no interpreter lock while the engine runs, and
    the caller goes on to the next batch's forward pass.  When a batch's gradients are there,
    `backward_hook` is called per module as a backward pass would have (`replay_backward`) and
    `process_batch` launches the batch's kernels.

    `streams=2` (the default; `BGX_OVERLAP_STREAMS=1` for one): batches alternate between the caller's
    stream and one extra stream of the same priority, so the two passes that overlap on the host also sit
    in different queues on the GPU.  A batch's hooks and launches go to its own stream, after the other
    stream's work so far, and the other stream's later work waits for them: the collector's kernels have
    the GPU to themselves, and its workspace and store are never touched by two launches at once.  With
    one stream the kernels of neighbouring batches interleave in the caller's queue.

    The rows and losses are those of the plain loop, bit for bit.  Nothing is accumulated into `.grad`.
    Two batches' activations are alive at a time.
    """

    def __init__(self, model, collector: HookCollectorBase, cfg: IndexConfig, *, streams: int | None = None):
        from concurrent.futures import ThreadPoolExecutor

        self.model = model
        self.collector = collector
        self.forward_loss = forward_loss_factory(cfg)
        self._pool = ThreadPoolExecutor(max_workers=1, thread_name_prefix="bgx-backward")
        self._pending = None
        self._entered = False
        self._trainable = [q for q in model.parameters() if q.requires_grad]
        # The backward pass is asked to go down to the output of the input embedding (every layer's nodes run,
        # so hooks that others have put on the layers still fire) rather than to the parameters: a parameter's
        # gradient accumulator belongs to one stream, and the engine makes that stream wait for the end of
        # every backward pass on the other one -- in the middle of the next batch's forward pass, whenever the
        # host happens to be that far.  Models without `get_input_embeddings` are asked for the parameters.
        self._embedding_output: Tensor | None = None
        self._embedding_hook = None
        embedding = getattr(model, "get_input_embeddings", None)
        embedding = embedding() if callable(embedding) and os.environ.get("BGX_OVERLAP_ROOT") != "parameters" else None
        if isinstance(embedding, nn.Module) and not self._has_foreign_hooks(embedding):
            self._embedding_hook = embedding.register_forward_hook(self._keep_embedding_output)
        # With two streams, batches alternate between them: the kernels of one batch's backward pass and of
        # the next batch's forward pass then sit in different queues and the many small ones among them run
        # side by side.  A batch's own launches (which share the collector's workspace and store with every
        # other batch's) wait for both streams and hold both, see `step`.
        self._streams: list = []
        self._n_streams = min(2, streams if streams is not None else int(os.environ.get("BGX_OVERLAP_STREAMS", "2")))
        self._step_no = 0
        if self._n_streams > 1:
            # every other batch's graph ends at parameters whose gradient accumulators sit on the caller's
            # stream; the engine orders the two streams itself, and says so once per process unless told not to
            quiet = getattr(torch.autograd.graph, "set_warn_on_accumulate_grad_stream_mismatch", None)
            if quiet is not None:
                quiet(False)

    @staticmethod
    def _has_foreign_hooks(embedding: nn.Module) -> bool:
        """Whether someone else watches the input embedding: hooks on the module, or on its parameters'
        gradients.  Stopping the backward pass at the embedding's output leaves the embedding's own backward
        node out (the reference runs it: the embedding is the one trainable module,
        bergson/utils/worker_utils.py:224-225), so such hooks would not fire; with them present the backward
        pass goes down to the parameters as `backward()` does."""
        module_hooks = ("_forward_hooks", "_forward_pre_hooks", "_backward_hooks", "_backward_pre_hooks")
        if any(len(getattr(embedding, attr, None) or ()) for attr in module_hooks):
            return True
        for q in embedding.parameters(recurse=False):
            if getattr(q, "_backward_hooks", None) or getattr(q, "_post_accumulate_grad_hooks", None):
                return True
        return False

    def _keep_embedding_output(self, _module, _inp, out):
        if self.collector._recording is not None and isinstance(out, Tensor) and out.requires_grad:
            self._embedding_output = out

    @staticmethod
    def _gradients(total: Tensor, outputs: list[Tensor], stream, n_recorded: int):
        # retain_graph: the engine then frees no saved tensor while it runs.  Almost every one of them has
        # been seen by Python, and releasing such a tensor from the engine's thread takes the interpreter
        # lock -- hundreds of times per pass, each time against the thread that is issuing the next forward
        # pass.  The graph is dropped by the caller's thread instead (`_finish`), which holds the lock anyway.
        if stream is None:  # host tensors (the loop logic is testable without a GPU; the kernels are not)
            return torch.autograd.grad(total, outputs, allow_unused=True, retain_graph=True)[:n_recorded]
        with torch.cuda.device(total.device), torch.cuda.stream(stream):
            return torch.autograd.grad(total, outputs, allow_unused=True, retain_graph=True)[:n_recorded]

    def step(self, indices: list[int], batch: dict, x: Tensor, y: Tensor, collection_mask: Tensor) -> None:
        col = self.collector
        if not self._entered:
            col.__enter__()
            self._entered = True
        stream = None
        if x.is_cuda:
            stream = caller = torch.cuda.current_stream(x.device)
            if self._n_streams > 1:
                if not self._streams:
                    self._streams = [caller, _second_stream(x.device)]
                stream = self._streams[self._step_no % 2]
                if stream is not caller:
                    stream.wait_stream(caller)  # the batch's tensors were made on the caller's stream
                    for t in (x, y, collection_mask):
                        t.record_stream(stream)
            self._step_no += 1
        record = col.begin_recording(collection_mask, [len(seq) for seq in batch["input_ids"]]
                                     if isinstance(batch, dict) and "input_ids" in batch else None)
        try:
            with torch.cuda.stream(stream) if stream is not None else nullcontext():
                losses = self.forward_loss(self.model, x, y, batch)
                total = losses.sum()
        finally:
            col.end_recording()
        # besides the recorded outputs: the embedding's output (see __init__), or the trainable parameters,
        # whose gradients are dropped as the plain loop drops them with zero_grad
        root, self._embedding_output = self._embedding_output, None
        outputs = record.outputs() + ([root] if root is not None else self._trainable)
        del root
        if self._n_streams > 1 and stream is not None:
            # the previous batch's launch gets the GPU to itself: it starts when this forward pass has
            # finished too, and this batch's backward pass waits for it (an HBM-bound kernel sharing the
            # chip with the other queue's kernels takes half as long again, and slows them in turn)
            self._finish(before=stream)
            future = self._pool.submit(self._gradients, total, outputs, stream, len(record.entries))
        else:
            future = self._pool.submit(self._gradients, total, outputs, stream, len(record.entries))
            self._finish()
        del outputs
        self._pending = (indices, record, losses.detach(), future, stream, total)

    def _finish(self, before=None) -> None:
        """Hooks and `process_batch` of the batch whose backward pass is out, on that batch's stream;
        `before` = the stream of the batch that follows (its work so far precedes the launch, its later
        work follows it)."""
        if self._pending is None:
            return
        (indices, record, losses, future, stream, total), self._pending = self._pending, None
        grads = future.result()
        del total, future  # with the record's outputs (cleared by replay_backward), the last owners of the graph
        if stream is None or self._n_streams <= 1:
            self.collector.replay_backward(record, grads)
            self.collector.process_batch(indices, losses=losses)
            return
        with torch.cuda.stream(stream):
            if before is not None:
                stream.wait_stream(before)
            self.collector.replay_backward(record, grads)
            self.collector.process_batch(indices, losses=losses)
        if before is not None:
            before.wait_stream(stream)

    def drain(self) -> None:
        """Finish the batch whose backward pass is still out; the caller's stream then waits for the
        streams the batches ran on."""
        self._finish()
        for s in self._streams[1:]:
            self._streams[0].wait_stream(s)

    def close(self, failed: bool = False) -> None:
        if self._pending is not None:
            future = self._pending[3]
            self._pending = None
            try:
                future.result()  # let the backward pass that is still out finish before the hooks go away
            except Exception:
                pass  # close() runs after a failure too; the first error is the one the caller sees
        self._pool.shutdown(wait=True)
        if self._embedding_hook is not None:
            self._embedding_hook.remove()
            self._embedding_hook = None
        if self._entered:
            self.collector.__exit__(RuntimeError if failed else None, None, None)
            self._entered = False
