"""Gradient-processing configuration and optimizer-state normalisers.

Mirrors bergson/gradients.py: `Normalizer` registry :12-74, `GradientProcessor`
:77-239 (files processor_config.yaml / normalizers.pth / hessians.pth /
hessians_eigen.pth), `LayerAdapter` :242-273, `AdafactorNormalizer` :276-363,
`AdamNormalizer` :366-420.  The normalisers here are containers: on the
collection path their arithmetic runs inside the HIP kernels.
"""
from __future__ import annotations

from abc import ABC
from dataclasses import asdict, dataclass, field
from pathlib import Path
from typing import Literal, Mapping

import torch
import torch.nn as nn
import yaml
from torch import Tensor

try:  # HF Conv1D is optional: the package works without transformers
    from transformers.pytorch_utils import Conv1D as HFConv1D
except Exception:  # pragma: no cover

    class HFConv1D(nn.Module):  # type: ignore[no-redef]
        pass


NORMALIZER_TYPES: dict[str, type["Normalizer"]] = {}


class Normalizer(ABC):
    """Second-moment statistics of one matrix-valued parameter."""

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        NORMALIZER_TYPES[cls.__name__] = cls

    @staticmethod
    def from_state_dict(state_dict: dict) -> "Normalizer":
        state_dict = dict(state_dict)
        class_name = state_dict.pop("__class__")
        assert isinstance(class_name, str), "Expected '__class__' to be a string"
        if (cls := NORMALIZER_TYPES.get(class_name)) is None:
            raise ValueError(f"Unknown normalizer class: '{class_name}'")
        if "avg_sq" in state_dict:  # renamed field of old stores
            state_dict["weight_avg_sq"] = state_dict.pop("avg_sq")
        return cls(**state_dict)

    def state_dict(self) -> dict:
        tensors = {k: v for k, v in self.__dict__.items() if isinstance(v, Tensor)}
        return {"__class__": self.__class__.__name__, **tensors}


@dataclass
class AdafactorNormalizer(Normalizer):
    """Row [O] and column [I] sums of second moments, optional bias moments [O]."""

    row: Tensor
    col: Tensor
    bias_avg_sq: Tensor | None = None

    def __post_init__(self):
        assert self.row.ndim == 1, f"Expected 1D tensor for row, got {self.row.ndim}D"
        assert self.col.ndim == 1, f"Expected 1D tensor for col, got {self.col.ndim}D"
        if self.bias_avg_sq is not None:
            assert self.bias_avg_sq.ndim == 1, f"Expected 1D tensor for bias_avg_sq, got {self.bias_avg_sq.ndim}D"

    def to_adam(self) -> "AdamNormalizer":
        """Materialise the rank-one second-moment matrix (gradients.py:351-363)."""
        weight_avg_sq = torch.outer(self.row, self.col) / self.row.mean()
        return AdamNormalizer(weight_avg_sq=weight_avg_sq, bias_avg_sq=self.bias_avg_sq)


@dataclass
class AdamNormalizer(Normalizer):
    """Full second moments [O, I], optional bias moments [O]."""

    weight_avg_sq: Tensor
    bias_avg_sq: Tensor | None = None

    def to_adafactor(self) -> AdafactorNormalizer:
        """Row / column means (gradients.py:402-420)."""
        assert self.weight_avg_sq.ndim == 2, f"Expected 2D tensor for avg_sq, got {self.weight_avg_sq.ndim}D"
        return AdafactorNormalizer(row=self.weight_avg_sq.mean(dim=1), col=self.weight_avg_sq.mean(dim=0),
                                   bias_avg_sq=self.bias_avg_sq)


@dataclass
class GradientProcessor:
    """Configuration for processing and compressing gradients (gradients.py:77-134)."""

    normalizers: Mapping[str, Normalizer] = field(default_factory=dict)
    hessians: dict[str, Tensor] = field(default_factory=dict)
    hessians_eigen: Mapping[str, tuple[Tensor, Tensor]] = field(default_factory=dict)
    projection_dim: int | None = None
    reshape_to_square: bool = False
    projection_type: Literal["normal", "rademacher"] = "rademacher"
    projection_target: Literal["per_module", "global"] = "per_module"
    projection_scale: Literal["jl", "row_norm"] = "jl"
    include_bias: bool = False

    def __post_init__(self):
        self._projection_matrices: dict[tuple[str, str, torch.device], Tensor] = {}

    @classmethod
    def load(cls, path: Path | str, *, map_location=None, skip_hessians: bool = False) -> "GradientProcessor":
        """Read processor_config.yaml, normalizers.pth and the hessian files (gradients.py:136-211)."""
        path = Path(path)
        hess_path = path / "hessians.pth"
        if not hess_path.exists():
            hess_path = path / "preconditioners.pth"
        hess_eigen_path = path / "hessians_eigen.pth"
        if not hess_eigen_path.exists():
            hess_eigen_path = path / "preconditioners_eigen.pth"
        with (path / "processor_config.yaml").open("r") as f:
            cfg = yaml.safe_load(f)
        # defaults of stores written before these keys existed
        cfg.setdefault("projection_type", "normal")
        cfg.setdefault("include_bias", False)
        cfg.setdefault("projection_scale", "row_norm")
        for legacy_key in list(cfg.keys()):
            if "preconditioner" in legacy_key or "precond" in legacy_key:
                new_key = (legacy_key.replace("preconditioners", "hessians").replace("preconditioner", "hessian")
                           .replace("precond", "hess"))
                cfg[new_key] = cfg.pop(legacy_key)
        norm_state = torch.load(path / "normalizers.pth", map_location=map_location, weights_only=True)
        normalizers = {name: Normalizer.from_state_dict(state) for name, state in norm_state.items()}
        hessians, hessians_eigen = {}, {}
        if not skip_hessians and hess_path.exists():
            hessians = torch.load(hess_path, map_location=map_location, weights_only=True)
        if not skip_hessians and hess_eigen_path.exists():
            hessians_eigen = torch.load(hess_eigen_path, map_location=map_location, weights_only=True)
        return cls(normalizers=normalizers, hessians=hessians, hessians_eigen=hessians_eigen, **cfg)

    def save(self, path: Path | str) -> None:
        """Write the four artefact files (gradients.py:213-239)."""
        path = Path(path)
        path.mkdir(parents=True, exist_ok=True)
        cfg = asdict(self)
        del cfg["normalizers"], cfg["hessians"], cfg["hessians_eigen"]
        with (path / "processor_config.yaml").open("w") as f:
            yaml.safe_dump(cfg, f, sort_keys=False)
        norm_state = {name: n.state_dict() for name, n in self.normalizers.items()}
        torch.save(norm_state, path / "normalizers.pth")
        torch.save(self.hessians, path / "hessians.pth")
        torch.save(self.hessians_eigen, path / "hessians_eigen.pth")


class LayerAdapter:
    """Feature-count attributes of the supported layer types (gradients.py:242-273)."""

    supported_modules = (nn.Linear, HFConv1D, nn.Conv1d, nn.Conv2d, nn.Conv3d)

    @staticmethod
    def in_attr(layer: nn.Module) -> str:
        if isinstance(layer, nn.Linear):
            return "in_features"
        if isinstance(layer, HFConv1D):
            return "nx"
        if isinstance(layer, (nn.Conv1d, nn.Conv2d, nn.Conv3d)):
            return "in_channels"
        raise ValueError(f"Unsupported layer type: {type(layer)}")

    @staticmethod
    def out_attr(layer: nn.Module) -> str:
        if isinstance(layer, nn.Linear):
            return "out_features"
        if isinstance(layer, HFConv1D):
            return "nf"
        if isinstance(layer, (nn.Conv1d, nn.Conv2d, nn.Conv3d)):
            return "out_channels"
        raise ValueError(f"Unsupported layer type: {type(layer)}")

    @staticmethod
    def weight_transposed(layer: nn.Module) -> bool:
        return isinstance(layer, HFConv1D)
