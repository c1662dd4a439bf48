"""Configuration dataclasses of the collection / scoring path.

Field names and defaults follow bergson/config/config.py (`AttentionConfig`
:548, `IndexConfig` :562-660, `QueryConfig` :707-751, `PreprocessConfig`
:754-779, `ScoreConfig` :782-814) so that keyword arguments written for the
reference keep working.  Only the fields the path reads are carried; the CLI /
YAML machinery of the reference is not part of this package.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path
from typing import Literal


@dataclass
class AttentionConfig:
    """How to split an attention module's output features into heads."""

    num_heads: int = 0
    head_size: int = 0
    head_dim: int = 0
    """Axis of `num_heads` in the activation gradient [N, S, O]; only the feature axis (2 or -1) is supported."""


@dataclass
class IndexConfig:
    """Settings of a gradient-store build."""

    run_path: str = ""
    """Directory of the finished store; artefacts are written to `run_path + '.part'` first."""
    projection_dim: int = 0
    include_bias: bool = False
    reshape_to_square: bool = False
    projection_type: Literal["normal", "rademacher"] = "rademacher"
    projection_scale: Literal["jl", "row_norm"] = "jl"
    projection_target: Literal["per_module", "global"] = "per_module"
    token_batch_size: int = 2048
    max_batch_size: int | None = None
    loss_fn: Literal["ce", "kl"] = "ce"
    loss_reduction: Literal["mean", "sum"] = "sum"
    label_smoothing: float = 0.0
    split_attention_modules: list[str] = field(default_factory=list)
    attention: AttentionConfig = field(default_factory=AttentionConfig)
    profile: bool = False
    filter_modules: str | None = None
    attribute_tokens: bool = False
    modules: list[str] = field(default_factory=list)
    drop_columns: bool = True
    debug: bool = False

    @property
    def partial_run_path(self) -> Path:
        return Path(self.run_path + ".part")


@dataclass
class InversionConfig:
    """How to invert a Hessian with regularisation (bergson/config/config.py:78-96): `inversion` is one of
    "damped_inverse" 1/(l + c mean(l)), "tikhonov_filtered" l/(l^2 + (c mean(l))^2), "pseudoinverse" 1/l where
    l > c mean(l) else 0, "factored_tikhonov" (= damped_inverse for a dense Hessian); c = damping_factor."""

    inversion: str = "damped_inverse"
    damping_factor: float = 0.1


@dataclass
class PreprocessConfig:
    """Gradient preprocessing shared by build, reduce and score."""

    unit_normalize: bool = False
    hessian_path: str | None = None
    """A saved GradientProcessor with dense autocorrelation Hessians: gradients are multiplied by H^-1, or by
    H^-1/2 on both sides when unit_normalize is set."""
    ev_correction: bool = False
    inversion_cfg: InversionConfig = field(default_factory=InversionConfig)
    aggregation: Literal["mean", "sum", "none"] = "none"
    normalize_aggregated_grad: bool = False


@dataclass
class ScoreConfig:
    """Settings of on-the-fly scoring."""

    query_path: str = ""
    score: Literal["nearest", "individual"] = "individual"
    batch_size: int = 1024
    query_batch_size: int | None = None
    precision: Literal["auto", "bf16", "fp16", "fp32"] = "fp32"
    modules: list[str] = field(default_factory=list)
    higher_is_better: bool = True


@dataclass
class QueryConfig:
    """Settings for querying an existing store."""

    index: str = ""
    model: str = ""
    text_field: str = "text"
    unit_norm: bool = True
    hessian_path: str | None = None
    ev_correction: bool = False
    faiss: bool = False
    top_k: int = 5
    record: str = ""
