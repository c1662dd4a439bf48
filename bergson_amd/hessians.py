"""Dense (autocorrelation) preconditioner: fitting, inversion and application.

Mirrors, for the dense per-module Gram only:
  * `eigenvalue_multiplier`, `invert_psd_matrix`       bergson/hessians/inversion.py:36-222
  * `DensePreconditioner`, `load_preconditioner`        bergson/hessians/preconditioner.py:51-92, :464-495
  * `process_autocorrelation_matrices` (one process)    bergson/process_autocorrelation.py:7-49
  * the split index transform                           bergson/score/score.py:111-135

The matrices are prepared once on the host (an fp64 eigendecomposition per module, as in the
reference); what runs per batch -- `g @ H^p` for every module of a row block, and the Gram
accumulation `H += P^T P` during collection -- is one fused HIP launch each (`ops.block_gemm`,
`ops.gram_accumulate`).  The factored EKFAC family is not part of this package.
"""
from __future__ import annotations

from pathlib import Path
from typing import Callable, Literal

import torch
from torch import Tensor

from . import ops
from .config import InversionConfig
from .data import column_offsets
from .gradients import GradientProcessor

Inversion = Literal["damped_inverse", "factored_tikhonov", "pseudoinverse", "tikhonov_filtered"]
INVERSIONS: tuple[str, ...] = ("damped_inverse", "factored_tikhonov", "pseudoinverse", "tikhonov_filtered")


def damped_inverse_eigfn(eigvals: Tensor, mean: Tensor, damping_factor: float) -> Tensor:
    """1 / (lambda + c * mean(lambda))."""
    return (eigvals + damping_factor * mean).reciprocal()


def tikhonov_filtered_eigfn(eigvals: Tensor, mean: Tensor, damping_factor: float) -> Tensor:
    """lambda / (lambda^2 + alpha^2), alpha = c * mean(lambda)."""
    alpha_sq = (damping_factor * mean) ** 2
    return eigvals / (eigvals * eigvals + alpha_sq)


def pseudoinverse_eigfn(eigvals: Tensor, mean: Tensor, damping_factor: float) -> Tensor:
    """1 / lambda where lambda > c * mean(lambda), else 0."""
    tol = damping_factor * mean
    return torch.where(eigvals > tol, eigvals.reciprocal(), torch.zeros_like(eigvals))


EIGENFNS: dict[str, Callable[[Tensor, Tensor, float], Tensor]] = {
    "damped_inverse": damped_inverse_eigfn,
    "tikhonov_filtered": tikhonov_filtered_eigfn,
    "pseudoinverse": pseudoinverse_eigfn,
}


def eigenvalue_multiplier(inversion: str, eigvals: Tensor, mean: Tensor, damping_factor: float, *,
                          power: float = -1.0) -> Tensor:
    """The factor m(lambda) that scales an eigenvalue toward its inverse; raised to -power when that is
    not 1 (power = -0.5: the square-root inverse, which applied twice gives the inverse)."""
    if inversion not in EIGENFNS:
        raise ValueError(f"inversion {inversion!r} has no dense form (choose from {sorted(EIGENFNS)})")
    multiplier = EIGENFNS[inversion](eigvals, mean, damping_factor)
    frac = -power
    if frac != 1.0:
        multiplier = multiplier.clamp_min(0).pow(frac)
    return multiplier


def invert_psd_matrix(H: Tensor, inversion: str = "damped_inverse", damping_factor: float = 0.1,
                      power: float = -1.0, dtype: torch.dtype = torch.float64) -> Tensor:
    """Regularised inverse power of a p.s.d. matrix through its eigendecomposition, in `dtype`, returned in
    H's dtype.  `factored_tikhonov` has no dense analogue and means `damped_inverse` here."""
    original_dtype = H.dtype
    H = H.to(dtype=dtype)
    eigvals, eigvecs = torch.linalg.eigh(H)
    eigvals = eigvals.clamp_min(0)  # eigh of a numerically p.s.d. Gram gives small negative values
    dense_inversion = "damped_inverse" if inversion == "factored_tikhonov" else inversion
    scaled = eigenvalue_multiplier(dense_inversion, eigvals, eigvals.mean(), damping_factor, power=power)
    return (eigvecs * scaled @ eigvecs.mH).to(original_dtype)


class DensePreconditioner:
    """Per-module `H^p` matrices (fp32, on the device that applies them)."""

    def __init__(self, h_inv: dict[str, Tensor]):
        self.h_inv = h_inv

    @classmethod
    def from_processor(cls, processor: GradientProcessor, *, inversion_cfg: InversionConfig | None = None,
                       power: float = -1.0, device: str | torch.device = "cuda") -> "DensePreconditioner":
        """Invert each Gram of `processor` to `H^power`: fp64 eigendecomposition on the host, result fp32 on
        `device`."""
        inversion_cfg = inversion_cfg or InversionConfig()
        h_inv = {
            name: invert_psd_matrix(H.to(device="cpu", dtype=torch.float32), inversion=inversion_cfg.inversion,
                                    damping_factor=inversion_cfg.damping_factor, power=power).to(device).contiguous()
            for name, H in processor.hessians.items()
        }
        return cls(h_inv)

    def apply(self, grads: dict[str, Tensor]) -> dict[str, Tensor]:
        """`{name: g.float() @ H^p}`; modules without a matrix pass through unchanged."""
        if not self.h_inv:
            return grads
        out = {}
        for name, g in grads.items():
            if name not in self.h_inv:
                out[name] = g
                continue
            h = self.h_inv[name]
            rows = g.to(h.device)
            if rows.dtype not in ops.DTYPE_CODE:
                rows = rows.float()
            if rows.dim() != 2 or rows.stride(-1) != 1:
                rows = rows.reshape(-1, rows.shape[-1]).contiguous()
            res = ops.block_gemm(rows, [(h, 0)], out_dtype=torch.float32)
            out[name] = res.reshape(g.shape).to(g.device)
        return out

    def apply_rows(self, rows: Tensor, grad_sizes: dict[str, int], out_dtype: torch.dtype = torch.float32,
                   out: Tensor | None = None) -> Tensor:
        """The same on a concatenated row block `[n, sum(grad_sizes)]` in one launch (module order and
        widths as in `grad_sizes`)."""
        blocks = [(self.h_inv[name], lo) for name, (lo, _) in column_offsets(grad_sizes).items() if name in self.h_inv]
        for name, (lo, hi) in column_offsets(grad_sizes).items():
            if name in self.h_inv and self.h_inv[name].shape[0] != hi - lo:
                raise ValueError(f"{name}: matrix of size {self.h_inv[name].shape[0]} for a block of {hi - lo} columns")
        return ops.block_gemm(rows, blocks, out_dtype=out_dtype, out=out)


def is_factored_hessian(hessian_path: str | Path) -> bool:
    """A factored (EKFAC-family) Hessian directory holds eigenvector shards instead of a saved processor
    (preconditioner.py:457-461)."""
    return (Path(hessian_path) / "eigen_activation_sharded").is_dir()


def load_preconditioner(hessian_path: str | Path | None, *, inversion_cfg: InversionConfig | None = None,
                        power: float | None = -1.0, ev_correction: bool = False,
                        device: str | torch.device = "cuda") -> DensePreconditioner | None:
    """The preconditioner for the Hessian saved at `hessian_path`; None when the path or `power` is unset."""
    if power is None or hessian_path is None:
        return None
    if is_factored_hessian(hessian_path):
        raise NotImplementedError("factored (EKFAC) Hessians are outside this package; fit a dense one "
                                  "(InMemoryCollector(skip_hessians=False))")
    processor = GradientProcessor.load(Path(hessian_path), map_location="cpu")
    return DensePreconditioner.from_processor(processor, inversion_cfg=inversion_cfg, power=power, device=device)


def process_autocorrelation_matrices(processor: GradientProcessor, hessians: dict[str, Tensor], num_rows: int,
                                     grad_sizes: dict[str, int], rank: int = 0) -> None:
    """Normalise the accumulated Grams by the number of rows and attach them, with their eigendecompositions
    (fp64 on the host, stored in the Gram's dtype), to the processor.  One process."""
    hessians_eigen = {}
    for name, prec in hessians.items():
        hessians[name] = (prec / num_rows).cpu()
    for name in hessians:
        dtype = hessians[name].dtype
        eigvals, eigvecs = torch.linalg.eigh(hessians[name].to(torch.float64))
        hessians_eigen[name] = (eigvals.to(dtype).contiguous(), eigvecs.to(dtype).contiguous())
    processor.hessians = hessians
    processor.hessians_eigen = hessians_eigen


def make_split_hessian(hessians: dict[str, Tensor], modules: list[str], device: torch.device, dtype: torch.dtype):
    """Per-batch index transform of split (two-sided) preconditioning: every module's rows times its
    matrix, results in `dtype`."""
    mats = {m: hessians[m].to(device=device, dtype=torch.float32).contiguous() for m in modules}

    sizes = {m: mats[m].shape[0] for m in modules}
    cols = column_offsets(sizes)
    blocks = [(mats[m], lo) for m, (lo, _) in cols.items()]
    out_dtype = dtype if dtype in ops.DTYPE_CODE else torch.float32

    def transform(grads: dict[str, Tensor]) -> dict[str, Tensor]:
        from .builder import RowBlock

        rows = grads.rows if isinstance(grads, RowBlock) and grads.rows is not None and list(grads) == modules else None
        if rows is None:
            rows = torch.cat([grads[m].to(device, non_blocking=True) for m in modules], dim=1)
        if rows.dtype not in ops.DTYPE_CODE:
            rows = rows.float()
        block = RowBlock()
        block.rows = ops.block_gemm(rows.contiguous(), blocks, out_dtype=out_dtype)
        for m, (lo, hi) in cols.items():
            block[m] = block.rows[:, lo:hi]
        return block

    return transform
