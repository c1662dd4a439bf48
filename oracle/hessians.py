"""CPU restatement of the dense (autocorrelation) preconditioner.  TEST INFRASTRUCTURE ONLY.

Follows bergson/hessians/inversion.py:43-222 (eigenvalue functions, `eigenvalue_multiplier`,
`invert_psd_matrix`), bergson/hessians/preconditioner.py:77-92 (`DensePreconditioner.apply`),
bergson/collector/in_memory_collector.py:149-154 (Gram accumulation) and
bergson/process_autocorrelation.py:32-44 (normalisation by the row count).

Written with numpy in float64 from the formulas in those files -- deliberately not with the torch calls
the package itself uses -- and pinned in tests/test_oracle_hessians.py by closed forms: a diagonal matrix
(where every mode is an elementwise formula), H^-1 H = I at zero damping, (H^-1/2)^2 = H^-1, the
pseudo-inverse of a rank-deficient matrix against numpy.linalg.pinv, and a 2 x 2 case worked by hand.
"""
from __future__ import annotations

import numpy as np


def eigen_multiplier(inversion: str, lam: np.ndarray, damping_factor: float, power: float = -1.0) -> np.ndarray:
    """m(lambda) of inversion.py:43-99, :140-178 on a full spectrum (mean taken over it)."""
    lam = np.asarray(lam, dtype=np.float64)
    mean = lam.mean()
    if inversion in ("damped_inverse", "factored_tikhonov"):  # the latter falls back on the dense path (:215-217)
        m = 1.0 / (lam + damping_factor * mean)
    elif inversion == "tikhonov_filtered":
        alpha = damping_factor * mean
        m = lam / (lam * lam + alpha * alpha)
    elif inversion == "pseudoinverse":
        tol = damping_factor * mean
        with np.errstate(divide="ignore"):
            m = np.where(lam > tol, 1.0 / lam, 0.0)
    else:
        raise ValueError(inversion)
    frac = -power
    if frac != 1.0:
        m = np.maximum(m, 0.0) ** frac
    return m


def invert_psd(H: np.ndarray, inversion: str = "damped_inverse", damping_factor: float = 0.1,
               power: float = -1.0) -> np.ndarray:
    """V diag(m(max(lambda, 0))) V^T in float64 (inversion.py:181-222)."""
    lam, vec = np.linalg.eigh(np.asarray(H, dtype=np.float64))
    lam = np.maximum(lam, 0.0)
    m = eigen_multiplier(inversion, lam, damping_factor, power)
    return (vec * m) @ vec.T


def apply_dense(grads: dict[str, np.ndarray], h_inv: dict[str, np.ndarray]) -> dict[str, np.ndarray]:
    """{name: g @ H^p}, modules without a matrix unchanged (preconditioner.py:77-92); float64."""
    return {name: (np.asarray(g, dtype=np.float64) @ np.asarray(h_inv[name], dtype=np.float64)) if name in h_inv
            else np.asarray(g, dtype=np.float64) for name, g in grads.items()}


def gram(rows_per_batch: list[np.ndarray], num_rows: int) -> np.ndarray:
    """sum_batches P^T P / num_rows (in_memory_collector.py:149-154, process_autocorrelation.py:32-33)."""
    d = rows_per_batch[0].shape[1]
    acc = np.zeros((d, d), dtype=np.float64)
    for P in rows_per_batch:
        P = np.asarray(P, dtype=np.float64)
        acc += P.T @ P
    return acc / num_rows
