"""Pins the CPU restatement of the dense preconditioner (oracle/hessians.py) by closed forms, and the
package's host-side inversion (bergson_amd/hessians.py, plain torch on the CPU) against that oracle."""
import numpy as np
import pytest
import torch

from oracle import hessians as oh


def _spd(d, seed, rank=None):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((d, rank or d))
    return A @ A.T / (rank or d)


@pytest.mark.parametrize("mode", ["damped_inverse", "tikhonov_filtered", "pseudoinverse", "factored_tikhonov"])
@pytest.mark.parametrize("power", [-1.0, -0.5])
def test_diagonal_matrix_is_the_elementwise_formula(mode, power):
    lam = np.array([4.0, 1.0, 0.25, 0.01])
    c = 0.1
    mean = lam.mean()
    want = {"damped_inverse": 1 / (lam + c * mean), "factored_tikhonov": 1 / (lam + c * mean),
            "tikhonov_filtered": lam / (lam ** 2 + (c * mean) ** 2),
            "pseudoinverse": np.where(lam > c * mean, 1 / lam, 0.0)}[mode]
    if power == -0.5:
        want = np.sqrt(want)
    got = oh.invert_psd(np.diag(lam), mode, c, power)
    assert np.allclose(got, np.diag(want), rtol=1e-12, atol=1e-14)


def test_two_by_two_by_hand():
    # H = [[2, 1], [1, 2]]: eigenvalues 1 and 3 (mean 2), eigenvectors (1, -1)/sqrt2 and (1, 1)/sqrt2;
    # damped inverse with c = 0.5: multipliers 1/2 and 1/4 -> H^-1 = [[3/8, -1/8], [-1/8, 3/8]]
    got = oh.invert_psd(np.array([[2.0, 1.0], [1.0, 2.0]]), "damped_inverse", 0.5)
    assert np.allclose(got, np.array([[0.375, -0.125], [-0.125, 0.375]]), atol=1e-14)


def test_zero_damping_is_the_inverse_and_half_power_squares_to_it():
    H = _spd(12, 0)
    inv = oh.invert_psd(H, "damped_inverse", 0.0)
    assert np.allclose(inv @ H, np.eye(12), atol=1e-9)
    for mode in ("damped_inverse", "tikhonov_filtered", "pseudoinverse"):
        half = oh.invert_psd(H, mode, 0.1, power=-0.5)
        assert np.allclose(half @ half, oh.invert_psd(H, mode, 0.1), rtol=1e-9, atol=1e-12)
        assert np.allclose(half, half.T, atol=1e-12)


def test_pseudoinverse_of_a_rank_deficient_matrix():
    H = _spd(10, 1, rank=4)
    got = oh.invert_psd(H, "pseudoinverse", 1e-9)
    assert np.allclose(got, np.linalg.pinv(H, hermitian=True), rtol=1e-7, atol=1e-9)


def test_gram_is_the_second_moment():
    rng = np.random.default_rng(2)
    batches = [rng.standard_normal((n, 6)) for n in (3, 5, 1)]
    allrows = np.concatenate(batches)
    want = sum(np.outer(r, r) for r in allrows) / 9
    assert np.allclose(oh.gram(batches, 9), want, atol=1e-12)


def test_apply_passes_unknown_modules_through():
    g = {"a": np.ones((2, 3)), "b": np.arange(6.0).reshape(2, 3)}
    h = {"a": 2 * np.eye(3)}
    out = oh.apply_dense(g, h)
    assert np.allclose(out["a"], 2 * np.ones((2, 3))) and np.allclose(out["b"], g["b"])


# ---- the package's host-side preparation (torch on the CPU, no kernel involved) against the oracle -------------
@pytest.mark.parametrize("mode", ["damped_inverse", "tikhonov_filtered", "pseudoinverse", "factored_tikhonov"])
@pytest.mark.parametrize("power", [-1.0, -0.5])
def test_package_inversion_matches_the_oracle(mode, power):
    from bergson_amd.hessians import invert_psd_matrix

    H = _spd(24, 3)
    got = invert_psd_matrix(torch.from_numpy(H).float(), mode, 0.1, power)
    assert got.dtype == torch.float32
    want = oh.invert_psd(H.astype(np.float32), mode, 0.1, power)
    assert np.abs(got.double().numpy() - want).max() <= 1e-5 * np.abs(want).max()


def test_package_rejects_unknown_inversion():
    from bergson_amd.hessians import eigenvalue_multiplier

    with pytest.raises(ValueError):
        eigenvalue_multiplier("cauchy", torch.ones(3), torch.tensor(1.0), 0.1)
