"""Pins the oracle's hook arithmetic against autograd and closed forms (fp32 / fp64, CPU).

Identities restated from the reference's tests/test_gradients.py and tests/test_attribute_tokens.py:
  * batch of one: hook output == L @ normalize(W.grad [| b.grad]) @ R^T with W.grad from autograd;
  * batch of N: hook output row n == the same from a per-sample backward;
  * Adafactor closed form (row_factor = sqrt(mean r) * rsqrt(r), col_factor = rsqrt(c), eps 1e-30)
    and Adam closed form (grad / (sqrt(v) + 1e-8));
  * the per-token rows of a sequence sum to its per-sequence row;
and brute force over explicit loops in fp64 on tiny shapes.
"""
import pytest
import torch
import torch.nn as nn

from oracle import hooks as H
from oracle.projection import module_projections


def _capture(lin: nn.Linear, x: torch.Tensor, loss_fn):
    """Runs x through lin, returns (a, g) as module hooks would see them, plus per-sample W / b grads."""
    cap = {}
    h1 = lin.register_forward_hook(lambda m, i, o: cap.__setitem__("a", i[0].detach()))
    h2 = lin.register_full_backward_hook(lambda m, gi, go: cap.__setitem__("g", go[0].detach()))
    x = x.clone().requires_grad_(True)
    loss_fn(lin(x)).backward()
    h1.remove(), h2.remove()
    wg, bg = [], []
    for n in range(x.shape[0]):
        lin.zero_grad()
        loss_fn(lin(x[n:n + 1].detach())).backward()
        wg.append(lin.weight.grad.clone())
        bg.append(lin.bias.grad.clone() if lin.bias is not None else None)
    return cap["a"], cap["g"], wg, bg


def _loss(out):
    return (out.pow(2) * torch.linspace(0.5, 1.5, out.shape[-1])).sum() + out.sin().sum()


def _normalizer(kind, O, I, bias, gen):
    if kind == "adafactor":
        return H.Adafactor(torch.rand(O, generator=gen) + 0.1, torch.rand(I, generator=gen) + 0.1,
                           torch.rand(O, generator=gen) + 0.1 if bias else None)
    if kind == "adam":
        return H.Adam(torch.rand(O, I, generator=gen) + 0.1, torch.rand(O, generator=gen) + 0.1 if bias else None)
    return None


def _closed_form(w, b, norm):
    """normalize(W.grad [| b.grad]) by the published formulas, written without the oracle's helpers."""
    if isinstance(norm, H.Adafactor):
        r, c = norm.row + 1e-30, norm.col + 1e-30
        w = w * (r.mean().sqrt() / r.sqrt())[:, None] / c.sqrt()[None, :]
        if b is not None:
            b = b / (norm.bias_avg_sq + 1e-8).sqrt()
    elif isinstance(norm, H.Adam):
        w = w / (norm.weight_avg_sq.sqrt() + 1e-8)
        if b is not None:
            b = b / (norm.bias_avg_sq.sqrt() + 1e-8)
    return w if b is None else torch.cat([w, b[:, None]], dim=1)


@pytest.mark.parametrize("kind", [None, "adafactor", "adam"])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("p", [None, 4])
def test_per_sample_gradient_matches_autograd(kind, bias, p):
    torch.manual_seed(0)
    gen = torch.Generator().manual_seed(1)
    N, S, I, O = 3, 5, 7, 6
    lin = nn.Linear(I, O, bias=True)
    x = torch.randn(N, S, I, generator=gen)
    a, g, wg, bg = _capture(lin, x, _loss)
    norm = _normalizer(kind, O, I, bias, gen)
    left = right = None
    if p is not None:
        left, right = module_projections("toy", p, O, I, torch.float32, collect_bias=bias)
    got = H.module_gradient(a, g, norm, left, right, collect_bias=bias)
    for n in range(N):
        full = _closed_form(wg[n], bg[n] if bias else None, norm)
        want = full if p is None else left @ full @ right.T
        torch.testing.assert_close(got[n], want.flatten(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("kind", [None, "adafactor", "adam"])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("p", [None, 4])
def test_token_rows_sum_to_sequence_row(kind, bias, p):
    gen = torch.Generator().manual_seed(2)
    N, S, I, O = 2, 6, 5, 4
    a = torch.randn(N, S, I, generator=gen)
    g = torch.randn(N, S, O, generator=gen)
    norm = _normalizer(kind, O, I, bias, gen)
    left = right = None
    if p is not None:
        left, right = module_projections("toy2", p, O, I, torch.float32, collect_bias=bias)
    lengths = torch.tensor([6, 4])
    mask = (torch.arange(S)[None] + 1) < lengths[:, None]
    g = g * torch.cat([mask[:, :, None]], dim=0)  # zero where nothing is collected, as a causal model gives
    seq = H.module_gradient(a, g, norm, left, right, collect_bias=bias)
    tok = H.module_gradient(a, g, norm, left, right, collect_bias=bias, attribute_tokens=True, collection_mask=mask)
    assert tok.shape[0] == int(mask.sum())
    torch.testing.assert_close(tok[:5].sum(0), seq[0], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(tok[5:].sum(0), seq[1], rtol=1e-4, atol=1e-5)


def test_projected_adafactor_brute_force_fp64():
    gen = torch.Generator().manual_seed(3)
    N, S, I, O, p = 2, 3, 4, 3, 2
    a = torch.randn(N, S, I, generator=gen, dtype=torch.float64)
    g = torch.randn(N, S, O, generator=gen, dtype=torch.float64)
    L = torch.randn(p, O, generator=gen, dtype=torch.float64)
    R = torch.randn(p, I, generator=gen, dtype=torch.float64)
    row = torch.rand(O, generator=gen, dtype=torch.float64) + 0.1
    col = torch.rand(I, generator=gen, dtype=torch.float64) + 0.1
    got = H.module_gradient(a, g, H.Adafactor(row, col), L, R)
    rmean = sum(float(r) + 1e-30 for r in row) / O
    for n in range(N):
        for i in range(p):
            for j in range(p):
                acc = 0.0
                for s in range(S):
                    for o in range(O):
                        for k in range(I):
                            f = (rmean ** 0.5) / ((float(row[o]) + 1e-30) ** 0.5) / ((float(col[k]) + 1e-30) ** 0.5)
                            acc += float(L[i, o]) * float(g[n, s, o]) * float(a[n, s, k]) * f * float(R[j, k])
                assert got[n, i * p + j].item() == pytest.approx(acc, rel=1e-10, abs=1e-12)


def test_clamp_bounds_applied():
    a = torch.full((1, 2, 2), 100.0)
    g = torch.full((1, 2, 2), 100.0)
    out = H.module_gradient(a, g, None, None, None, lo=-5.0, hi=5.0)
    assert out.tolist() == [[5.0] * 4]


def test_normalizer_helpers_match_closed_forms():
    gen = torch.Generator().manual_seed(4)
    G = torch.randn(3, 5, generator=gen)
    n = H.Adafactor(torch.rand(3, generator=gen) + 0.1, torch.rand(5, generator=gen) + 0.1, torch.rand(3, generator=gen))
    torch.testing.assert_close(H.adafactor_normalize_weight(G, n), _closed_form(G, None, n))
    m = H.Adam(torch.rand(3, 5, generator=gen), torch.rand(3, generator=gen))
    torch.testing.assert_close(H.adam_normalize_weight(G, m), G / (m.weight_avg_sq.sqrt() + 1e-8))
    b = torch.randn(3, generator=gen)
    torch.testing.assert_close(H.adam_normalize_bias(b, m), b / (m.bias_avg_sq.sqrt() + 1e-8))
    torch.testing.assert_close(H.adafactor_normalize_bias(b, n), b / (n.bias_avg_sq + 1e-8).sqrt())


def test_global_projection_is_the_projection_of_the_concatenated_gradient():
    """projection_target="global" (collector.py:364-402): summing each module's block `P_m @ R_m^T` equals
    projecting the concatenation of the per-sample autograd gradients with the concatenated blocks, and the
    blocks are the matrices named "<module>/single"."""
    from oracle.projection import projection_matrix

    torch.manual_seed(0)
    gen = torch.Generator().manual_seed(3)
    N, S, pd = 3, 4, 5
    lins = {"m.a": nn.Linear(6, 5), "m.b": nn.Linear(5, 7)}
    acc = None
    grads, blocks = [], []
    for name, lin in lins.items():
        x = torch.randn(N, S, lin.in_features, generator=gen)
        a, g, wg, _ = _capture(lin, x, _loss)
        P = H.module_gradient(a, g, None, None, None)
        R = projection_matrix(f"{name}/single", pd, P.shape[1], torch.float32)
        acc = H.accumulate_global_projection(acc, P, R)
        grads.append(torch.stack([w.flatten() for w in wg]))
        blocks.append(R)
    want = torch.cat(grads, dim=1) @ torch.cat(blocks, dim=1).T
    assert acc.shape == (N, pd)
    torch.testing.assert_close(acc, want, rtol=1e-4, atol=1e-5)
