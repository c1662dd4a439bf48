"""The hook pair of one module: normaliser scaling, projection, token reduction.

Follows bergson/collector/collector.py:518-543 (forward hook) and :592-743
(`_compute_gradient`), with the normalisers of bergson/gradients.py:276-400.
Every op runs in the dtype of its operands, as in the reference, so that the
rounding points at bf16 are the reference's.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import Tensor


@dataclass
class Adafactor:
    """Row [O] / column [I] second moments (gradients.py:276-298)."""

    row: Tensor
    col: Tensor
    bias_avg_sq: Tensor | None = None


@dataclass
class Adam:
    """Full second moments [O, I] (gradients.py:366-378)."""

    weight_avg_sq: Tensor
    bias_avg_sq: Tensor | None = None


def adafactor_normalize_weight(grad: Tensor, n: Adafactor, eps: float = 1e-30) -> Tensor:
    """Closed form on a full [.., O, I] gradient (gradients.py:300-337)."""
    r, c = n.row.add(eps), n.col.add(eps)
    a = r.mean().sqrt() * r.rsqrt()
    b = c.rsqrt()
    return grad * a[:, None] * b[None, :]


def adafactor_normalize_bias(grad: Tensor, n: Adafactor, eps: float = 1e-8) -> Tensor:
    """eps inside the square root (gradients.py:339-349)."""
    assert n.bias_avg_sq is not None
    return grad * n.bias_avg_sq.add(eps).rsqrt()


def adam_normalize_weight(grad: Tensor, n: Adam, eps: float = 1e-8) -> Tensor:
    """eps outside the square root; in place in the reference, so the result keeps grad's dtype
    (gradients.py:380-388)."""
    return grad.clone().div_(n.weight_avg_sq.sqrt().add_(eps))


def adam_normalize_bias(grad: Tensor, n: Adam, eps: float = 1e-8) -> Tensor:
    """gradients.py:390-400."""
    assert n.bias_avg_sq is not None
    return grad / (n.bias_avg_sq.sqrt() + eps)


def forward_hook(a: Tensor, normalizer, right: Tensor | None, collect_bias: bool = False) -> Tensor:
    """What the forward hook stashes for the backward hook (collector.py:518-543).

    a [N, S, I]; right [p, I (+1)] or None when not projecting.
    """
    if isinstance(normalizer, Adam):
        return a
    if isinstance(normalizer, Adafactor):
        a_factor = normalizer.col.add(1e-30).rsqrt()
        a = a * a_factor.type_as(a)
    if right is not None and not collect_bias:
        a = a @ right.T
    return a


def _with_bias_projection(g: Tensor, a: Tensor, bias_grad: Tensor, left: Tensor, right: Tensor, i: int,
                          attribute_tokens: bool) -> Tensor:
    """collector.py:552-590: L @ [g^T a | b] @ R^T without forming the [O, I+1] matrix."""
    rt = right.T  # [I+1, p]
    gp = g @ left.T
    ap = a @ rt[:i]
    bp = bias_grad @ left.T
    if attribute_tokens:
        P = gp.unsqueeze(-1) * ap.unsqueeze(-2)
    else:
        P = gp.mT @ ap
    return P + bp.unsqueeze(-1) * rt[i]


def backward_hook(stash: Tensor, g: Tensor, normalizer, left: Tensor | None, right: Tensor | None, *,
                  collect_bias: bool = False, attribute_tokens: bool = False, collection_mask: Tensor | None = None,
                  lo: float = float("-inf"), hi: float = float("inf")) -> Tensor:
    """`_compute_gradient` (collector.py:592-743).

    stash: what forward_hook returned; g [N, S, O].
    left [p, O] / right [p, I(+1)] or both None when projection is off.
    Returns [N, grad_dim], or [n_valid_tokens, grad_dim] when attribute_tokens.
    """
    a = stash
    project = left is not None
    o = g.shape[-1]

    if isinstance(normalizer, Adam):  # :609-644
        i = a.shape[-1]
        if collect_bias:
            b = adam_normalize_bias(g, normalizer)
            bias_grad = b if attribute_tokens else b.sum(dim=1)
        else:
            bias_grad = None
        if attribute_tokens:
            P = g.unsqueeze(-1) * a.unsqueeze(-2)
            P = adam_normalize_weight(P, normalizer)
            if bias_grad is not None:
                P = torch.cat([P, bias_grad.unsqueeze(-1)], dim=-1)
            if project:
                P = left @ P @ right.T
            P = P.flatten(2)[collection_mask]
        else:
            P = g.mT @ a
            P = adam_normalize_weight(P, normalizer)
            if bias_grad is not None:
                P = torch.cat([P, bias_grad.unsqueeze(2)], dim=2)
            if project:
                P = left @ P @ right.T
    elif isinstance(normalizer, Adafactor):  # :646-700
        if collect_bias:
            b = adafactor_normalize_bias(g, normalizer)
            bias_grad = b if attribute_tokens else b.sum(dim=1)
        else:
            bias_grad = None
        g_factor = normalizer.row.add(1e-30)
        g_factor = g_factor.mean().sqrt() * g_factor.rsqrt()
        g = g * g_factor.type_as(g)
        P = _no_adam_tail(a, g, bias_grad, left, right, attribute_tokens, collection_mask)
    else:  # :701-740
        if collect_bias:
            bias_grad = g if attribute_tokens else g.sum(dim=1)
        else:
            bias_grad = None
        P = _no_adam_tail(a, g, bias_grad, left, right, attribute_tokens, collection_mask)

    return P.flatten(1).clamp_(lo, hi)


def _no_adam_tail(a: Tensor, g: Tensor, bias_grad: Tensor | None, left: Tensor | None, right: Tensor | None,
                  attribute_tokens: bool, collection_mask: Tensor | None) -> Tensor:
    """Shared tail of the Adafactor and no-normaliser branches (collector.py:660-700, :711-740)."""
    project = left is not None
    if bias_grad is not None and project:
        i = right.shape[1] - 1
        P = _with_bias_projection(g, a, bias_grad, left, right, i, attribute_tokens)
        if attribute_tokens:
            P = P.flatten(2)[collection_mask]
        return P
    if bias_grad is None and project:
        g = g @ left.T  # a was projected in the forward hook
    if attribute_tokens:
        P = g.unsqueeze(-1) * a.unsqueeze(-2)
        if bias_grad is not None:
            P = torch.cat([P, bias_grad.unsqueeze(-1)], dim=-1)
        return P.flatten(2)[collection_mask]
    P = g.mT @ a
    if bias_grad is not None:
        P = torch.cat([P, bias_grad.unsqueeze(2)], dim=2)
    return P


def module_gradient(a: Tensor, g: Tensor, normalizer, left: Tensor | None, right: Tensor | None, **kw) -> Tensor:
    """forward_hook followed by backward_hook for one module."""
    stash = forward_hook(a, normalizer, right, kw.get("collect_bias", False))
    return backward_hook(stash, g, normalizer, left, right, **kw)


def accumulate_global_projection(acc: Tensor | None, P: Tensor, R_single: Tensor) -> Tensor:
    """`accumulate_global_projection` (collector.py:364-390): P [rows, O*I(+O)] is the clamped, flattened
    gradient of one module, R_single [proj_dim, P.shape[1]] that module's block of the global projection;
    the projected blocks of all modules are added in the model dtype."""
    projected = P @ R_single.T
    if acc is None:
        return projected
    return acc.add_(projected)
