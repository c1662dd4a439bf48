"""Scoring of gradient rows against queries.

Follows bergson/score/scorer.py:89-115 (`Scorer.score`),
bergson/query/attributor.py:125-167 and :169-235 (`Attributor`), and
bergson/process_grads.py:139-182 (`normalize_and_aggregate_grads`).
"""
from __future__ import annotations

import torch
from torch import Tensor


def scorer_score(index_grads: dict[str, Tensor], query_grads: dict[str, Tensor], modules: list[str], *,
                 dtype: torch.dtype = torch.float32, unit_normalize: bool = False,
                 score_mode: str = "individual") -> Tensor:
    """scores[b, q] = sum_m g_b[m] . q_q[m], index side optionally unit-normalised (scorer.py:89-115)."""
    scores = None
    sq_norm = None
    for m in modules:
        g = index_grads[m].to(dtype)
        part = g @ query_grads[m].to(dtype).T
        scores = part if scores is None else scores.add_(part)
        if unit_normalize:
            n = g.pow(2).sum(dim=1)
            sq_norm = n if sq_norm is None else sq_norm.add_(n)
    assert scores is not None
    if unit_normalize:
        scores.div_(sq_norm.sqrt().clamp_min_(1e-12).unsqueeze(1))
    if score_mode == "nearest":
        return scores.max(dim=-1, keepdim=True).values
    return scores


def normalize_and_aggregate_queries(query_grads: dict[str, Tensor], modules: list[str], *, unit_normalize: bool,
                                    aggregation: str = "none", normalize_aggregated: bool = False
                                    ) -> dict[str, Tensor]:
    """process_grads.py:139-182: fp32 per-query unit norm over all modules, then mean / sum over queries, then
    (optionally) one norm over everything that is left; nothing to do = inputs returned in their dtype."""
    if aggregation == "none" and not unit_normalize:
        return {m: query_grads[m] for m in modules}
    q = {m: query_grads[m].to(torch.float32) for m in modules}
    if unit_normalize:
        norms = torch.cat([q[m] for m in modules], dim=1).norm(dim=1, keepdim=True)
        q = {m: q[m] / norms for m in modules}
    if aggregation == "mean":
        q = {m: q[m].mean(dim=0, keepdim=True) for m in modules}
    elif aggregation == "sum":
        q = {m: q[m].sum(dim=0, keepdim=True) for m in modules}
    if normalize_aggregated:
        norm = torch.cat([q[m].flatten() for m in modules], dim=0).norm()
        q = {m: q[m] / norm for m in modules}
    return q


def attributor_normalize_index(grads: dict[str, Tensor], modules: list[str]) -> dict[str, Tensor]:
    """attributor.py:137-167: g / sqrt(sum over all modules of g^2), NaN/inf -> 0."""
    norm_sq = sum((torch.square(grads[m]).sum(dim=1, keepdim=True) for m in modules), start=0.0)
    norm = norm_sq**0.5
    return {m: torch.nan_to_num(grads[m] / norm, nan=0.0, posinf=0.0, neginf=0.0) for m in modules}


def attributor_search(index_grads: dict[str, Tensor], queries: dict[str, Tensor], modules: list[str], k: int | None,
                      *, dtype: torch.dtype = torch.float32, unit_norm: bool = False, reverse: bool = False):
    """attributor.py:169-235 without FAISS / preconditioning: returns (values [Q, k], indices [Q, k])."""
    grads = {m: index_grads[m].to(dtype) for m in modules}
    if unit_norm:
        grads = attributor_normalize_index(grads, modules)
    q = {m: queries[m].to(dtype).clone() for m in modules}
    if unit_norm:
        norm = torch.cat([q[m] for m in modules], dim=1).norm(dim=1, keepdim=True)
        for m in modules:
            q[m] /= norm + torch.finfo(norm.dtype).eps
    n = next(iter(grads.values())).shape[0]
    k = min(k or n, n)
    scores = torch.stack([q[m] @ grads[m].mT for m in modules], dim=-1).sum(-1)
    return torch.topk(scores, k, largest=not reverse)
