"""Batching, padding, loss and the whole collection loop on PyTorch CPU.

Follows bergson/data.py:190-377 (`allocate_batches`), :743-806
(`pad_and_tensor`), bergson/collector/collector.py:857-985 (the loop and
`fwd_bwd`), :435-472 (hook registration) and bergson/collection.py:11-45.
"""
from __future__ import annotations

import random

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from . import hooks
from .projection import module_projections, projection_matrix


def allocate_batches(doc_lengths: list[int], N: int, seed: int = 42, max_batch_size: int | None = None
                     ) -> list[list[int]]:
    """Greedy bin packing for a single worker (data.py:239-377 with world_size = 1)."""
    docs = sorted(((i, l) for i, l in enumerate(doc_lengths) if l >= 2), key=lambda x: x[1], reverse=True)
    if len(docs) < 1:
        raise RuntimeError("Not enough documents (with 2+ tokens) to distribute across workers.")
    if docs[0][1] > N:
        raise RuntimeError(f"At least one document is too long for the token batch size {N}.")
    batches: list[list[int]] = []
    cur: list[int] = []
    for idx, length in docs:
        if not cur:
            cur.append(idx)
            continue
        cost = max(length, doc_lengths[cur[0]]) * (len(cur) + 1)
        fits_count = max_batch_size is None or len(cur) + 1 <= max_batch_size
        if cost <= N and fits_count:
            cur.append(idx)
        else:
            batches.append(cur)
            cur = [idx]
    if cur:
        batches.append(cur)
    random.seed(seed)
    random.shuffle(batches)
    return batches


def pad_and_tensor(sequences: list[list[int]], labels: list[list[int]] | None = None, padding_value: int = 0):
    """(ids [N,S], labels [N,S] with -100 padding, collection_mask [N,S]) (data.py:743-806)."""
    if labels is None:
        labels = sequences
    max_len = max(len(s) for s in sequences)
    x = torch.tensor([s + [padding_value] * (max_len - len(s)) for s in sequences], dtype=torch.long)
    y = torch.tensor([l + [-100] * (max_len - len(l)) for l in labels], dtype=torch.long)
    lengths = torch.tensor([len(s) for s in sequences])
    mask = (torch.arange(max_len).unsqueeze(0) + 1) < lengths.unsqueeze(1)
    return x, y, mask


def losses_and_backward(model, x: Tensor, y: Tensor, loss_reduction: str = "sum", label_smoothing: float = 0.0,
                        advantage: list[float] | None = None) -> Tensor:
    """collector.py:948-983 (cross-entropy branch; `advantage` is the batch's optional "advantage" column,
    :975-976)."""
    logits = model(x).logits[:, :-1]
    masks = y[:, 1:] != -100
    denoms = masks.sum(dim=1, dtype=logits.dtype) if loss_reduction == "mean" else 1.0
    losses = F.cross_entropy(logits.reshape(-1, logits.size(-1)), y[:, 1:].flatten(), reduction="none",
                             label_smoothing=label_smoothing).reshape_as(y[:, 1:])
    losses = losses.sum(1) / denoms
    if advantage is not None:
        # in place by an fp32 tensor: the product is formed in fp32 and rounded once to the dtype of the losses
        losses *= torch.tensor(advantage, device=losses.device)
    losses.sum().backward()
    model.zero_grad()
    return losses


def target_linears(base_model: nn.Module) -> dict[str, nn.Linear]:
    """nn.Linear modules under the base model in named_modules order (collector.py:159-183)."""
    return {n: m for n, m in base_model.named_modules() if isinstance(m, nn.Linear)}


def collect(model, base_model: nn.Module, docs: list[list[int]], batches: list[list[int]], *, p: int | None,
            normalizers: dict | None = None, projection_type: str = "normal", attribute_tokens: bool = False,
            include_bias: bool = False, save_dtype: torch.dtype | None = None, loss_reduction: str = "sum",
            unit_normalize: bool = False, global_dim: int | None = None, label_smoothing: float = 0.0,
            labels: list[list[int]] | None = None, advantages: list[float] | None = None,
            device: str | torch.device = "cpu") -> tuple[Tensor, Tensor]:
    """The whole reference loop on CPU: returns (rows, losses).

    `device`: where the model lives and the hooks' tensor arithmetic runs.  "cpu" is the checker and the
    timed CPU baseline; with the model on a GPU the very same op sequence runs as stock PyTorch device ops --
    what the benchmark times beside the fused kernels as the sequence they replace.
    `labels` (per document, -100 = not supervised) and `advantages` (one factor per document) are the
    dataset's optional "labels" and "advantage" columns (collector.py:877-886, :975-976).

    rows is [num_docs, D] (per sequence) or [sum(max(len-1, 0)), D] (per token), in save_dtype.
    global_dim (with p=None) is projection_target="global": every module's unprojected gradient goes through
    its block of one [global_dim, sum of module sizes] projection and the blocks are summed
    (collector.py:364-402), so D = global_dim.
    """
    from .store import preprocess, token_offsets

    normalizers = normalizers or {}
    targets = target_linears(base_model)
    param_dtype = next(model.parameters()).dtype
    save_dtype = save_dtype or param_dtype
    lo, hi = torch.finfo(save_dtype).min, torch.finfo(save_dtype).max
    proj = {}
    stash: dict[str, Tensor] = {}
    mod_grads: dict[str, Tensor] = {}
    state = {"mask": None}

    def get_proj(name, mod, dtype):
        if p is None:
            return None, None
        if name not in proj:
            bias = include_bias and mod.bias is not None
            proj[name] = tuple(t.to(device) for t in module_projections(
                name, p, mod.out_features, mod.in_features, dtype, projection_type, "jl", bias))
        return proj[name]

    def fwd(name):
        def hook(mod, inp, _out):
            a = inp[0].detach()
            bias = include_bias and mod.bias is not None
            _, right = get_proj(name, mod, a.dtype)
            stash[name] = hooks.forward_hook(a, normalizers.get(name), right, bias)
        return hook

    def bwd(name):
        def hook(mod, _gin, gout):
            g = gout[0].detach()
            bias = include_bias and mod.bias is not None
            left, right = get_proj(name, mod, g.dtype)
            P = hooks.backward_hook(stash.pop(name), g, normalizers.get(name), left, right, collect_bias=bias,
                                    attribute_tokens=attribute_tokens, collection_mask=state["mask"], lo=lo, hi=hi)
            if global_dim is not None:
                R = projection_matrix(f"{name}/single", global_dim, P.shape[1], P.dtype, projection_type, "jl"
                                      ).to(device)
                mod_grads["gradients"] = hooks.accumulate_global_projection(mod_grads.get("gradients"), P, R)
            else:
                mod_grads[name] = P.to(save_dtype)
        return hook

    handles = []
    for name, mod in targets.items():
        handles.append(mod.register_forward_hook(fwd(name)))
        handles.append(mod.register_full_backward_hook(bwd(name)))

    lengths = [len(d) for d in docs]
    offsets = token_offsets(lengths)
    rows = None
    losses_out = torch.zeros(len(docs), dtype=torch.float32)
    try:
        for indices in batches:
            x, y, mask = pad_and_tensor([docs[i] for i in indices],
                                        None if labels is None else [labels[i] for i in indices])
            x, y, mask = x.to(device), y.to(device), mask.to(device)
            state["mask"] = mask
            losses = losses_and_backward(model, x, y, loss_reduction, label_smoothing,
                                         None if advantages is None else [advantages[i] for i in indices])
            if global_dim is not None:  # finalize_global_projection, collector.py:392-402
                mod_grads["gradients"] = mod_grads["gradients"].to(save_dtype)
                grad_sizes = {"gradients": global_dim}
            else:
                grad_sizes = {n: mod_grads[n].shape[1] for n in targets}
            g = preprocess(mod_grads, grad_sizes, unit_normalize)
            mod_grads.clear()
            if rows is None:
                n_rows = int(offsets[-1]) if attribute_tokens else len(docs)
                rows = torch.zeros(n_rows, g.shape[1], dtype=save_dtype, device=device)
            if attribute_tokens:
                r = 0
                for idx in indices:
                    n = int(offsets[idx + 1] - offsets[idx])
                    rows[int(offsets[idx]):int(offsets[idx + 1])] = g[r:r + n]
                    r += n
            else:
                rows[indices] = g
            losses_out[indices] = losses.detach().float().cpu()
    finally:
        for h in handles:
            h.remove()
    return rows, losses_out
