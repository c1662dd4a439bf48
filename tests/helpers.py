"""Shared helpers of the parity tests."""
from __future__ import annotations

import torch


def rel_l2(x: torch.Tensor, ref: torch.Tensor) -> float:
    x = x.detach().double().cpu()
    ref = ref.detach().double().cpu()
    denom = ref.norm().item()
    return (x - ref).norm().item() / (denom if denom > 0 else 1.0)


# tolerances of the projected-gradient parity (relative L2 against the reference op sequence)
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}
