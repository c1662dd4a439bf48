"""Seeded projection matrices (bergson/collector/collector.py:1029-1063)."""
from __future__ import annotations

import hashlib
import math

import numpy as np
import torch


def identifier_seed(identifier: str) -> int:
    """md5 of the identifier, big-endian, reduced mod 2**63 - 1 (collector.py:1040-1042)."""
    digest = hashlib.md5(identifier.encode("utf-8")).digest()
    return int.from_bytes(digest, byteorder="big") % (2**63 - 1)


def projection_matrix(identifier: str, m: int, n: int, dtype: torch.dtype, projection_type: str = "normal",
                      projection_scale: str = "jl") -> torch.Tensor:
    """[m, n] matrix drawn on the CPU generator in `dtype` (collector.py:1044-1063)."""
    seed = identifier_seed(identifier)
    if projection_type == "normal":
        gen = torch.Generator("cpu").manual_seed(seed)
        A = torch.randn(m, n, dtype=dtype, generator=gen)
    elif projection_type == "rademacher":
        raw = np.random.Generator(np.random.PCG64(seed)).bytes((m * n + 7) // 8)
        bits = np.unpackbits(np.frombuffer(raw, dtype=np.uint8))[: m * n].reshape(m, n)
        A = torch.from_numpy(bits).to(dtype=dtype)
        A = A.add_(-0.5).mul_(2)
    else:
        raise ValueError(f"Unknown projection type: {projection_type}")
    if projection_scale == "row_norm":
        A /= A.norm(dim=1, keepdim=True)
    else:
        A /= math.sqrt(m)
    return A


def module_projections(name: str, p: int, out_features: int, in_features: int, dtype: torch.dtype,
                       projection_type: str = "normal", projection_scale: str = "jl",
                       collect_bias: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """(left [p, O], right [p, I (+1 with bias)]) for module `name` (collector.py:336-362, :540, :575-576)."""
    left = projection_matrix(f"{name}/left", p, out_features, dtype, projection_type, projection_scale)
    right = projection_matrix(f"{name}/right", p, in_features + int(collect_bias), dtype, projection_type,
                              projection_scale)
    return left, right
