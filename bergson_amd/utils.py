"""dtype helpers of the boundary (bergson/utils/utils.py:119-202)."""
from __future__ import annotations

import numpy as np
import torch
from torch import Tensor

_DTYPE_PRIORITY = {torch.float64: 0, torch.float32: 1, torch.float16: 2, torch.bfloat16: 3}

# numpy has no bfloat16: bf16 stores are mapped as uint16 bit patterns and named by string
BF16_NAME = "bfloat16"


def get_gradient_dtype(model) -> torch.dtype:
    """dtype of the parameters that require grad; widest first when mixed (utils.py:119-138)."""
    dtypes = {p.dtype for p in model.parameters() if p.requires_grad and p.dtype.is_floating_point}
    assert len(dtypes) > 0, "No trainable parameters found"
    if len(dtypes) == 1:
        return dtypes.pop()
    ordered = sorted(dtypes, key=lambda d: _DTYPE_PRIORITY.get(d, 99))
    print(f"Multiple gradient dtypes found: {dtypes}. Using {ordered[0]}.")
    return ordered[0]


def dtype_name(dtype: torch.dtype) -> str:
    """The `base_dtype` string written to info.json (numpy dtype name; 'bfloat16' for bf16)."""
    return {torch.float16: "float16", torch.float32: "float32", torch.float64: "float64",
            torch.bfloat16: BF16_NAME}[dtype]


def torch_dtype_from_name(name: str) -> torch.dtype:
    return {"float16": torch.float16, "float32": torch.float32, "float64": torch.float64,
            BF16_NAME: torch.bfloat16}[name]


def storage_np_dtype(name: str) -> np.dtype:
    """numpy dtype used to map a store of base dtype `name` (uint16 bit patterns for bfloat16)."""
    return np.dtype(np.uint16) if name == BF16_NAME else np.dtype(name)


def tensor_to_numpy(t: Tensor) -> np.ndarray:
    """CPU tensor -> numpy without changing bits (bf16 as uint16) (utils.py:144-154)."""
    if t.dtype == torch.bfloat16:
        return t.view(torch.uint16).numpy()
    return t.numpy()


def numpy_to_tensor(arr: np.ndarray, base_dtype: str | None = None) -> Tensor:
    """numpy -> CPU tensor without changing bits (utils.py:157-174); uint16 + 'bfloat16' -> bf16."""
    if base_dtype == BF16_NAME or arr.dtype.str == "|V2":
        return torch.from_numpy(np.ascontiguousarray(arr).view(np.uint16).copy()).view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(arr))


def convert_precision_to_torch(precision: str) -> torch.dtype:
    return {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[precision]
