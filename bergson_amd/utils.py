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


class DeviceIndexRing:
    """Document indices of a batch as an int64 device tensor without stalling the host.

    A Python list handed to torch for indexing, or an unpinned CPU tensor moved to the GPU, is copied with a
    stream synchronisation: the host then waits for the whole backward pass it has just queued.  The lists
    go through a ring of pinned slots instead; a slot is reused only after the copy out of it has finished
    (an event per slot, normally long since signalled)."""

    def __init__(self, slots: int = 32):
        self.slots = slots
        self._buf: torch.Tensor | None = None
        self._events: list = [None] * slots
        self._next = 0
        self._last: tuple | None = None  # (key, tensor) of the most recent list: a batch asks more than once

    def get(self, indices, device: torch.device) -> torch.Tensor:
        key = (tuple(indices), str(device))
        if self._last is not None and self._last[0] == key:
            return self._last[1]
        n = len(indices)
        if self._buf is None or self._buf.shape[1] < n:
            if self._buf is not None:
                torch.cuda.synchronize()  # copies out of the old ring
            self._buf = torch.empty((self.slots, max(256, 2 * n)), dtype=torch.int64, pin_memory=True)
            self._events = [None] * self.slots
        i = self._next
        self._next = (i + 1) % self.slots
        if self._events[i] is not None:
            self._events[i].synchronize()
        row = self._buf[i, :n]
        row.copy_(torch.as_tensor(indices, dtype=torch.int64))
        out = row.to(device, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev
        self._last = (key, out)
        return out
