"""Score stores (bergson/score/score_writer.py).

`scores.bin` holds one structured record per document (or per token, with
`offsets.npy`): for every query i a `score_i` value followed by a one-byte
`written_i` flag, each pair aligned to the next power of two, the record
padded to 8 bytes (`_score_struct_dtype`, score_writer.py:16-58).  Batches are
written through strided views of the mapped file, all query columns of a batch
in one assignment.
"""
from __future__ import annotations

import json
from abc import ABC, abstractmethod
from pathlib import Path
from typing import Any

import numpy as np
import torch
import torch.distributed as dist

from .data import compute_num_token_grads
from .utils import BF16_NAME, dtype_name, storage_np_dtype, tensor_to_numpy


def _score_struct_dtype(num_scores: int, score_dtype_name: str) -> tuple[dict, dict]:
    """(numpy dtype spec, JSON-safe spec) of the interleaved (score_i, written_i) record."""
    np_dtype = storage_np_dtype(score_dtype_name)
    score_size = np_dtype.itemsize
    pair_size = score_size + 1
    aligned_pair_size = 1 << (pair_size - 1).bit_length()
    names, formats, json_formats, offsets = [], [], [], []
    for i in range(num_scores):
        names += [f"score_{i}", f"written_{i}"]
        formats += [np_dtype, "bool"]
        json_formats += [score_dtype_name, "bool"]
        offsets += [i * aligned_pair_size, i * aligned_pair_size + score_size]
    itemsize = ((num_scores * aligned_pair_size + 7) // 8) * 8
    spec = {"names": names, "formats": formats, "offsets": offsets, "itemsize": itemsize}
    spec_json = {"names": names, "formats": json_formats, "offsets": offsets, "itemsize": itemsize}
    return spec, spec_json


class ScoreWriter(ABC):
    scores: Any

    @abstractmethod
    def __call__(self, indices: list[int], scores: torch.Tensor, query_offset: int = 0):
        """Write `scores` [rows, width] at query columns query_offset.. of the given documents."""

    @abstractmethod
    def flush(self): ...


class InMemorySequenceScoreWriter(ScoreWriter):
    def __init__(self, num_items: int, num_scores: int, dtype: torch.dtype = torch.float32):
        self.scores = torch.zeros((num_items, num_scores), device="cpu", dtype=dtype)

    def __call__(self, indices: list[int], scores: torch.Tensor, query_offset: int = 0):
        width = scores.shape[1]
        self.scores[indices, query_offset:query_offset + width] = scores.to(dtype=self.scores.dtype).cpu()

    def flush(self):
        pass


class InMemoryTokenScoreWriter(ScoreWriter):
    def __init__(self, data, num_scores: int, dtype: torch.dtype = torch.float32):
        self.num_token_grads = compute_num_token_grads(data)
        self.offsets = np.zeros(len(self.num_token_grads) + 1, dtype=np.int64)
        np.cumsum(self.num_token_grads, out=self.offsets[1:])
        self.scores = [torch.zeros((int(n), num_scores), device="cpu", dtype=dtype) for n in self.num_token_grads]
        self.dtype = dtype

    def __call__(self, indices: list[int], scores: torch.Tensor, query_offset: int = 0):
        host = scores.to(dtype=self.dtype).cpu()
        width = host.shape[1]
        row = 0
        for idx in indices:
            sl = int(self.num_token_grads[idx])
            self.scores[idx][:, query_offset:query_offset + width] = host[row:row + sl]
            row += sl

    def flush(self):
        pass


class _MemmapScoreWriter(ScoreWriter):
    """Creates / reopens scores.bin + info.json and exposes strided score / flag views."""

    def __init__(self, path: Path, num_items: int, num_rows: int, num_scores: int, *, attribute_tokens: bool,
                 dtype: torch.dtype, flush_interval: int, overwrite: bool, distributed: bool,
                 offsets: np.ndarray | None):
        self.path = Path(path)
        self.num_scores = num_scores
        self.dtype = dtype
        self.flush_interval = flush_interval
        self.num_batches_since_flush = 0
        self.path.mkdir(parents=True, exist_ok=True)
        scores_file_path = self.path / "scores.bin"
        name = dtype_name(dtype)
        spec, spec_json = _score_struct_dtype(num_scores, name)
        struct = np.dtype(spec)
        synchronize = distributed and dist.is_initialized()
        rank = dist.get_rank() if synchronize else 0
        if rank == 0 and (overwrite or not scores_file_path.exists()):
            print(f"Creating new scores file: {scores_file_path}")
            if num_rows > 0:
                np.memmap(str(scores_file_path), dtype=struct, mode="w+", shape=(num_rows,)).flush()
            else:
                scores_file_path.write_bytes(b"")
            with (self.path / "info.json").open("w") as f:
                json.dump({"attribute_tokens": attribute_tokens, "num_items": num_items, "num_rows": num_rows,
                           "num_scores": num_scores, "dtype": spec_json}, f, indent=2)
            if offsets is not None:
                np.save(self.path / "offsets.npy", offsets)
        if synchronize:
            dist.barrier()
        if num_rows > 0:
            self.scores = np.memmap(str(scores_file_path), dtype=struct, mode="r+", shape=(num_rows,))
        else:
            self.scores = np.zeros((0,), dtype=struct)
        score_np = storage_np_dtype(name)
        pair = spec["offsets"][2] if num_scores > 1 else struct.itemsize
        self._score_view = np.ndarray((num_rows, num_scores), dtype=score_np, buffer=self.scores, offset=0,
                                      strides=(struct.itemsize, pair))
        self._flag_view = np.ndarray((num_rows, num_scores), dtype=np.bool_, buffer=self.scores,
                                     offset=score_np.itemsize, strides=(struct.itemsize, pair))

    def _put(self, rows, scores: torch.Tensor, query_offset: int) -> None:
        host = tensor_to_numpy(scores.to(dtype=self.dtype).cpu())
        width = host.shape[1]
        self._score_view[rows, query_offset:query_offset + width] = host
        self._flag_view[rows, query_offset:query_offset + width] = True
        self.num_batches_since_flush += 1
        if self.num_batches_since_flush >= self.flush_interval:
            self.flush()

    def flush(self):
        if isinstance(self.scores, np.memmap):
            self.scores.flush()
        self.num_batches_since_flush = 0


class MemmapSequenceScoreWriter(_MemmapScoreWriter):
    """One record per document (score_writer.py:283-368).  An existing scores.bin is reused unless
    `overwrite`, so an interrupted run resumes and query slices fill further columns."""

    def __init__(self, path: Path, num_items: int, num_scores: int, *, dtype: torch.dtype = torch.float32,
                 flush_interval: int = 64, overwrite: bool = False, distributed: bool = True):
        super().__init__(path, num_items, num_items, num_scores, attribute_tokens=False, dtype=dtype,
                         flush_interval=flush_interval, overwrite=overwrite, distributed=distributed, offsets=None)

    def __call__(self, indices: list[int], scores: torch.Tensor, query_offset: int = 0):
        self._put(np.asarray(indices, dtype=np.int64), scores, query_offset)


class MemmapTokenScoreWriter(_MemmapScoreWriter):
    """One record per token; document i owns rows offsets[i]:offsets[i+1] (score_writer.py:147-245)."""

    def __init__(self, path: Path, num_token_grads: np.ndarray, num_scores: int, *,
                 dtype: torch.dtype = torch.float32, flush_interval: int = 64, overwrite: bool = False,
                 distributed: bool = True):
        self.num_token_grads = np.asarray(num_token_grads, dtype=np.int64)
        self.offsets = np.zeros(len(self.num_token_grads) + 1, dtype=np.int64)
        np.cumsum(self.num_token_grads, out=self.offsets[1:])
        super().__init__(path, len(self.num_token_grads), int(self.offsets[-1]), num_scores, attribute_tokens=True,
                         dtype=dtype, flush_interval=flush_interval, overwrite=overwrite, distributed=distributed,
                         offsets=self.offsets)

    @classmethod
    def from_dataset(cls, path: Path, data, num_scores: int, **kwargs):
        return cls(path, compute_num_token_grads(data), num_scores, **kwargs)

    def __call__(self, indices: list[int], scores: torch.Tensor, query_offset: int = 0):
        rows = np.concatenate([np.arange(self.offsets[i], self.offsets[i + 1]) for i in indices]) if indices else \
            np.zeros((0,), dtype=np.int64)
        assert len(rows) == scores.shape[0], f"{scores.shape[0]} score rows for {len(rows)} token rows"
        self._put(rows, scores, query_offset)


def save_sequence_scores(path: Path, scores: np.ndarray, *, dtype: torch.dtype = torch.float32) -> None:
    """One-shot writer for a full [num_items, num_scores] matrix (score_writer.py:371-388)."""
    if scores.ndim == 1:
        scores = scores[:, None]
    num_items, num_scores = scores.shape
    writer = MemmapSequenceScoreWriter(path, num_items, num_scores, dtype=dtype, overwrite=True, distributed=False)
    writer(list(range(num_items)), torch.from_numpy(np.ascontiguousarray(scores)))
    writer.flush()


def save_token_scores(path: Path, scores: np.ndarray, offsets: np.ndarray, *, dtype: torch.dtype = torch.float32
                      ) -> None:
    """One-shot writer for a flat [total_tokens, num_scores] array (score_writer.py:248-280)."""
    if scores.ndim == 1:
        scores = scores[:, None]
    num_token_grads = np.diff(offsets).astype(np.int64)
    writer = MemmapTokenScoreWriter(path, num_token_grads, scores.shape[1], dtype=dtype, overwrite=True,
                                    distributed=False)
    writer(list(range(len(num_token_grads))), torch.from_numpy(np.ascontiguousarray(scores)))
    writer.flush()
