"""On-disk gradient / score stores, batch allocation and padding.

Byte-compatible with the reference's formats (bergson/data.py): `gradients.bin`
is a raw row-major [num_grads, sum(grad_sizes)] array of `base_dtype`,
`info.json` carries {attribute_tokens, num_items, num_grads, grad_sizes,
base_dtype}, per-token stores add `offsets.npy`.  numpy has no bfloat16, so a
bfloat16 store is mapped as uint16 bit patterns; `info.json` still says
"bfloat16" and the bytes are the same.
"""
from __future__ import annotations

import heapq
import json
import os
import random
from pathlib import Path
from typing import Any, Iterator

import numpy as np
import torch
import torch.distributed as dist
from numpy.lib.recfunctions import structured_to_unstructured

from .utils import BF16_NAME, storage_np_dtype


def _dtype_name(dtype) -> str:
    """Accepts a numpy dtype, a dtype name or torch.bfloat16 / 'bfloat16'."""
    if isinstance(dtype, str):
        return dtype
    if isinstance(dtype, torch.dtype):
        from .utils import dtype_name

        return dtype_name(dtype)
    return np.dtype(dtype).name


def _lengths_of(data) -> np.ndarray:
    cols = data.column_names
    if "length" in cols:
        return np.asarray(data["length"], dtype=np.int64)
    if "input_ids" in cols:
        return np.asarray([len(x) for x in data["input_ids"]], dtype=np.int64)
    return np.asarray([len(x) for x in data["labels"]], dtype=np.int64)


def compute_num_token_grads(data) -> np.ndarray:
    """Per-token rows stored per example: max(length - 1, 0) (bergson/data.py:37-62)."""
    return np.maximum(_lengths_of(data) - 1, 0)


def _rank() -> int:
    return dist.get_rank() if dist.is_initialized() else 0


def _allocate_file(path: Path, nbytes: int) -> None:
    with open(path, "wb") as f:
        f.truncate(nbytes)
        os.fsync(f.fileno())


def _create_store(root: Path, n_rows: int, grad_sizes: dict[str, int], dtype, *, num_items: int,
                  offsets: np.ndarray | None) -> np.ndarray:
    """The files of a gradient store and a writable map of its rows: `gradients.bin` (n_rows x sum(grad_sizes) raw
    values, sized without writing zeros and synced before any other rank maps it), `info.json`, and for a ragged
    per-token store `offsets.npy` (bergson/data.py:65-137, :392-445).  Rank 0 creates, everyone maps."""
    root = Path(root)
    name = _dtype_name(dtype)
    np_dtype = storage_np_dtype(name)
    width = sum(grad_sizes.values())
    rows_file = root / "gradients.bin"
    if _rank() == 0:
        root.mkdir(parents=True, exist_ok=True)
        _allocate_file(rows_file, n_rows * width * np_dtype.itemsize)
        if offsets is not None:
            np.save(root / "offsets.npy", offsets)
        info = {"attribute_tokens": offsets is not None, "num_items": num_items, "num_grads": n_rows,
                "grad_sizes": grad_sizes, "base_dtype": name}
        (root / "info.json").write_text(json.dumps(info, indent=2))
    if dist.is_initialized():
        dist.barrier()
    if n_rows == 0:  # an empty file cannot be mapped
        return np.zeros((0, width), dtype=np_dtype)
    return np.memmap(rows_file, dtype=np_dtype, mode="r+", shape=(n_rows, width))


def create_token_index(root: Path, num_token_grads: np.ndarray, grad_sizes: dict[str, int], dtype
                       ) -> tuple[np.memmap, np.ndarray]:
    """Ragged per-token store: rows offsets[i] .. offsets[i + 1] belong to example i (bergson/data.py:65-137)."""
    offsets = np.concatenate(([0], np.cumsum(num_token_grads, dtype=np.int64))).astype(np.int64)
    rows = _create_store(root, int(offsets[-1]), grad_sizes, dtype, num_items=len(num_token_grads), offsets=offsets)
    return rows, offsets  # type: ignore[return-value]


def create_index(root: Path, num_grads: int, grad_sizes: dict[str, int], dtype) -> np.memmap:
    """Flat store: row i is example i (bergson/data.py:392-445)."""
    return _create_store(root, num_grads, grad_sizes, dtype, num_items=num_grads, offsets=None)  # type: ignore[return-value]


def column_offsets(grad_sizes: dict[str, int]) -> dict[str, tuple[int, int]]:
    """(start, end) columns of each module in grad_sizes order (bergson/data.py:380-389)."""
    offsets, start = {}, 0
    for name, size in grad_sizes.items():
        offsets[name] = (start, start + size)
        start += size
    return offsets


def load_info(root_dir: Path | str) -> dict:
    with (Path(root_dir) / "info.json").open("r") as f:
        return json.load(f)


def store_base_dtype(info: dict) -> str:
    """`base_dtype`, or the scalar dtype of an old structured store (bergson/data.py:508-512)."""
    if "base_dtype" in info:
        return info["base_dtype"]
    fmt = info["dtype"]["formats"][0]
    return BF16_NAME if "bfloat16" in str(fmt) or str(fmt) == "|V2" else np.dtype(fmt).base.name


def load_gradients(root_dir: Path | str) -> np.memmap:
    """Read-only map of the flat [num_grads, total_grad_dim] array (bergson/data.py:492-519).

    A bfloat16 store comes back as uint16 bit patterns; `utils.numpy_to_tensor(arr, 'bfloat16')` reinterprets them.
    """
    root_dir = Path(root_dir)
    info = load_info(root_dir)
    np_dtype = storage_np_dtype(store_base_dtype(info))
    return np.memmap(root_dir / "gradients.bin", dtype=np_dtype, mode="r",
                     shape=(info["num_grads"], sum(info["grad_sizes"].values())))


def load_token_gradients(root_dir: Path | str) -> tuple[np.memmap, np.ndarray, np.ndarray]:
    """(mmap, num_token_grads, offsets) of a per-token store (bergson/data.py:138-156)."""
    root_dir = Path(root_dir)
    mmap = load_gradients(root_dir)
    offsets = np.load(root_dir / "offsets.npy")
    return mmap, np.diff(offsets).astype(np.int64), offsets


class TokenGradients:
    """`tg[i]` = example i's [num_token_grads[i], grad_dim] rows (bergson/data.py:159-183)."""

    def __init__(self, root_dir: Path | str):
        self.mmap, self._num_token_grads, self._offsets = load_token_gradients(root_dir)

    @property
    def num_token_grads(self) -> np.ndarray:
        return self._num_token_grads

    def __len__(self) -> int:
        return len(self._num_token_grads)

    def __getitem__(self, i: int) -> np.ndarray:
        return np.asarray(self.mmap[self._offsets[i]:self._offsets[i + 1]])


class ModuleGradients:
    """Module-name-keyed column views over a flat store (bergson/data.py:522-548)."""

    def __init__(self, mmap: np.memmap, grad_sizes: dict[str, int]):
        self.mmap = mmap
        self.offsets = column_offsets(grad_sizes)

    def __getitem__(self, name: str) -> np.ndarray:
        lo, hi = self.offsets[name]
        return self.mmap[:, lo:hi]

    def __len__(self) -> int:
        return len(self.mmap)

    def __iter__(self) -> Iterator[str]:
        return iter(self.offsets)

    def __contains__(self, name: str) -> bool:
        return name in self.offsets

    def keys(self):
        return self.offsets.keys()


def load_module_gradients(root_dir: Path | str) -> ModuleGradients:
    root_dir = Path(root_dir)
    return ModuleGradients(load_gradients(root_dir), load_info(root_dir)["grad_sizes"])


class Scores:
    """A score store: structured (score_i, written_i) rows (bergson/data.py:587-644)."""

    def __init__(self, mmap: np.memmap, info: dict[str, Any], offsets: np.ndarray | None = None):
        self.mmap = mmap
        self.info = info
        self.offsets = offsets
        self.num_scores = info["num_scores"]
        self._score_fields = [f"score_{i}" for i in range(self.num_scores)]

    def __len__(self) -> int:
        return self.info["num_items"]

    def __getitem__(self, key: Any) -> np.ndarray:
        return structured_to_unstructured(self.mmap[key][self._score_fields])

    def get(self, key: Any, score_idx: int = 0) -> np.ndarray:
        return self.mmap[key][f"score_{score_idx}"]

    def is_written(self) -> bool:
        return all(np.all(self.mmap[f"written_{i}"]) for i in range(self.num_scores))

    def to_grid(self) -> torch.Tensor:
        """Per-token store -> zero-padded [docs, seq_len(, num_scores)] grid."""
        assert self.offsets is not None, "to_grid() requires a per-token store"
        tokens_per_doc = np.diff(self.offsets).astype(np.int64)
        seq_len = int(tokens_per_doc.max()) + 1
        grid = np.zeros((len(self), seq_len, self.num_scores), dtype=np.float32)
        for doc in range(len(self)):
            grid[doc, :tokens_per_doc[doc]] = self[self.offsets[doc]:self.offsets[doc + 1]]
        scores = torch.from_numpy(grid)
        return scores[..., 0] if self.num_scores == 1 else scores


def score_np_dtype(info_dtype: dict) -> np.dtype:
    """numpy structured dtype from the JSON spec; bfloat16 score fields map as 2-byte voids."""
    formats = ["V2" if f == BF16_NAME else f for f in info_dtype["formats"]]
    return np.dtype({"names": info_dtype["names"], "formats": formats, "offsets": info_dtype["offsets"],
                     "itemsize": info_dtype["itemsize"]})


def load_scores(path: Path | str) -> Scores:
    """bergson/data.py:647-664."""
    path = Path(path)
    info = load_info(path)
    mmap = np.memmap(path / "scores.bin", dtype=score_np_dtype(info["dtype"]), mode="r", shape=(info["num_rows"],))
    offsets = np.load(path / "offsets.npy") if info.get("attribute_tokens") else None
    return Scores(mmap, info, offsets)


# ---- batching ---------------------------------------------------------------------------

def allocate_batches(doc_lengths: list[int], N: int, seed: int = 42, max_batch_size: int | None = None
                     ) -> list[list[int]]:
    """This rank's batches under `max_len_in_batch * batch_size <= N` (bergson/data.py:190-236)."""
    rank = dist.get_rank() if dist.is_initialized() else 0
    world_size = dist.get_world_size() if dist.is_initialized() else 1
    (batches,) = _allocate_batches_world(doc_lengths, N, world_size, seed, ranks=[rank],
                                         max_batch_size=max_batch_size)
    return batches


def pack_by_padded_cost(doc_lengths: list[int], budget: int, max_batch_size: int | None = None) -> list[list[int]]:
    """Batches of document indices under `longest document * documents <= budget` (bergson/data.py:290-322).

    Documents are taken longest first (equal lengths in index order), and a batch is filled until the next
    document would break the budget or the size limit.  Since the first document of a batch is its longest,
    a batch headed by a document of length L holds exactly min(budget // L, max_batch_size) documents
    (fewer only at the end of the data), so the batches are consecutive runs of the sorted order and no
    per-document test is needed.  Documents with fewer than two tokens have no next-token label and are left
    out (their rows of the store stay zero)."""
    lengths = np.asarray(doc_lengths, dtype=np.int64)
    order = np.argsort(-lengths, kind="stable")
    order = order[lengths[order] >= 2]
    if order.size and lengths[order[0]] > budget:
        raise RuntimeError(f"At least one document is too long for the token batch size {budget}.")
    batches, at = [], 0
    while at < order.size:
        room = int(budget // lengths[order[at]])
        if max_batch_size is not None:
            room = min(room, max_batch_size)
        batches.append(order[at:at + max(room, 1)].tolist())
        at += max(room, 1)
    return batches


def spread_over_ranks(batches: list[list[int]], world_size: int) -> list[list[list[int]]]:
    """Makes the number of batches a multiple of `world_size` by peeling single documents off existing
    batches, and deals them out round-robin: result[r] = batches r, r + world_size, ... (bergson/data.py:
    324-369).  With fewer batches than ranks, documents are first split off the currently largest batch
    (the earliest such batch on ties) until every rank has one; the batch order after that step is the
    array order of Python's binary heap under the keys (-size, insertion number), as in the reference."""
    if world_size == 1:
        return [batches]
    if len(batches) < world_size:
        ticket = len(batches)
        heap: list[tuple[int, int, list[int]]] = []
        for t, b in enumerate(batches):
            heapq.heappush(heap, (-len(b), t, b))
        while len(heap) < world_size:
            _, _, largest = heapq.heappop(heap)
            if len(largest) < 2:
                raise RuntimeError("Not enough documents to give each worker at least one batch.")
            peeled = [largest.pop()]
            heapq.heappush(heap, (-len(largest), ticket, largest))
            heapq.heappush(heap, (-1, ticket + 1, peeled))
            ticket += 2
        batches = [entry[2] for entry in heap]
    missing = -len(batches) % world_size
    visit = 0
    while missing and visit < len(batches):
        donor = batches[visit % len(batches)]
        visit += 1
        if len(donor) > 1:
            batches.append([donor.pop()])
            missing -= 1
    if missing:
        raise AssertionError("Could not construct a number of batches divisible by the world size. If variability "
                             "of item lengths in your dataset is low consider using a different dataset size or "
                             "token batch size.")
    return [batches[r::world_size] for r in range(world_size)]


def _allocate_batches_world(doc_lengths: list[int], N: int, world_size: int, seed: int = 42,
                            ranks: list[int] | None = None, max_batch_size: int | None = None
                            ) -> list[list[list[int]]]:
    """The batches of the given ranks (all when None): `pack_by_padded_cost`, `spread_over_ranks`, then each
    rank's list shuffled by `random.seed(seed); random.shuffle` (bergson/data.py:239-377)."""
    doc_lengths = list(doc_lengths)
    usable = sum(1 for n in doc_lengths if n >= 2)
    if usable < len(doc_lengths) and _rank() == 0:
        print(f"Skipping {len(doc_lengths) - usable} documents with fewer than 2 tokens (no valid next-token labels).")
    if usable < world_size:
        raise RuntimeError("Not enough documents (with 2+ tokens) to distribute across workers.")
    per_rank = spread_over_ranks(pack_by_padded_cost(doc_lengths, N, max_batch_size), world_size)
    assert all(max(doc_lengths[i] for i in b) * len(b) <= N for share in per_rank for b in share)
    picked = []
    for r in (range(world_size) if ranks is None else ranks):
        random.seed(seed)
        random.shuffle(per_rank[r])
        picked.append(per_rank[r])
    return picked


def pad_and_tensor(sequences: list[list[int]], labels: list[list[int]] | None = None, *, padding_value: int = 0,
                   dtype: torch.dtype | None = torch.long, device: torch.device | None = None,
                   sync_max_len: bool = True) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(padded ids, padded labels (-100), shift_loss_masks, collection_masks) (bergson/data.py:743-806).

    collection_masks[n, s] = s + 1 < len(sequences[n]): every real position but the last.
    shift_loss_masks[n, s] = labels[n, s + 1] is supervised (False in the last column).
    Everything is laid out on the host -- two [N, S] integer arrays filled row by row -- and uploaded once; the
    masks are computed on the device from the uploaded labels and lengths.
    """
    labels = sequences if labels is None else labels
    lengths = [len(seq) for seq in sequences]
    width = max(lengths)
    if sync_max_len and dist.is_initialized():
        widest = torch.tensor(width, device=device)
        dist.all_reduce(widest, op=dist.ReduceOp.MAX)
        width = int(widest)
    ids = np.full((len(sequences), width), padding_value, dtype=np.int64)
    lab = np.full((len(sequences), width), -100, dtype=np.int64)
    for n, (seq, label) in enumerate(zip(sequences, labels)):
        ids[n, :len(seq)] = seq
        lab[n, :len(label)] = label
    tokens, labels_t = torch.from_numpy(ids), torch.from_numpy(lab)
    if dtype is not None and dtype != torch.long:
        tokens, labels_t = tokens.to(dtype), labels_t.to(dtype)
    tokens = tokens.to(device, non_blocking=True)
    labels_t = labels_t.to(device, non_blocking=True)
    supervised_next = torch.nn.functional.pad(labels_t[:, 1:] != -100, (0, 1), value=False)
    lengths_t = torch.tensor(lengths).to(device, non_blocking=True)
    collection_masks = torch.arange(1, width + 1, device=device).unsqueeze(0) < lengths_t.unsqueeze(1)
    return tokens, labels_t, supervised_next, collection_masks
