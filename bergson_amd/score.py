"""Thin `score` entry points: score a dataset on the fly against a query store
(bergson/score/score.py:51-256, :259-431).

`get_query_grads` reads the query store, `create_scorer` normalises / aggregates the queries and builds
the `Scorer` with its memory-mapped writer, `score_dataset` runs the collection loop with that scorer
(one pass per query slice when `query_batch_size` is set).  A dense Hessian at `preprocess_cfg.hessian_path`
preconditions the queries once and, in split mode, every batch of index rows.
"""
from __future__ import annotations

import shutil
from pathlib import Path

import numpy as np
import torch

from .build import attention_cfgs_of, create_processor, document_lengths
from .collection import collect_gradients
from .config import IndexConfig, PreprocessConfig, ScoreConfig
from .data import allocate_batches, column_offsets, load_gradients, load_info, store_base_dtype
from .gradients import GradientProcessor
from .process_grads import normalize_and_aggregate_grads
from .score_writer import MemmapSequenceScoreWriter, MemmapTokenScoreWriter
from .scorer import Scorer
from .utils import convert_precision_to_torch, get_gradient_dtype, numpy_to_tensor


def get_query_grads(score_cfg: ScoreConfig, query_range: tuple[int, int] | None = None) -> dict[str, torch.Tensor]:
    """Per-module query gradients from the store at `score_cfg.query_path` (score.py:51-103); fills
    `score_cfg.modules` with the store's modules when it is empty."""
    query_path = Path(score_cfg.query_path)
    if not query_path.exists():
        raise FileNotFoundError(f"Query dataset not found at {score_cfg.query_path}. "
                                "Please build a query dataset index first.")
    info = load_info(query_path)
    grad_sizes = info["grad_sizes"]
    if not score_cfg.modules:
        score_cfg.modules = list(grad_sizes)
    mmap = load_gradients(query_path)
    if query_range is not None:
        mmap = mmap[query_range[0]:query_range[1]]
    base = store_base_dtype(info)
    grads = {}
    for name, (lo, hi) in column_offsets(grad_sizes).items():
        t = numpy_to_tensor(np.array(mmap[:, lo:hi]), base)
        grads[name] = t.float() if base == "bfloat16" else t
    return grads


def create_scorer(path: Path, data, score_cfg: ScoreConfig, preprocess_cfg: PreprocessConfig, device: torch.device,
                  dtype: torch.dtype, *, attribute_tokens: bool = False, query_range: tuple[int, int] | None = None,
                  num_queries_total: int | None = None) -> Scorer:
    """Scorer with a memory-mapped writer at `path` (score.py:138-256)."""
    query_grads = get_query_grads(score_cfg, query_range)
    # H^-1/2 on both sides when the scores are cosines (split mode), H^-1 on the queries otherwise
    # (score.py:167-192).  The query store is taken to hold raw gradients.
    from .hessians import load_preconditioner, make_split_hessian

    preconditioner = load_preconditioner(preprocess_cfg.hessian_path, inversion_cfg=preprocess_cfg.inversion_cfg,
                                         power=-0.5 if preprocess_cfg.unit_normalize else -1.0,
                                         ev_correction=preprocess_cfg.ev_correction, device=device)
    index_transform = None
    if preconditioner is not None:
        query_grads = preconditioner.apply({m: g.to(device) for m, g in query_grads.items()})
        if preprocess_cfg.unit_normalize:
            index_transform = make_split_hessian(preconditioner.h_inv, score_cfg.modules, device, dtype)
    if query_range is not None and preprocess_cfg.aggregation != "none":
        raise ValueError("query_batch_size requires aggregation='none': aggregation mixes gradients across "
                         "queries, which a row slice would corrupt.")
    if query_range is not None and score_cfg.score != "individual":
        raise ValueError("query_batch_size requires score='individual': 'nearest' reduces over all queries, "
                         "which per-chunk passes would compute wrongly.")
    query_grads = normalize_and_aggregate_grads(
        query_grads, score_cfg.modules, unit_normalize=preprocess_cfg.unit_normalize, device=device,
        aggregate_grads=preprocess_cfg.aggregation,
        normalize_aggregated_grad=preprocess_cfg.normalize_aggregated_grad)
    num_queries = len(query_grads[score_cfg.modules[0]])
    if score_cfg.score == "nearest":
        num_scores = 1
    else:
        num_scores = num_queries_total if num_queries_total is not None else num_queries
    if attribute_tokens:
        writer = MemmapTokenScoreWriter.from_dataset(Path(path), data, num_scores, dtype=dtype)
    else:
        writer = MemmapSequenceScoreWriter(Path(path), len(data), num_scores, dtype=dtype)
    return Scorer(query_grads=query_grads, modules=score_cfg.modules, writer=writer, device=device, dtype=dtype,
                  unit_normalize=preprocess_cfg.unit_normalize, score_mode=score_cfg.score,
                  attribute_tokens=attribute_tokens,
                  query_offset=query_range[0] if query_range is not None else 0,
                  **({"index_transform": index_transform} if index_transform is not None else {}))


def score_dataset(index_cfg: IndexConfig, score_cfg: ScoreConfig, preprocess_cfg: PreprocessConfig | None = None, *,
                  model, data, processor: GradientProcessor | None = None, batches: list[list[int]] | None = None):
    """Score every document of `data` against the query store; scores land in `<run_path>/scores.bin`.

    With `score_cfg.query_batch_size` the whole dataset is passed once per query slice, each pass filling
    its own columns of the same score file (score.py:337-363).
    """
    if not index_cfg.run_path:
        raise ValueError("index_cfg.run_path must name the score directory")
    preprocess_cfg = preprocess_cfg or PreprocessConfig()
    part = index_cfg.partial_run_path
    part.mkdir(parents=True, exist_ok=True)
    if processor is None:
        # score with the projection the query store was built with
        processor = GradientProcessor.load(Path(score_cfg.query_path), map_location=str(model.device))
    if batches is None:
        batches = allocate_batches(document_lengths(data), index_cfg.token_batch_size,
                                   max_batch_size=index_cfg.max_batch_size)
    dtype = get_gradient_dtype(model) if score_cfg.precision == "auto" else convert_precision_to_torch(score_cfg.precision)
    num_queries = load_info(Path(score_cfg.query_path))["num_grads"]
    if score_cfg.query_batch_size:
        ranges = [(lo, min(num_queries, lo + score_cfg.query_batch_size))
                  for lo in range(0, num_queries, score_cfg.query_batch_size)]
    else:
        ranges = [None]
    scorer = None
    for qr in ranges:
        scorer = create_scorer(part, data, score_cfg, preprocess_cfg, torch.device(model.device), dtype,
                               attribute_tokens=index_cfg.attribute_tokens, query_range=qr,
                               num_queries_total=num_queries if qr is not None else None)
        collect_gradients(model, data, processor, index_cfg, batches=batches,
                          target_modules=set(score_cfg.modules) if score_cfg.modules else None,
                          attention_cfgs=attention_cfgs_of(index_cfg), scorer=scorer,
                          preprocess_cfg=PreprocessConfig())
        scorer.writer.flush()
    shutil.move(str(part), index_cfg.run_path)
    return scorer
