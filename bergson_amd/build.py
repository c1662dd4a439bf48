"""Thin `build` entry point: dataset -> on-disk gradient store (bergson/build.py:31-145).

Model loading, tokenisation and process launching are the caller's business (they are outside this
package): `build` takes a model that already sits on the GPU and a dataset of token ids, and does what
`build_worker` + `build` do from there on -- processor, batch allocation, collection into
`<run_path>.part`, and the rename to `<run_path>` once everything is written.
"""
from __future__ import annotations

import shutil

from .collection import collect_gradients
from .config import AttentionConfig, IndexConfig, PreprocessConfig
from .data import allocate_batches
from .gradients import GradientProcessor, Normalizer


def create_processor(cfg: IndexConfig, normalizers: dict[str, Normalizer] | None = None) -> GradientProcessor:
    """GradientProcessor carrying the projection settings of `cfg` (bergson/utils/worker_utils.py:63-100)."""
    return GradientProcessor(
        normalizers=normalizers or {},
        projection_dim=cfg.projection_dim or None,
        reshape_to_square=cfg.reshape_to_square,
        projection_type=cfg.projection_type,
        projection_target=cfg.projection_target,
        projection_scale=cfg.projection_scale,
        include_bias=cfg.include_bias,
    )


def document_lengths(data) -> list[int]:
    if "length" in data.column_names:
        return list(data["length"])
    return [len(x) for x in data["input_ids"]]


def attention_cfgs_of(cfg: IndexConfig) -> dict[str, AttentionConfig]:
    return {module: cfg.attention for module in cfg.split_attention_modules}


def build(index_cfg: IndexConfig, preprocess_cfg: PreprocessConfig | None = None, *, model, data,
          processor: GradientProcessor | None = None, normalizers: dict[str, Normalizer] | None = None,
          batches: list[list[int]] | None = None, **collector_kwargs):
    """Collect every document's gradients into `<run_path>.part`, then move it to `<run_path>`.

    Returns the collector.  An interrupted build leaves the `.part` directory behind.
    """
    if not index_cfg.run_path:
        raise ValueError("index_cfg.run_path must name the store directory")
    preprocess_cfg = preprocess_cfg or PreprocessConfig()
    index_cfg.partial_run_path.mkdir(parents=True, exist_ok=True)
    processor = processor or create_processor(index_cfg, normalizers)
    if batches is None:
        batches = allocate_batches(document_lengths(data), index_cfg.token_batch_size,
                                   max_batch_size=index_cfg.max_batch_size)
    collector = collect_gradients(model, data, processor, index_cfg, batches=batches,
                                  target_modules=set(index_cfg.modules) if index_cfg.modules else None,
                                  attention_cfgs=attention_cfgs_of(index_cfg), preprocess_cfg=preprocess_cfg,
                                  **collector_kwargs)
    if collector.rank == 0:
        shutil.move(str(index_cfg.partial_run_path), index_cfg.run_path)
    return collector
