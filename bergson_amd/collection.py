"""`collect_gradients` convenience entry point (bergson/collection.py:11-45)."""
from __future__ import annotations

from .collector import CollectorComputer
from .config import AttentionConfig, IndexConfig, PreprocessConfig
from .gradient_collectors import GradientCollector
from .gradients import GradientProcessor


def collect_gradients(model, data, processor: GradientProcessor, cfg: IndexConfig, *,
                      batches: list[list[int]] | None = None, target_modules: set[str] | None = None,
                      attention_cfgs: dict[str, AttentionConfig] | None = None, scorer=None,
                      preprocess_cfg: PreprocessConfig | None = None, overlap_backward: bool | None = None,
                      **collector_kwargs):
    """Hooks `model.base_model`, runs every batch and writes the store at `cfg.partial_run_path`.

    Returns the collector (the reference returns None; callers that ignore the result are unaffected).
    `overlap_backward` is handed to `CollectorComputer`; other extra keywords go to `GradientCollector`.
    """
    collector = GradientCollector(
        model=model.base_model,
        cfg=cfg,
        processor=processor,
        target_modules=target_modules,
        data=data,
        scorer=scorer,
        preprocess_cfg=preprocess_cfg or PreprocessConfig(),
        attention_cfgs=attention_cfgs or {},
        filter_modules=cfg.filter_modules,
        **collector_kwargs,
    )
    computer = CollectorComputer(model=model, data=data, collector=collector, batches=batches, cfg=cfg,
                                 overlap_backward=overlap_backward)
    computer.run_with_collector_hooks(desc="New worker - Collecting gradients")
    collector.total_processed = computer.total_processed
    return collector
