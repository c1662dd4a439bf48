"""bergson_amd: MI355X-native projected per-example gradient collection and gradient-store scoring.

The public names mirror the part of `bergson`'s surface that sits on that path
(bergson/__init__.py:5-62).  All arithmetic of the path runs in hand-written
HIP kernels behind the C ABI of `include/bergson_amd.h`; there is no CPU path.
"""
from .attributor import Attributor
from .build import build, create_processor
from .builder import Builder
from .collection import collect_gradients
from .collector import CollectorComputer, HookCollectorBase, create_projection_matrix, fwd_bwd_factory
from .config import AttentionConfig, IndexConfig, InversionConfig, PreprocessConfig, QueryConfig, ScoreConfig
from .data import (
    TokenGradients,
    allocate_batches,
    create_index,
    create_token_index,
    load_gradients,
    load_module_gradients,
    load_scores,
    load_token_gradients,
    pad_and_tensor,
)
from .gradient_collectors import GradientCollector, StreamingGradientCollector, TraceCollector
from .hessians import DensePreconditioner, invert_psd_matrix, load_preconditioner
from .gradients import AdafactorNormalizer, AdamNormalizer, GradientProcessor, LayerAdapter, Normalizer
from .in_memory_collector import InMemoryCollector
from .optimizer_state import load_from_optimizer
from .process_grads import normalize_and_aggregate_grads, normalize_flat_grad
from .score import create_scorer, get_query_grads, score_dataset
from .scorer import Scorer

__all__ = [
    "Attributor", "Builder", "collect_gradients", "CollectorComputer", "HookCollectorBase",
    "create_projection_matrix", "fwd_bwd_factory", "AttentionConfig", "IndexConfig", "PreprocessConfig",
    "QueryConfig", "ScoreConfig", "TokenGradients", "allocate_batches", "create_index", "create_token_index",
    "load_gradients", "load_module_gradients", "load_scores", "load_token_gradients", "pad_and_tensor",
    "GradientCollector", "StreamingGradientCollector", "TraceCollector", "AdafactorNormalizer", "AdamNormalizer",
    "GradientProcessor", "LayerAdapter", "Normalizer", "InMemoryCollector", "normalize_and_aggregate_grads",
    "normalize_flat_grad", "Scorer", "InversionConfig", "DensePreconditioner", "invert_psd_matrix",
    "load_preconditioner", "load_from_optimizer", "build", "create_processor", "create_scorer", "get_query_grads", "score_dataset",
]


def __getattr__(name: str):
    # the Trainer callback pulls in transformers' trainer modules: imported on first use only
    if name in ("GradientCollectorCallback", "prepare_for_gradient_collection"):
        from . import huggingface

        return getattr(huggingface, name)
    raise AttributeError(f"module 'bergson_amd' has no attribute {name!r}")
