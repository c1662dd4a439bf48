"""Synthetic models, documents and optimizer moments of the benchmark configurations.

Nothing is downloaded: models are random-initialised from `transformers` configs of the stated shapes,
token ids are uniform random, lengths and second moments come from seeded numpy generators.
"""
from __future__ import annotations

import numpy as np
import torch

NEOX_SHAPES = {
    # name: (layers, d_model, heads, mlp, rotary_pct)
    "pythia-14m": (6, 128, 4, 512, 0.25),
    "pythia-160m": (12, 768, 12, 3072, 0.25),
    "pythia-410m": (24, 1024, 16, 4096, 0.25),
}


def make_gpt_neox(shape: str, dtype: torch.dtype, device, *, seed: int = 0, vocab: int = 50304,
                  max_positions: int = 4096, layers: int | None = None):
    """Random-init GPT-NeoX of a Pythia shape, prepared as the reference prepares models for collection:
    every parameter frozen except the input embedding (bergson/utils/worker_utils.py:224-225), so that
    autograd computes activation gradients only."""
    from transformers import GPTNeoXConfig, GPTNeoXForCausalLM

    n_layers, d, heads, mlp, rotary = NEOX_SHAPES[shape]
    cfg = GPTNeoXConfig(vocab_size=vocab, hidden_size=d, num_hidden_layers=layers or n_layers,
                        num_attention_heads=heads, intermediate_size=mlp, rotary_pct=rotary,
                        max_position_embeddings=max_positions, use_cache=False,
                        hidden_dropout=0.0, attention_dropout=0.0)
    torch.manual_seed(seed)
    model = GPTNeoXForCausalLM(cfg).to(dtype)
    model.requires_grad_(False)
    model.get_input_embeddings().requires_grad_(True)
    model.eval()
    return model.to(device)


def make_llama(dtype: torch.dtype, device, *, layers: int = 32, d: int = 4096, heads: int = 32, kv_heads: int = 8,
               mlp: int = 14336, vocab: int = 128256, seed: int = 0, max_positions: int = 4096):
    """Random-init Llama-3-8B-shaped decoder (shape arguments allow reduced copies for tests), frozen except
    for the input embedding like `make_gpt_neox`.  The parameters are drawn directly on `device` in `dtype`:
    the full 32-layer shape is 16 GB in bf16, which a GPU initialises in seconds."""
    from transformers import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(vocab_size=vocab, hidden_size=d, num_hidden_layers=layers, num_attention_heads=heads,
                      num_key_value_heads=kv_heads, intermediate_size=mlp, max_position_embeddings=max_positions,
                      use_cache=False, attention_dropout=0.0, tie_word_embeddings=False)
    torch.manual_seed(seed)
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        with torch.device(device):
            model = LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    model.requires_grad_(False)
    model.get_input_embeddings().requires_grad_(True)
    model.eval()
    return model


def lognormal_lengths(n_docs: int, *, mu: float = 6.0, sigma: float = 1.0, lo: int = 16, hi: int = 2048,
                      seed: int = 0) -> list[int]:
    rng = np.random.default_rng(seed)
    return np.clip(np.round(rng.lognormal(mu, sigma, n_docs)), lo, hi).astype(np.int64).tolist()


def random_docs(lengths: list[int], vocab: int = 50304, seed: int = 0) -> list[list[int]]:
    rng = np.random.default_rng(seed + 1)
    return [rng.integers(0, vocab, size=l).tolist() for l in lengths]


class ListDataset:
    """Minimal stand-in for a `datasets.Dataset` of token ids: `len`, `column_names`, `ds[list_of_indices]`.
    Optional per-document columns: `labels` (token labels, -100 = not supervised) and `advantage`."""

    def __init__(self, docs: list[list[int]], *, labels: list[list[int]] | None = None,
                 advantage: list[float] | None = None):
        self.docs = docs
        self.columns = {"input_ids": docs, "length": [len(d) for d in docs]}
        if labels is not None:
            self.columns["labels"] = labels
        if advantage is not None:
            self.columns["advantage"] = advantage
        self.column_names = list(self.columns)

    def __len__(self) -> int:
        return len(self.docs)

    def __getitem__(self, key):
        if isinstance(key, str):
            return self.columns[key]
        if isinstance(key, (list, tuple)):
            return {name: [col[i] for i in key] for name, col in self.columns.items()}
        return {name: col[key] for name, col in self.columns.items()}


def adafactor_moments(base_model, *, scale: float = 1e-4, seed: int = 0) -> dict[str, tuple[torch.Tensor, torch.Tensor]]:
    """name -> (row [O], col [I]) second moments |N(0,1)| * scale for every nn.Linear of `base_model`."""
    rng = np.random.default_rng(seed + 2)
    out = {}
    for name, mod in base_model.named_modules():
        if isinstance(mod, torch.nn.Linear):
            row = torch.from_numpy(np.abs(rng.standard_normal(mod.out_features)).astype(np.float32) * scale)
            col = torch.from_numpy(np.abs(rng.standard_normal(mod.in_features)).astype(np.float32) * scale)
            out[name] = (row, col)
    return out
