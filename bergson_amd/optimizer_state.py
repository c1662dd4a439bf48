"""Normalizers from a saved optimizer state (restates bergson/utils/load_from_optimizer.py:23-398, :513-542).

`load_from_optimizer(model, path)` reads an `optimizer.pt` (Adam / AdamW `exp_avg_sq`, Adafactor
`exp_avg_sq_row` / `exp_avg_sq_col`, bitsandbytes 8-bit Adam `state2`) and returns the
`AdamNormalizer` / `AdafactorNormalizer` of every weight matrix, keyed by the module's name
relative to `model.base_model` and oriented `[out, in]` -- what the collection hooks look up.

Host-side parsing only.  Differences from the reference, all forced by this environment: the file is
read with `torch.load(weights_only=True)` (an optimizer state holds tensors and plain containers);
`hf://` locations are refused (no network); PEFT models need the `peft` package, which is absent.
"""
from __future__ import annotations

from enum import Enum
from pathlib import Path

import torch
from torch import Tensor, nn

from .gradients import AdafactorNormalizer, AdamNormalizer, LayerAdapter, Normalizer


def load_optimizer(optimizer_state: str | Path) -> dict:
    """State dict from a file, or from `optimizer.pt` inside a checkpoint directory."""
    text = str(optimizer_state)
    if text.startswith("hf://"):
        raise NotImplementedError("optimizer states on the Hugging Face hub cannot be fetched here; download the "
                                  "file and pass its local path")
    local = Path(text)
    if not local.exists():
        raise FileNotFoundError(f"Optimizer state '{text}' is not a local path and does not start with 'hf://'.")
    path = local / "optimizer.pt" if local.is_dir() else local
    return torch.load(path, map_location="cpu", weights_only=True)


class OptimizerStateFormat(Enum):
    """How one parameter's second moments are stored: a full tensor, or Adafactor's row / column factors."""

    UNFACTORED = 1
    FACTORED = 2


_BNB_KEY = "__bnb_optimizer_quant_state__"  # bitsandbytes 8-bit Adam keeps its second moments under ["state2"]


def get_optimizer_state_format(param_state) -> OptimizerStateFormat | None:
    """Which of the two layouts a parameter's state entry has; None for anything else."""
    if isinstance(param_state, dict):
        quant = param_state.get(_BNB_KEY)
        if "exp_avg_sq" in param_state or (isinstance(quant, dict) and "state2" in quant):
            return OptimizerStateFormat.UNFACTORED
        if "exp_avg_sq_row" in param_state:
            return OptimizerStateFormat.FACTORED
    return None


def get_unfactored_second_moment(state: dict) -> Tensor:
    """The full second-moment tensor of an UNFACTORED entry (Adam, 8-bit Adam, Adafactor's 1-D parameters)."""
    return state["exp_avg_sq"] if "exp_avg_sq" in state else state[_BNB_KEY]["state2"]


def _base_model_prefix(model) -> str:
    """Dotted path of `model.base_model` inside `model`, with a trailing dot ("" when it is the model)."""
    base = getattr(model, "base_model", model)
    if base is model:
        return ""
    for name, module in model.named_modules():
        if module is base:
            return f"{name}." if name else ""
    return ""


def orient_second_moment(t: Tensor, out_dim: int, in_dim: int, layer=None) -> Tensor | None:
    """`t` as `[out, in]`.  A supported layer's class settles how it stores its weight (HF Conv1D keeps
    `[in, out]`), which shapes cannot do for square weights; otherwise the shapes decide.  None when
    nothing fits."""
    if layer is not None and isinstance(layer, LayerAdapter.supported_modules):
        oriented = t.T if LayerAdapter.weight_transposed(layer) else t
        return oriented.contiguous() if tuple(oriented.shape) == (out_dim, in_dim) else None
    if tuple(t.shape) == (out_dim, in_dim):
        return t.contiguous()
    if tuple(t.shape) == (in_dim, out_dim):
        return t.T.contiguous()
    return None


def _submodule(model, layer_name: str):
    try:
        return model.get_submodule(layer_name)
    except (AttributeError, ValueError):
        return None


def _orient_weight_second_moment(exp_avg_sq: Tensor, model, layer_name: str) -> Tensor:
    module = _submodule(model, layer_name)
    try:
        o = getattr(module, LayerAdapter.out_attr(module))
        i = getattr(module, LayerAdapter.in_attr(module))
    except (AttributeError, ValueError):
        return exp_avg_sq
    oriented = orient_second_moment(exp_avg_sq, o, i, layer=module)
    return exp_avg_sq if oriented is None else oriented


def _orient_factored_second_moment(row: Tensor, col: Tensor, model, layer_name: str) -> tuple[Tensor, Tensor]:
    """Adafactor reduces over the weight as stored, so a layer that stores `[in, out]` has its factors
    swapped with respect to what AdafactorNormalizer expects."""
    module = _submodule(model, layer_name)
    if module is not None and isinstance(module, LayerAdapter.supported_modules) and LayerAdapter.weight_transposed(module):
        return col, row
    return row, col


def _get_bias_second_moment(layer_name: str, param_index_to_name: dict[int, str], optimizer_state: dict,
                            include_bias: bool) -> Tensor | None:
    """Second moments of `<layer>.bias` when asked for and stored unfactored.  An entry that records its own
    `param_name` wins over the positional mapping."""
    if not include_bias:
        return None
    wanted = layer_name + ".bias"
    states = optimizer_state["state"]
    entry = next((e for e in states.values() if isinstance(e, dict) and e.get("param_name") == wanted), None)
    if entry is None:
        idx = next((i for i, name in param_index_to_name.items() if name == wanted), None)
        entry = states.get(idx) if idx is not None else None
    if get_optimizer_state_format(entry) != OptimizerStateFormat.UNFACTORED:
        return None
    return get_unfactored_second_moment(entry)


def _normalizer_of(state: dict, fmt: OptimizerStateFormat, bias: Tensor | None, device, model,
                   layer_name: str) -> Normalizer | None:
    """One weight's normalizer, oriented [out, in]; None when the entry is not a matrix's."""
    if fmt == OptimizerStateFormat.UNFACTORED:
        v = get_unfactored_second_moment(state)
        if v.ndim != 2:
            return None
        if model is not None:
            v = _orient_weight_second_moment(v, model, layer_name)
        return AdamNormalizer(weight_avg_sq=v.to(device), bias_avg_sq=bias)
    row, col = state["exp_avg_sq_row"], state.get("exp_avg_sq_col")
    if row.ndim != 1 or col is None:
        return None
    if model is not None:
        row, col = _orient_factored_second_moment(row, col, model, layer_name)
    return AdafactorNormalizer(row=row.to(device), col=col.to(device), bias_avg_sq=bias)


def get_normalizers(optimizer_state: dict, target_param_index_to_name: dict[int, str], target_modules,
                    adapter_suffix: str, include_bias: bool, device, base_prefix: str = "",
                    model=None) -> dict[str, Normalizer]:
    """Walks the state entries of `*.weight` parameters.  Keys are module names below `model.base_model`
    (`base_prefix`, e.g. "transformer." for GPT-2, is stripped): that is the name the collection hooks use."""
    found: dict[str, Normalizer] = {}
    for key, state in optimizer_state["state"].items():
        idx = int(key)
        named = state.get("param_name") if isinstance(state, dict) else None
        param_name = named or target_param_index_to_name.get(idx)
        if not param_name or not param_name.endswith(".weight"):
            continue
        layer_name = param_name[:-len(".weight")]
        module_name = layer_name.removeprefix("base_model.").removeprefix(base_prefix) + adapter_suffix
        if target_modules is not None and module_name not in target_modules:
            continue
        fmt = get_optimizer_state_format(state)
        if fmt is None:
            print("Unrecognized format, skipping normalizer for param_idx", idx)
            continue
        bias = _get_bias_second_moment(layer_name, target_param_index_to_name, optimizer_state, include_bias)
        norm = _normalizer_of(state, fmt, None if bias is None else bias.to(device), device, model, layer_name)
        if norm is not None:
            found[module_name] = norm
    return found


def optimizer_param_index_to_name(optimizer_pt: dict, model) -> dict[int, str]:
    """State index -> parameter name.  One param group: `model.named_parameters()` order.  Two groups: the
    HF Trainer's weight-decay / no-decay split, rebuilt with transformers' own helpers.  Second-moment
    shapes are checked against the parameters they map to."""
    groups = optimizer_pt.get("param_groups", [])
    if len(groups) <= 1:
        mapping = {idx: name for idx, (name, _) in enumerate(model.named_parameters())}
    else:
        from transformers.pytorch_utils import ALL_LAYERNORM_LAYERS
        from transformers.trainer_pt_utils import get_parameter_names

        decay = {n for n in get_parameter_names(model, ALL_LAYERNORM_LAYERS) if "bias" not in n}
        named = [n for n, p in model.named_parameters() if p.requires_grad]
        ordered = [n for n in named if n in decay] + [n for n in named if n not in decay]
        n_decay = sum(1 for n in named if n in decay)
        expected = [n_decay, len(named) - n_decay]
        sizes = [len(g.get("params", [])) for g in groups]
        if len(groups) != 2 or sizes != expected:
            raise ValueError(f"Cannot map optimizer.pt state indices to params: {len(groups)} param groups of sizes "
                             f"{sizes} do not match HF Trainer's decay/no-decay split {expected} for this model.")
        mapping = dict(zip([i for g in groups for i in g["params"]], ordered))
    shapes = {n: tuple(p.shape) for n, p in model.named_parameters()}
    for idx, entry in optimizer_pt.get("state", {}).items():
        if not isinstance(entry, dict) or "param_name" in entry or "exp_avg_sq" not in entry:
            continue
        name = mapping.get(int(idx))
        if name is not None and tuple(entry["exp_avg_sq"].shape) != shapes.get(name):
            raise ValueError(f"optimizer.pt state entry {idx} has second-moment shape "
                             f"{tuple(entry['exp_avg_sq'].shape)} but maps to {name!r} of shape {shapes.get(name)}; "
                             "the index layout is not the expected one.")
    return mapping


def load_from_optimizer(model: nn.Module, optimizer_state: str | Path, include_bias: bool = False,
                        target_modules: set[str] | None = None) -> dict[str, Normalizer]:
    """Normalizers of the model's weight matrices from the second moments saved at `optimizer_state`."""
    state = load_optimizer(optimizer_state)
    if hasattr(model, "peft_config"):
        raise NotImplementedError("PEFT checkpoints need the `peft` package, which this environment lacks")
    mapping = optimizer_param_index_to_name(state, model)
    device = next(model.parameters()).device
    normalizers = get_normalizers(state, mapping, target_modules, "", include_bias, device,
                                  _base_model_prefix(model), model)
    assert normalizers, (f"No optimizer second moments found in '{optimizer_state}'. "
                         "Ensure the checkpoint was saved from an Adam-family or Adafactor optimizer.")
    kinds = ", ".join(sorted({type(n).__name__ for n in normalizers.values()}))
    print(f"Loaded {len(normalizers)} normalizers ({kinds}) from '{optimizer_state}'")
    return normalizers
