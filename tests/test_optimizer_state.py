"""`load_from_optimizer`: normalizers from real optimizer states (host logic, CPU).

The states come from actual `torch.optim.AdamW` / `transformers.optimization.Adafactor` steps on small
models built locally, so the expected second moments are the optimizer's own tensors; what is checked is
the mapping (index -> parameter -> module name below base_model), the [out, in] orientation for layers that
store their weight transposed, and the filters.  Mirrors the cases of the reference's
tests/test_adam_state_loading.py that need neither the hub nor peft.
"""
import pytest
import torch
import torch.nn as nn
from transformers.pytorch_utils import Conv1D

from bergson_amd.gradients import AdafactorNormalizer, AdamNormalizer
from bergson_amd.optimizer_state import (OptimizerStateFormat, get_optimizer_state_format,
                                         get_unfactored_second_moment, load_from_optimizer, load_optimizer,
                                         optimizer_param_index_to_name, orient_second_moment)


class Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.ln = nn.LayerNorm(6)
        self.fc = nn.Linear(6, 10, bias=True)      # weight [out=10, in=6]
        self.c_proj = Conv1D(6, 10)                # nx=10 -> nf=6, weight stored [in=10, out=6]
        self.sq = Conv1D(6, 6)                     # square and transposed: shapes cannot tell


class Body(nn.Module):
    def __init__(self):
        super().__init__()
        self.emb = nn.Embedding(12, 6)
        self.h = nn.ModuleList([Block(), Block()])


class Model(nn.Module):
    """`transformer` plays the part of a HF model's base_model (GPT-2 layout)."""

    def __init__(self):
        super().__init__()
        torch.manual_seed(0)
        self.transformer = Body()
        self.head = nn.Linear(6, 12, bias=False)

    @property
    def base_model(self):
        return self.transformer

    def forward(self, ids):
        x = self.transformer.emb(ids)
        for b in self.transformer.h:
            x = b.sq(b.c_proj(b.fc(b.ln(x))))
        return self.head(x)


def _train(model, opt, steps=3):
    torch.manual_seed(1)
    for _ in range(steps):
        loss = model(torch.randint(0, 12, (4, 5))).square().mean()
        loss.backward()
        opt.step()
        opt.zero_grad()


def test_adamw_single_group(tmp_path):
    model = Model()
    opt = torch.optim.AdamW(model.parameters(), lr=1e-2)
    _train(model, opt)
    torch.save(opt.state_dict(), tmp_path / "optimizer.pt")
    norms = load_from_optimizer(model, str(tmp_path), include_bias=True)   # directory form
    names = [n for n, _ in model.named_parameters()]
    state = opt.state_dict()["state"]
    by_name = {names[i]: s["exp_avg_sq"] for i, s in state.items()}
    # keys are relative to base_model ("transformer." stripped); head is outside it and keeps its name; every
    # 2-D `.weight` gets an entry (the embedding's is simply never looked up), LayerNorm's 1-D weight none
    assert set(norms) == {f"h.{i}.{m}" for i in (0, 1) for m in ("fc", "c_proj", "sq")} | {"head", "emb"}
    assert all(isinstance(n, AdamNormalizer) for n in norms.values())
    for i in (0, 1):
        fc = norms[f"h.{i}.fc"]
        assert torch.equal(fc.weight_avg_sq, by_name[f"transformer.h.{i}.fc.weight"]) and fc.weight_avg_sq.shape == (10, 6)
        assert torch.equal(fc.bias_avg_sq, by_name[f"transformer.h.{i}.fc.bias"])
        cp = norms[f"h.{i}.c_proj"]                                         # stored [in, out] -> transposed
        assert cp.weight_avg_sq.shape == (6, 10)
        assert torch.equal(cp.weight_avg_sq, by_name[f"transformer.h.{i}.c_proj.weight"].T)
        assert torch.equal(cp.bias_avg_sq, by_name[f"transformer.h.{i}.c_proj.bias"])
        sq = norms[f"h.{i}.sq"]                                              # square: the layer type decides
        assert torch.equal(sq.weight_avg_sq, by_name[f"transformer.h.{i}.sq.weight"].T)
        assert not torch.equal(sq.weight_avg_sq, by_name[f"transformer.h.{i}.sq.weight"])
    assert norms["head"].bias_avg_sq is None


def test_file_form_target_modules_and_no_bias(tmp_path):
    model = Model()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2)
    _train(model, opt)
    path = tmp_path / "state.pth"
    torch.save(opt.state_dict(), path)
    norms = load_from_optimizer(model, path, target_modules={"h.1.fc", "h.0.sq"})
    assert set(norms) == {"h.1.fc", "h.0.sq"} and norms["h.1.fc"].bias_avg_sq is None


def test_trainer_style_decay_groups(tmp_path):
    """Two param groups in the HF Trainer's order (decayed weights first, then biases and LayerNorm): state
    indices follow the groups, not named_parameters()."""
    from transformers.pytorch_utils import ALL_LAYERNORM_LAYERS
    from transformers.trainer_pt_utils import get_parameter_names

    model = Model()
    decay = [n for n in get_parameter_names(model, ALL_LAYERNORM_LAYERS) if "bias" not in n]
    params = dict(model.named_parameters())
    opt = torch.optim.AdamW([{"params": [params[n] for n in params if n in decay], "weight_decay": 0.1},
                             {"params": [params[n] for n in params if n not in decay], "weight_decay": 0.0}], lr=1e-2)
    _train(model, opt)
    sd = opt.state_dict()
    torch.save(sd, tmp_path / "optimizer.pt")
    mapping = optimizer_param_index_to_name(sd, model)
    ordered = [n for n in params if n in decay] + [n for n in params if n not in decay]
    assert [mapping[i] for i in range(len(ordered))] == ordered
    norms = load_from_optimizer(model, tmp_path / "optimizer.pt", include_bias=True)
    by_name = {ordered[i]: s["exp_avg_sq"] for i, s in sd["state"].items()}
    assert torch.equal(norms["h.1.fc"].weight_avg_sq, by_name["transformer.h.1.fc.weight"])
    assert torch.equal(norms["h.1.fc"].bias_avg_sq, by_name["transformer.h.1.fc.bias"])
    assert torch.equal(norms["h.0.c_proj"].weight_avg_sq, by_name["transformer.h.0.c_proj.weight"].T)
    # a split that is not the Trainer's is refused rather than guessed
    sd["param_groups"][0]["params"] = sd["param_groups"][0]["params"][:-1]
    with pytest.raises(ValueError, match="decay/no-decay"):
        optimizer_param_index_to_name(sd, model)


def test_adafactor_factored_state(tmp_path):
    from transformers.optimization import Adafactor

    model = Model()
    opt = Adafactor(model.parameters(), lr=1e-2, relative_step=False, scale_parameter=False)
    _train(model, opt)
    torch.save(opt.state_dict(), tmp_path / "optimizer.pt")
    norms = load_from_optimizer(model, tmp_path, include_bias=True)
    names = [n for n, _ in model.named_parameters()]
    state = opt.state_dict()["state"]
    fc = norms["h.0.fc"]
    s = state[names.index("transformer.h.0.fc.weight")]
    assert isinstance(fc, AdafactorNormalizer)
    assert torch.equal(fc.row, s["exp_avg_sq_row"]) and fc.row.shape == (10,)
    assert torch.equal(fc.col, s["exp_avg_sq_col"]) and fc.col.shape == (6,)
    assert torch.equal(fc.bias_avg_sq, state[names.index("transformer.h.0.fc.bias")]["exp_avg_sq"])  # 1-D: unfactored
    cp = norms["h.0.c_proj"]                         # stored [in=10, out=6]: the factors swap
    s = state[names.index("transformer.h.0.c_proj.weight")]
    assert torch.equal(cp.row, s["exp_avg_sq_col"]) and cp.row.shape == (6,)
    assert torch.equal(cp.col, s["exp_avg_sq_row"]) and cp.col.shape == (10,)


def test_recorded_param_names_take_precedence(tmp_path):
    model = Model()
    v = torch.full((10, 6), 7.0)
    sd = {"state": {0: {"exp_avg_sq": v, "param_name": "transformer.h.1.fc.weight"},
                    1: {"exp_avg_sq": torch.full((10,), 3.0), "param_name": "transformer.h.1.fc.bias"}},
          "param_groups": [{"params": [0, 1]}]}
    torch.save(sd, tmp_path / "optimizer.pt")
    norms = load_from_optimizer(model, tmp_path, include_bias=True)
    assert set(norms) == {"h.1.fc"} and torch.equal(norms["h.1.fc"].weight_avg_sq, v)
    assert torch.equal(norms["h.1.fc"].bias_avg_sq, torch.full((10,), 3.0))


def test_formats_and_orientation_helpers():
    assert get_optimizer_state_format({"exp_avg_sq": 1}) is OptimizerStateFormat.UNFACTORED
    assert get_optimizer_state_format({"exp_avg_sq_row": 1}) is OptimizerStateFormat.FACTORED
    bnb = {"__bnb_optimizer_quant_state__": {"state2": torch.ones(2)}}
    assert get_optimizer_state_format(bnb) is OptimizerStateFormat.UNFACTORED
    assert torch.equal(get_unfactored_second_moment(bnb), torch.ones(2))
    assert get_optimizer_state_format({"step": 3}) is None and get_optimizer_state_format(5) is None
    t = torch.arange(6.0).reshape(2, 3)
    assert torch.equal(orient_second_moment(t, 2, 3), t)
    assert torch.equal(orient_second_moment(t, 3, 2), t.T)
    assert orient_second_moment(t, 4, 4) is None
    assert torch.equal(orient_second_moment(t, 3, 2, layer=Conv1D(3, 2)), t.T)   # nx=2, nf=3: stored [2, 3]
    assert orient_second_moment(t, 2, 3, layer=Conv1D(3, 2)) is None


def test_errors(tmp_path):
    model = Model()
    with pytest.raises(FileNotFoundError):
        load_optimizer(tmp_path / "nope.pt")
    with pytest.raises(NotImplementedError):
        load_optimizer("hf://org/repo/checkpoint-5")
    torch.save({"state": {0: {"step": 1}}, "param_groups": [{"params": [0]}]}, tmp_path / "optimizer.pt")
    with pytest.raises(AssertionError, match="No optimizer second moments"):
        load_from_optimizer(model, tmp_path)
    # a state whose shapes do not fit the model's parameter order is refused
    torch.save({"state": {0: {"exp_avg_sq": torch.ones(3, 3)}}, "param_groups": [{"params": [0]}]},
               tmp_path / "optimizer.pt")
    with pytest.raises(ValueError, match="index layout"):
        load_from_optimizer(model, tmp_path)
