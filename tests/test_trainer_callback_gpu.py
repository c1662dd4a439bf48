"""GradientCollectorCallback inside a real `transformers.Trainer` run on the GPU, against a CPU replay.

The replay trains the same randomly initialised model on the CPU with torch.optim.AdamW in the order the
Trainer used (recorded by `track_order`), captures every target layer's input and output gradient with plain
module hooks, and forms each example's row with the oracle's `module_gradient` under the normalizer the
callback must have derived from the optimizer state of the previous step (Adam second moments / lr^2).
Tolerance: rows are stored in fp16 -> relative L2 <= 5e-3 per epoch store.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import rel_l2
from oracle import hooks as ohooks
from oracle import loop as oloop
from oracle.projection import module_projections

pytestmark = pytest.mark.gpu

LOSS_SCALE = 50.0


def _loss(outputs, labels, num_items_in_batch=None):
    logits = outputs["logits"] if isinstance(outputs, dict) else outputs.logits
    V = logits.shape[-1]
    return F.cross_entropy(logits[:, :-1].reshape(-1, V).float(), labels[:, 1:].reshape(-1), reduction="sum") / LOSS_SCALE


def _replay(cpu_model, docs, steps, lr, scale_by_lr, p=16):
    """rows[epoch][idx] = oracle row of example idx as trained on in that epoch."""
    base = cpu_model.base_model
    linears = oloop.target_linears(base)
    stash = {}

    def fwd(name):
        return lambda mod, inp, out: stash.__setitem__((name, "a"), inp[0].detach())

    def bwd(name):
        return lambda mod, gin, gout: stash.__setitem__((name, "g"), gout[0].detach())

    handles = []
    for name, lin in linears.items():
        handles.append(lin.register_forward_hook(fwd(name)))
        handles.append(lin.register_full_backward_hook(bwd(name)))
    opt = torch.optim.AdamW(cpu_model.parameters(), lr=lr, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    rows = {}
    lo, hi = torch.finfo(torch.float16).min, torch.finfo(torch.float16).max
    for epoch, idxs in steps:
        x = torch.tensor([docs[i] for i in idxs])
        # normalizers from the optimizer state as it stands before this step
        norms = {}
        for name, lin in linears.items():
            st = opt.state.get(lin.weight, {})
            if "exp_avg_sq" in st:
                norms[name] = ohooks.Adam(st["exp_avg_sq"].clone() / (lr ** 2 if scale_by_lr else 1.0))
        out = cpu_model(input_ids=x)
        _loss(out, x).backward()
        parts = []
        for name, lin in linears.items():
            # the callback builds its GradientProcessor with the defaults: rademacher projections (huggingface.py:119-126)
            left, right = module_projections(name, p, lin.out_features, lin.in_features, torch.float32,
                                             projection_type="rademacher")
            parts.append(ohooks.module_gradient(stash[(name, "a")], stash[(name, "g")], norms.get(name), left, right,
                                                lo=lo, hi=hi))
        batch_rows = torch.cat(parts, 1)
        for j, i in enumerate(idxs):
            rows.setdefault(epoch, {})[i] = batch_rows[j]
        opt.step()
        opt.zero_grad()
    for h in handles:
        h.remove()
    return rows


@pytest.mark.parametrize("use_optimizer_state,scale_by_lr", [(False, False), (True, True), (True, False)])
def test_callback_rows_match_cpu_replay(device, tmp_path, use_optimizer_state, scale_by_lr):
    from datasets import Dataset
    from transformers import Trainer, TrainingArguments

    from bergson_amd import load_gradients
    from bergson_amd.huggingface import GradientCollectorCallback, prepare_for_gradient_collection
    from bergson_amd.synthetic import make_gpt_neox, random_docs

    n, L, lr = 6, 12, 1e-3
    docs = random_docs([L] * n, seed=21)
    ds = Dataset.from_dict({"input_ids": docs, "labels": docs})
    model = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=2)
    cpu_model = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=2)
    args = TrainingArguments(output_dir=str(tmp_path / "out"), per_device_train_batch_size=2, num_train_epochs=2,
                             learning_rate=lr, lr_scheduler_type="constant", weight_decay=0.0, max_grad_norm=0.0,
                             report_to="none", save_strategy="no", logging_strategy="no", disable_tqdm=True, seed=0,
                             dataloader_pin_memory=False, optim="adamw_torch")
    cb = GradientCollectorCallback(tmp_path / "grads", projection_dim=16, dtype=np.dtype(np.float16),
                                   use_optimizer_state=use_optimizer_state, scale_by_lr=scale_by_lr, track_order=True)
    trainer = Trainer(model=model, args=args, train_dataset=ds, callbacks=[cb], compute_loss_func=_loss)
    prepare_for_gradient_collection(trainer)
    trainer.train()

    # the recorded order: (epoch, indices) per global step
    order = cb.order
    assert order is not None and len(order) == 2 * n
    steps = []
    for rec in order:
        if steps and steps[-1][2] == rec["global_step"]:
            steps[-1][1].append(rec["_idx"])
        else:
            steps.append([rec["epoch"], [rec["_idx"]], rec["global_step"]])
    assert len(steps) == 6 and all(len(s[1]) == 2 for s in steps)
    # epoch of a record is the epoch counter at the end of its step: the last step of epoch e reports e + 1
    per_epoch = [steps[:3], steps[3:]]
    replay_steps = [(e, s[1]) for e, chunk in enumerate(per_epoch) for s in chunk]
    if not use_optimizer_state:
        want = _replay(cpu_model, docs, replay_steps, lr, False)
    else:
        want = _replay(cpu_model, docs, replay_steps, lr, scale_by_lr)

    for e in (0, 1):
        path = tmp_path / "grads" / "train" / f"epoch_{e}"
        got = torch.from_numpy(np.array(load_gradients(path))).float()
        assert got.shape == (n, 8 * 256)
        ref = torch.stack([want[e][i] for i in range(n)]).float()
        assert sorted(want[e]) == list(range(n))
        assert torch.isfinite(got).all() and got.abs().max() > 0
        if rel_l2(got, ref) > 5e-3:
            cos = torch.nn.functional.normalize(got, dim=1) @ torch.nn.functional.normalize(ref, dim=1).T
            print("cosine got x ref\n", cos, "\nnorms", got.norm(dim=1), ref.norm(dim=1), "steps", replay_steps, flush=True)
            for m in range(8):
                print("module", m, rel_l2(got[:, m * 256:(m + 1) * 256], ref[:, m * 256:(m + 1) * 256]))
        assert rel_l2(got, ref) <= 5e-3, (e, rel_l2(got, ref))
        assert (path / "processor_config.yaml").exists() and (path / "info.json").exists()
    assert (tmp_path / "grads" / "order.hf").exists()


def test_callback_requires_prepared_trainer(tmp_path):
    from bergson_amd.huggingface import GradientCollectorCallback

    class Args:
        pass

    cb = GradientCollectorCallback(tmp_path / "g")
    with pytest.raises(RuntimeError, match="not enabled"):
        cb.on_train_begin(Args(), None, None, model=torch.nn.Linear(2, 2))
