"""`load_from_optimizer` feeding the collector on the GPU: second moments from real AdamW steps, read back from
`optimizer.pt`, used as Adam normalizers and (through `.to_adafactor()`) as Adafactor normalizers; every
module's block against the oracle's hook arithmetic under the optimizer's own `exp_avg_sq` tensors."""
import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import hooks as ohooks
from oracle.projection import module_projections

pytestmark = pytest.mark.gpu


def test_normalizers_from_adamw_state_drive_the_collector(device, tmp_path):
    from bergson_amd import AdamNormalizer, GradientCollector, GradientProcessor, IndexConfig
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.optimizer_state import load_from_optimizer
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=2, vocab=1024)
    model.requires_grad_(True)
    model.train()
    opt = torch.optim.AdamW(model.parameters(), lr=1e-3)
    gen = torch.Generator().manual_seed(3)
    for _ in range(3):
        ids = torch.randint(0, 1024, (4, 24), generator=gen).to(device)
        model(ids, labels=ids).loss.backward()
        opt.step()
        opt.zero_grad()
    torch.save(opt.state_dict(), tmp_path / "optimizer.pt")
    # the optimizer's own tensors, looked up by parameter name without the loader
    param_names = [n for n, _ in model.named_parameters()]
    own = {param_names[i]: s["exp_avg_sq"].detach().cpu() for i, s in opt.state_dict()["state"].items()}
    model.requires_grad_(False)
    model.get_input_embeddings().requires_grad_(True)
    model.eval()

    normalizers = load_from_optimizer(model, tmp_path)
    names = [n for n, m in model.base_model.named_modules() if isinstance(m, torch.nn.Linear)]
    assert set(names) <= set(normalizers) and all(isinstance(normalizers[n], AdamNormalizer) for n in names)
    for n in names:
        assert torch.equal(normalizers[n].weight_avg_sq.cpu(), own[f"gpt_neox.{n}.weight"])

    lengths = [33, 20, 41]
    docs = random_docs(lengths, vocab=1024, seed=4)
    captured, handles = {}, []
    for name in names:
        mod = model.base_model.get_submodule(name)
        handles.append(mod.register_forward_hook(
            lambda m, inp, out, name=name: captured.setdefault(name, {}).__setitem__("a", inp[0].detach().cpu())))
        handles.append(mod.register_full_backward_hook(
            lambda m, gin, gout, name=name: captured[name].__setitem__("g", gout[0].detach().cpu())))
    cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal")
    for kind in ("adam", "adafactor"):
        norms = {n: (normalizers[n] if kind == "adam" else normalizers[n].to_adafactor()) for n in names}
        col = GradientCollector(model=model.base_model, cfg=cfg, data=ListDataset(docs),
                                processor=GradientProcessor(normalizers=norms, projection_dim=16,
                                                            projection_type="normal"))
        CollectorComputer(model=model, data=ListDataset(docs), collector=col, batches=[[0, 1, 2]], cfg=cfg
                          ).run_with_collector_hooks()
        torch.cuda.synchronize()
        got = torch.from_numpy(np.array(col.builder.grad_buffer))
        assert got.shape == (3, len(names) * 256) and torch.isfinite(got).all()
        for b, name in enumerate(names):
            a, g = captured[name]["a"], captured[name]["g"]
            v = own[f"gpt_neox.{name}.weight"]
            onorm = ohooks.Adam(v) if kind == "adam" else ohooks.Adafactor(row=v.mean(dim=1), col=v.mean(dim=0))
            left, right = module_projections(name, 16, g.shape[-1], a.shape[-1], torch.float32)
            want = ohooks.module_gradient(a, g, onorm, left, right)
            assert rel_l2(got[:, b * 256:(b + 1) * 256], want) <= 1e-4, (kind, name)
    for h in handles:
        h.remove()
