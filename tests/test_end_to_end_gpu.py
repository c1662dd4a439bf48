"""The whole collection loop on the GPU against the CPU oracle.

Two kinds of comparison:
  * fp32, Pythia-14m shape: the product loop on the GPU against the oracle's loop on the CPU.  Both
    run the same transformers model; the model's own forward/backward differs between devices at
    fp32 rounding level, so the store rows are compared at rel-L2 <= 1e-3 (the kernels alone are held
    to 1e-5 on identical inputs in test_collect_gpu.py).
  * bf16, Pythia-160m shape: the (a, g) pairs the hooks saw on the GPU are captured and pushed through
    the oracle's hook arithmetic on the CPU; the store rows must agree within rel-L2 <= 1e-2.
"""
import json

import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import hooks as ohooks
from oracle import loop as oloop
from oracle.projection import module_projections

pytestmark = pytest.mark.gpu


def _processor(p, normalizers=None):
    from bergson_amd import GradientProcessor

    return GradientProcessor(normalizers=normalizers or {}, projection_dim=p, projection_type="normal")


def test_pythia14m_fp32_store_matches_cpu_loop(device, tmp_path):
    from bergson_amd import IndexConfig, allocate_batches, collect_gradients, load_gradients
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [64, 64, 40, 33, 17, 64, 2, 50, 1, 29]
    docs = random_docs(lengths, seed=3)
    batches = allocate_batches(lengths, 128)
    assert batches == oloop.allocate_batches(lengths, 128)
    model_cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0)
    want, want_losses = oloop.collect(model_cpu, model_cpu.base_model, docs, batches, p=16)

    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0)
    cfg = IndexConfig(run_path=str(tmp_path / "run"), projection_dim=16, projection_type="normal")
    col = collect_gradients(model, ListDataset(docs), _processor(16), cfg, batches=batches)
    torch.cuda.synchronize()
    part = cfg.partial_run_path
    info = json.loads((part / "info.json").read_text())
    assert info["base_dtype"] == "float32" and info["num_grads"] == len(docs) and not info["attribute_tokens"]
    assert list(info["grad_sizes"].values()) == [256] * 24
    assert list(info["grad_sizes"])[0] == "layers.0.attention.query_key_value"
    got = torch.from_numpy(np.array(load_gradients(part)))
    assert got.shape == (len(docs), 24 * 256)
    assert got[8].abs().sum() == 0  # a one-token document is never batched; its row stays zero
    assert rel_l2(got, want) <= 1e-3
    assert torch.allclose(col.per_doc_losses.cpu(), want_losses, rtol=1e-4, atol=1e-4)
    assert int(col.total_processed) == sum(l - 1 for l in lengths if l >= 2)
    assert (part / "processor_config.yaml").exists() and (part / "total_processed.pt").exists()


def test_pythia14m_fp32_per_token_store(device, tmp_path):
    from bergson_amd import IndexConfig, TokenGradients, allocate_batches, collect_gradients
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [30, 12, 1, 25, 7]
    docs = random_docs(lengths, seed=5)
    batches = allocate_batches(lengths, 64)
    model_cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=2)
    want, _ = oloop.collect(model_cpu, model_cpu.base_model, docs, batches, p=16, attribute_tokens=True)
    want_seq, _ = oloop.collect(model_cpu, model_cpu.base_model, docs, batches, p=16)

    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=2)
    cfg = IndexConfig(run_path=str(tmp_path / "tok"), projection_dim=16, projection_type="normal",
                      attribute_tokens=True)
    collect_gradients(model, ListDataset(docs), _processor(16), cfg, batches=batches)
    tg = TokenGradients(cfg.partial_run_path)
    assert tg.num_token_grads.tolist() == [29, 11, 0, 24, 6]
    got = torch.from_numpy(np.array(tg.mmap))
    assert got.shape == want.shape
    assert rel_l2(got, want) <= 1e-3
    # the rows of a document add up to its per-sequence gradient
    assert rel_l2(torch.from_numpy(tg[0]).sum(0), want_seq[0]) <= 1e-3


@pytest.mark.parametrize("store_dtype", [None, torch.float16])
def test_pythia160m_bf16_adafactor_against_captured_hooks(device, store_dtype):
    from bergson_amd import AdafactorNormalizer, GradientCollector, IndexConfig
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, adafactor_moments, make_gpt_neox, random_docs

    lengths = [300, 180, 260]
    docs = random_docs(lengths, seed=7)
    model = make_gpt_neox("pythia-160m", torch.bfloat16, device, seed=0, layers=3)
    moments = adafactor_moments(model.base_model, seed=0)
    normalizers = {n: AdafactorNormalizer(row=r.to(device), col=c.to(device)) for n, (r, c) in moments.items()}

    captured = {}
    handles = []
    for name, mod in model.base_model.named_modules():
        if isinstance(mod, torch.nn.Linear):
            handles.append(mod.register_forward_hook(
                lambda m, inp, out, name=name: captured.setdefault(name, {}).__setitem__("a", inp[0].detach().cpu())))
            handles.append(mod.register_full_backward_hook(
                lambda m, gin, gout, name=name: captured[name].__setitem__("g", gout[0].detach().cpu())))

    cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal")
    kw = {} if store_dtype is None else {"store_dtype": store_dtype}
    col = GradientCollector(model=model.base_model, cfg=cfg, data=ListDataset(docs), processor=_processor(16, normalizers),
                            **kw)
    CollectorComputer(model=model, data=ListDataset(docs), collector=col, batches=[[0, 1, 2]], cfg=cfg
                      ).run_with_collector_hooks()
    for h in handles:
        h.remove()
    out_dtype = store_dtype or torch.bfloat16
    assert col.builder.base_dtype == {torch.bfloat16: "bfloat16", torch.float16: "float16"}[out_dtype]
    buf = col.builder.grad_buffer
    got = torch.from_numpy(buf.astype(np.float32)) if out_dtype == torch.float16 else \
        torch.from_numpy(buf.copy()).view(torch.bfloat16).float()
    assert got.shape == (3, 12 * 256)

    lo, hi = torch.finfo(out_dtype).min, torch.finfo(out_dtype).max
    blocks = []
    for name, (row, col_m) in moments.items():
        a, g = captured[name]["a"], captured[name]["g"]
        left, right = module_projections(name, 16, g.shape[-1], a.shape[-1], torch.bfloat16)
        P = ohooks.module_gradient(a, g, ohooks.Adafactor(row=row, col=col_m), left, right)
        blocks.append(P.float().clamp(lo, hi))
    want = torch.cat(blocks, 1)
    assert torch.isfinite(got).all()
    assert rel_l2(got, want) <= 1e-2
    # every module on its own, so that a small block cannot hide behind a large one
    for b in range(12):
        assert rel_l2(got[:, b * 256:(b + 1) * 256], want[:, b * 256:(b + 1) * 256]) <= 1e-2


def test_pythia14m_fp32_adam_and_mixed_normalizers(device):
    """Adam on some modules, Adafactor on others, none on the rest: every module's block against the
    oracle's hook arithmetic on the captured (a, g)."""
    from bergson_amd import AdafactorNormalizer, AdamNormalizer, GradientCollector, IndexConfig
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [40, 25, 33]
    docs = random_docs(lengths, seed=9)
    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=2)
    names = [n for n, m in model.base_model.named_modules() if isinstance(m, torch.nn.Linear)]
    gen = torch.Generator().manual_seed(1)
    onorm, norms = {}, {}
    for k, n in enumerate(names):
        mod = model.base_model.get_submodule(n)
        O, I = mod.out_features, mod.in_features
        if k % 3 == 0:
            v = torch.rand(O, I, generator=gen) * 1e-4 + 1e-8
            onorm[n], norms[n] = ohooks.Adam(v), AdamNormalizer(v.to(device))
        elif k % 3 == 1:
            r, c = torch.rand(O, generator=gen) * 1e-4 + 1e-8, torch.rand(I, generator=gen) * 1e-4 + 1e-8
            onorm[n], norms[n] = ohooks.Adafactor(r, c), AdafactorNormalizer(r.to(device), c.to(device))
    captured = {}
    handles = []
    for name in names:
        mod = model.base_model.get_submodule(name)
        handles.append(mod.register_forward_hook(
            lambda m, inp, out, name=name: captured.setdefault(name, {}).__setitem__("a", inp[0].detach().cpu())))
        handles.append(mod.register_full_backward_hook(
            lambda m, gin, gout, name=name: captured[name].__setitem__("g", gout[0].detach().cpu())))
    for attribute_tokens in (False, True):
        cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal", attribute_tokens=attribute_tokens)
        col = GradientCollector(model=model.base_model, cfg=cfg, data=ListDataset(docs), processor=_processor(16, norms))
        CollectorComputer(model=model, data=ListDataset(docs), collector=col, batches=[[0, 1, 2]], cfg=cfg
                          ).run_with_collector_hooks()
        got = torch.from_numpy(np.array(col.builder.grad_buffer))
        mask = (torch.arange(40).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        for b, name in enumerate(names):
            a, g = captured[name]["a"], captured[name]["g"]
            left, right = module_projections(name, 16, g.shape[-1], a.shape[-1], torch.float32)
            want = ohooks.module_gradient(a, g, onorm.get(name), left, right, attribute_tokens=attribute_tokens,
                                          collection_mask=mask if attribute_tokens else None)
            assert rel_l2(got[:, b * 256:(b + 1) * 256], want) <= 1e-4, (attribute_tokens, name)
    for h in handles:
        h.remove()


@pytest.mark.parametrize("attribute_tokens", [False, True])
def test_unprojected_gradients_match_cpu_loop(device, tmp_path, attribute_tokens):
    """projection_dim=0: the store holds the weight-shaped gradients themselves."""
    from bergson_amd import GradientProcessor, IndexConfig, allocate_batches, collect_gradients, load_gradients
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [20, 9, 1, 16, 5]
    docs = random_docs(lengths, seed=7)
    batches = allocate_batches(lengths, 40)
    model_cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=1)
    want, _ = oloop.collect(model_cpu, model_cpu.base_model, docs, batches, p=None, attribute_tokens=attribute_tokens)
    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=1)
    cfg = IndexConfig(run_path=str(tmp_path / "full"), projection_dim=0, attribute_tokens=attribute_tokens)
    collect_gradients(model, ListDataset(docs), GradientProcessor(projection_dim=None), cfg, batches=batches)
    torch.cuda.synchronize()
    part = cfg.partial_run_path
    info = json.loads((part / "info.json").read_text())
    assert list(info["grad_sizes"].values()) == [384 * 128, 128 * 128, 512 * 128, 128 * 512]
    if attribute_tokens:
        from bergson_amd import TokenGradients

        tg = TokenGradients(part)
        got = torch.cat([torch.from_numpy(np.array(tg[i])) for i in range(len(docs))])
    else:
        got = torch.from_numpy(np.array(load_gradients(part)))
    assert got.shape == want.shape
    assert rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("attribute_tokens", [False, True])
def test_global_projection_matches_cpu_loop(device, tmp_path, attribute_tokens):
    """projection_target="global": one [projection_dim] row per document (or token) over all modules."""
    from bergson_amd import GradientProcessor, IndexConfig, allocate_batches, collect_gradients, load_gradients
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [20, 9, 1, 16, 5]
    docs = random_docs(lengths, seed=8)
    batches = allocate_batches(lengths, 40)
    model_cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=1)
    want, _ = oloop.collect(model_cpu, model_cpu.base_model, docs, batches, p=None, global_dim=32,
                            attribute_tokens=attribute_tokens)
    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=1)
    cfg = IndexConfig(run_path=str(tmp_path / "glob"), projection_dim=32, projection_type="normal",
                      attribute_tokens=attribute_tokens)
    proc = GradientProcessor(projection_dim=32, projection_type="normal", projection_target="global")
    collect_gradients(model, ListDataset(docs), proc, cfg, batches=batches)
    torch.cuda.synchronize()
    part = cfg.partial_run_path
    info = json.loads((part / "info.json").read_text())
    assert info["grad_sizes"] == {"gradients": 32}
    if attribute_tokens:
        from bergson_amd import TokenGradients

        tg = TokenGradients(part)
        got = torch.cat([torch.from_numpy(np.array(tg[i])) for i in range(len(docs))])
    else:
        got = torch.from_numpy(np.array(load_gradients(part)))
    assert got.shape == want.shape
    assert rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("attribute_tokens", [False, True])
def test_overlapped_loop_equals_plain_loop_bitwise(device, attribute_tokens):
    """The loop with two batches in flight (backward pass of one beside the forward pass of the next, on one
    stream and on two) writes the same store and the same losses as the loop that handles one batch at a
    time, bit for bit: same kernels on the same operands, only their place in the queues differs.  Many
    batches of different shapes, so that a launch that overtook its operands, or two launches sharing the
    workspace at once, would show."""
    from bergson_amd import AdafactorNormalizer, GradientCollector, IndexConfig, allocate_batches
    from bergson_amd.collector import CollectorComputer, OverlappedSteps
    from bergson_amd.synthetic import ListDataset, adafactor_moments, lognormal_lengths, make_gpt_neox, random_docs

    lengths = lognormal_lengths(40, mu=4.0, sigma=0.8, lo=2, hi=256, seed=11)
    docs = random_docs(lengths, seed=11)
    batches = allocate_batches(lengths, 256)
    assert len(batches) >= 8
    model = make_gpt_neox("pythia-160m", torch.bfloat16, device, seed=0, layers=2)
    moments = adafactor_moments(model.base_model, seed=0)
    normalizers = {n: AdafactorNormalizer(row=r.to(device), col=c.to(device)) for n, (r, c) in moments.items()}
    cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal", attribute_tokens=attribute_tokens)

    def run(overlap, streams, monkeypatch_streams):
        col = GradientCollector(model=model.base_model, cfg=cfg, data=ListDataset(docs),
                                processor=_processor(16, normalizers), store_dtype=torch.float16)
        monkeypatch_streams(streams)
        CollectorComputer(model=model, data=ListDataset(docs), collector=col, batches=batches, cfg=cfg,
                          overlap_backward=overlap).run_with_collector_hooks()
        torch.cuda.synchronize()
        return np.array(col.builder.grad_buffer).copy(), col.per_doc_losses.cpu().clone()

    init = OverlappedSteps.__init__

    def set_streams(n):
        def patched(self, *a, **k):
            k["streams"] = n
            init(self, *a, **k)
        OverlappedSteps.__init__ = patched

    try:
        plain, plain_losses = run(False, 1, set_streams)
        for streams in (1, 2):
            got, losses = run(True, streams, set_streams)
            assert np.array_equal(got.view(np.uint16), plain.view(np.uint16)), streams
            assert torch.equal(losses, plain_losses), streams
    finally:
        OverlappedSteps.__init__ = init
    assert np.abs(plain.astype(np.float32)).sum() > 0
    assert all(p.grad is None for p in model.parameters())


@pytest.mark.parametrize("overlap", [True, False])
@pytest.mark.parametrize("reduction,smoothing,use_labels,use_advantage", [
    ("mean", 0.0, False, False),
    ("sum", 0.1, False, False),
    ("mean", 0.1, True, False),
    ("sum", 0.0, True, True),
    ("mean", 0.1, False, True),
])
def test_loss_options_match_cpu_loop(device, reduction, smoothing, use_labels, use_advantage, overlap):
    """`loss_reduction="mean"`, `label_smoothing`, prompt-masked labels and the advantage column
    (bergson/collector/collector.py:948-983): the product loop, plain and overlapped, against the oracle's
    loop, whose loss arithmetic is pinned against autograd on the CPU."""
    from bergson_amd import IndexConfig, allocate_batches, collect_gradients
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [31, 18, 2, 25, 9, 40]
    docs = random_docs(lengths, seed=13)
    labels = [[-100] * (len(d) // 3) + d[len(d) // 3:] for d in docs] if use_labels else None
    advantage = [0.5, -1.5, 2.0, 1.0, 0.25, -0.75] if use_advantage else None
    batches = allocate_batches(lengths, 80)
    model_cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=2)
    want, want_losses = oloop.collect(model_cpu, model_cpu.base_model, docs, batches, p=16, loss_reduction=reduction,
                                      label_smoothing=smoothing, labels=labels, advantages=advantage)
    model = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=2)
    cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal", loss_reduction=reduction,
                      label_smoothing=smoothing)
    data = ListDataset(docs, labels=labels, advantage=advantage)
    col = collect_gradients(model, data, _processor(16), cfg, batches=batches, overlap_backward=overlap)
    torch.cuda.synchronize()
    got = torch.from_numpy(np.array(col.builder.grad_buffer))
    assert rel_l2(got, want) <= 1e-3
    assert torch.allclose(col.per_doc_losses.cpu(), want_losses, rtol=1e-4, atol=1e-4)
    for i in range(len(docs)):  # row by row: a short document must not hide behind a long one
        assert rel_l2(got[i], want[i]) <= 2e-3, i
