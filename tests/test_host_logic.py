"""Host-side logic that needs no GPU: batching, padding, target discovery, shapes, head splitting,
processor files, and that the product refuses to run without a GPU instead of falling back."""
import pytest
import torch
import torch.nn as nn

from oracle import loop as oloop


def test_allocate_batches_budget_order_and_oracle():
    from bergson_amd import allocate_batches
    from bergson_amd.data import _allocate_batches_world
    from bergson_amd.synthetic import lognormal_lengths

    lengths = lognormal_lengths(300, seed=0)
    assert min(lengths) >= 16 and max(lengths) <= 2048
    batches = allocate_batches(lengths, 4096)
    assert batches == oloop.allocate_batches(lengths, 4096)
    seen = sorted(i for b in batches for i in b)
    assert seen == list(range(300))
    assert all(max(lengths[i] for i in b) * len(b) <= 4096 for b in batches)
    assert batches == allocate_batches(lengths, 4096)  # deterministic: shuffled with a fixed seed
    # short documents are left out; a document longer than the budget is an error
    assert sorted(i for b in allocate_batches([5, 1, 0, 7], 16) for i in b) == [0, 3]
    with pytest.raises(RuntimeError, match="too long"):
        allocate_batches([10, 50], 20)
    # two workers get the same number of batches and disjoint documents
    w = _allocate_batches_world(lengths, 4096, 2)
    assert len(w[0]) == len(w[1])
    assert not set(i for b in w[0] for i in b) & set(i for b in w[1] for i in b)
    assert max(len(b) for b in allocate_batches(lengths, 4096, max_batch_size=3)) <= 3


def test_allocate_batches_hand_worked_answers():
    """Known answers worked out by hand from the specification (bergson/data.py:239-377), for the product and
    for the oracle's single-worker version.

    lengths [5, 3, 9, 2, 9, 1, 4], budget 18: document 5 has one token and is left out; longest first with
    ties in index order gives 2, 4, 0, 6, 1, 3 (lengths 9 9 5 4 3 2).  A batch headed by length 9 holds
    18 // 9 = 2 documents, the next is headed by 5 and holds 18 // 5 = 3, the last takes what is left:
    [[2, 4], [0, 6, 1], [3]].  random.seed(42); random.shuffle of three items puts them in the order 1, 0, 2.
    """
    from bergson_amd import allocate_batches
    from bergson_amd.data import _allocate_batches_world, pack_by_padded_cost, spread_over_ranks

    lengths = [5, 3, 9, 2, 9, 1, 4]
    assert pack_by_padded_cost(lengths, 18) == [[2, 4], [0, 6, 1], [3]]
    assert allocate_batches(lengths, 18) == [[0, 6, 1], [2, 4], [3]]
    assert oloop.allocate_batches(lengths, 18) == [[0, 6, 1], [2, 4], [3]]
    # at most two documents per batch: [2, 4], [0, 6], [1, 3]; a shuffle of three again
    assert allocate_batches(lengths, 18, max_batch_size=2) == [[0, 6], [2, 4], [1, 3]]
    assert oloop.allocate_batches(lengths, 18, max_batch_size=2) == [[0, 6], [2, 4], [1, 3]]
    # another seed: random.seed(7) orders three items 2, 0, 1
    assert allocate_batches(lengths, 18, seed=7) == [[3], [2, 4], [0, 6, 1]]
    # two workers: three batches become four by peeling document 4 off the first batch that has two or more,
    # [[2], [0, 6, 1], [3], [4]]; dealt in turn, worker 0 has [[2], [3]] and worker 1 [[0, 6, 1], [4]]; each list is
    # shuffled with seed 42, which swaps a pair
    assert _allocate_batches_world(lengths, 18, 2) == [[[3], [2]], [[4], [0, 6, 1]]]
    assert _allocate_batches_world(lengths, 18, 2, ranks=[1]) == [[[4], [0, 6, 1]]]
    # fewer batches than workers: documents are split off the largest batch until there are four,
    # [0,1,2,3,4] -> [0,1,2,3] + [4] -> [0,1,2] + [3] -> [0,1] + [2], kept in the order of the binary heap
    # on (-size, insertion number): [[0, 1], [3], [4], [2]]
    assert spread_over_ranks([[0, 1, 2, 3, 4]], 4) == [[[0, 1]], [[3]], [[4]], [[2]]]
    with pytest.raises(RuntimeError, match="at least one batch"):
        spread_over_ranks([[0], [1]], 3)
    with pytest.raises(RuntimeError, match="Not enough documents"):
        _allocate_batches_world([1, 0, 5], 16, 2)


def test_pad_and_tensor_masks():
    from bergson_amd import pad_and_tensor

    x, y, shift, coll = pad_and_tensor([[5, 6, 7], [8]], sync_max_len=False)
    assert x.tolist() == [[5, 6, 7], [8, 0, 0]]
    assert y.tolist() == [[5, 6, 7], [8, -100, -100]]
    assert coll.tolist() == [[True, True, False], [False, False, False]]
    assert shift.tolist() == [[True, True, False], [False, False, False]]
    ox, oy, om = oloop.pad_and_tensor([[5, 6, 7], [8]])
    assert torch.equal(ox, x) and torch.equal(oy, y) and torch.equal(om, coll)
    _, y2, shift2, coll2 = pad_and_tensor([[1, 2, 3, 4]], labels=[[-100, -100, 3, 4]], sync_max_len=False)
    assert shift2.tolist() == [[False, True, True, False]] and coll2.tolist() == [[True, True, True, False]]


class _Toy(nn.Module):
    def __init__(self):
        super().__init__()
        self.attn = nn.Linear(8, 12)
        self.mlp = nn.Sequential(nn.Linear(8, 16, bias=False), nn.GELU(), nn.Linear(16, 8))
        self.norm = nn.LayerNorm(8)
        self.device = torch.device("cpu")


def _stub(model, **kw):
    from bergson_amd import HookCollectorBase

    class Stub(HookCollectorBase):
        def setup(self): ...
        def teardown(self): ...
        def backward_hook(self, module, g): ...
        def process_batch(self, indices, **k): ...

    return Stub(model=model, **kw)


def test_discover_targets_filters_and_bias():
    from bergson_amd import GradientProcessor, HookCollectorBase

    m = _Toy()
    info = HookCollectorBase.discover_targets(m)
    assert list(info) == ["attn", "mlp.0", "mlp.2"]
    assert info["mlp.0"][1] == torch.Size([16, 8]) and info["attn"][2] is False
    assert HookCollectorBase.discover_targets(m, include_bias=True)["attn"][2] is True
    assert HookCollectorBase.discover_targets(m, include_bias=True)["mlp.0"][2] is False
    assert list(HookCollectorBase.discover_targets(m, filter_modules="mlp.*")) == ["attn"]
    assert list(HookCollectorBase.discover_targets(m, target_modules={"mlp.2"})) == ["mlp.2"]
    with pytest.raises(ValueError, match="attention_cfgs"):
        from bergson_amd import AttentionConfig
        _stub(m, processor=GradientProcessor(projection_dim=4), attention_cfgs={"nope": AttentionConfig(2, 6, 2)})


def test_shapes_and_head_normalizers():
    from bergson_amd import AdafactorNormalizer, AdamNormalizer, AttentionConfig, GradientProcessor

    m = _Toy()
    c = _stub(m, processor=GradientProcessor(projection_dim=4), attention_cfgs={"attn": AttentionConfig(3, 4, 2)})
    assert list(c.shapes()) == ["attn.head_0", "attn.head_1", "attn.head_2", "mlp.0", "mlp.2"]
    assert all(s == torch.Size([4, 4]) for s in c.shapes().values())
    full = _stub(m, processor=GradientProcessor(include_bias=True), attention_cfgs={"attn": AttentionConfig(3, 4, 2)})
    assert full.shapes()["attn.head_1"] == torch.Size([4, 9]) and full.shapes()["mlp.0"] == torch.Size([16, 8])
    assert full.shapes()["mlp.2"] == torch.Size([8, 17])
    row, col = torch.arange(12.0), torch.arange(8.0)
    c.processor.normalizers = {"attn": AdafactorNormalizer(row, col), "mlp.0": AdamNormalizer(torch.ones(16, 8))}
    h1 = c.normalizer_for("attn.head_1")
    assert h1.row.tolist() == [4.0, 5.0, 6.0, 7.0] and torch.equal(h1.col, col)
    assert c.normalizer_for("mlp.2") is None and c.normalizer_for("mlp.0").weight_avg_sq.shape == (16, 8)
    assert c.split_head_name("attn.head_2") == ("attn", 2) and c.split_head_name("attn") is None
    c.processor.normalizers = {"attn": AdamNormalizer(torch.arange(96.0).reshape(12, 8), torch.arange(12.0))}
    h2 = c.normalizer_for("attn.head_2")
    assert h2.weight_avg_sq.shape == (4, 8) and h2.bias_avg_sq.tolist() == [8.0, 9.0, 10.0, 11.0]


def test_heads_are_views_of_an_untouched_module():
    """A split module reaches the backward hook once per head as a view that answers with the head's name and
    width; the module keeps its own name and width throughout, also when the hook raises."""
    from bergson_amd import AttentionConfig, GradientProcessor, HookCollectorBase
    from bergson_amd.collector import HeadView

    m = _Toy()
    seen = []

    class Probe(HookCollectorBase):
        def setup(self): ...
        def teardown(self): ...
        def process_batch(self, indices, **k): ...

        @HookCollectorBase.split_attention_heads
        def backward_hook(self, module, g):
            assert isinstance(module, nn.Linear)
            seen.append((module._name, module.out_features, module.in_features, tuple(g.shape), g.data_ptr(),
                         m.attn._name, m.attn.out_features, type(module) is HeadView or module is m.attn or module is m.mlp[0]))
            if module._name.endswith("head_1") and getattr(self, "fail", False):
                raise RuntimeError("boom")

    c = Probe(model=m, processor=GradientProcessor(projection_dim=4), attention_cfgs={"attn": AttentionConfig(3, 4, 2)})
    m.attn._name, m.mlp[0]._name = "attn", "mlp.0"
    g = torch.zeros(2, 5, 12)
    c.backward_hook(m.attn, g)
    assert [(s[0], s[1], s[2], s[3]) for s in seen] == [(f"attn.head_{h}", 4, 8, (2, 5, 4)) for h in range(3)]
    assert [s[4] for s in seen] == [g.data_ptr() + 16 * h for h in range(3)]  # views into g, nothing copied
    assert all(s[5] == "attn" and s[6] == 12 and s[7] for s in seen)
    seen.clear()
    c.backward_hook(m.mlp[0], torch.zeros(2, 5, 16))  # an ordinary module goes through as itself
    assert seen[0][:4] == ("mlp.0", 16, 8, (2, 5, 16))
    c.fail = True
    with pytest.raises(RuntimeError, match="boom"):
        c.backward_hook(m.attn, g)
    assert m.attn._name == "attn" and m.attn.out_features == 12
    with pytest.raises(AssertionError, match="output features"):
        Probe(model=m, processor=GradientProcessor(projection_dim=4),
              attention_cfgs={"attn": AttentionConfig(2, 4, 2)}).backward_hook(m.attn, g)
    # attributes set through a view land on the module (the kept input, for one)
    view = HeadView(m.attn, c.blocks_of("attn")[2])
    view._inputs = g
    assert m.attn._inputs is g
    del view._inputs
    assert not hasattr(m.attn, "_inputs")


def test_projection_cache_and_roles():
    from bergson_amd import GradientProcessor

    c = _stub(_Toy(), processor=GradientProcessor(projection_dim=4, projection_type="normal"))
    a = c.projection("attn", 4, 8, "right", torch.device("cpu"), torch.float32)
    assert c.projection("attn", 4, 8, "right", torch.device("cpu"), torch.float32) is a
    b = c.projection("attn", 4, 12, "left", torch.device("cpu"), torch.float32)
    assert a.shape == (4, 8) and b.shape == (4, 12)
    assert ("attn", "right", torch.device("cpu")) in c.processor._projection_matrices


def test_processor_roundtrip(tmp_path):
    from bergson_amd import AdafactorNormalizer, AdamNormalizer, GradientProcessor

    p = GradientProcessor(normalizers={"a": AdafactorNormalizer(torch.ones(3), torch.ones(2) * 2),
                                       "b": AdamNormalizer(torch.ones(3, 2), torch.ones(3))},
                          projection_dim=16, projection_type="normal")
    p.save(tmp_path)
    for f in ["processor_config.yaml", "normalizers.pth", "hessians.pth", "hessians_eigen.pth"]:
        assert (tmp_path / f).exists()
    q = GradientProcessor.load(tmp_path)
    assert q.projection_dim == 16 and q.projection_type == "normal" and q.projection_scale == "jl"
    assert isinstance(q.normalizers["a"], AdafactorNormalizer) and q.normalizers["a"].col.tolist() == [2.0, 2.0]
    assert isinstance(q.normalizers["b"], AdamNormalizer) and q.normalizers["b"].bias_avg_sq.shape == (3,)
    ada = q.normalizers["b"].to_adafactor()
    assert ada.row.shape == (3,) and ada.col.shape == (2,)
    torch.testing.assert_close(q.normalizers["a"].to_adam().weight_avg_sq, torch.full((3, 2), 2.0))


def test_config_defaults_follow_the_reference():
    from bergson_amd import IndexConfig, PreprocessConfig, QueryConfig, ScoreConfig

    c = IndexConfig(run_path="runs/x")
    assert (c.projection_dim, c.projection_type, c.projection_scale, c.token_batch_size, c.loss_reduction,
            c.attribute_tokens, c.include_bias) == (0, "rademacher", "jl", 2048, "sum", False, False)
    assert str(c.partial_run_path) == "runs/x.part"
    assert PreprocessConfig().aggregation == "none" and not PreprocessConfig().unit_normalize
    assert ScoreConfig().precision == "fp32" and ScoreConfig().score == "individual"
    assert QueryConfig().unit_norm is True and QueryConfig().top_k == 5


def test_no_cpu_fallback():
    """The product path refuses CPU tensors and CPU devices."""
    from bergson_amd import Attributor, GradientProcessor, Scorer, ops
    from bergson_amd.score_writer import InMemorySequenceScoreWriter

    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.scan(torch.zeros(4, 8), torch.zeros(2, 8), unit_norm=True, k=1)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.unit_normalize_rows_(torch.zeros(4, 8))
    with pytest.raises(RuntimeError, match="no CPU path"):
        Scorer({"m": torch.zeros(2, 8)}, ["m"], InMemorySequenceScoreWriter(4, 2), torch.device("cpu"), torch.float32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        Attributor("/nonexistent", device="cpu")
    m = _Toy()
    c = _stub(m, processor=GradientProcessor(projection_dim=4, projection_type="normal"))
    with c:
        m.attn(torch.randn(1, 3, 8)).sum().backward()  # hooks fire; nothing computed for the stub
        mod = m.attn
        mod._inputs = torch.randn(1, 3, 8)
        with pytest.raises(RuntimeError, match="no CPU path"):
            c._compute_gradient(mod, torch.randn(1, 3, 12))


def test_batch_vectors_are_checked_before_any_launch():
    """lengths / rows of a wrong dtype, size or layout are refused on the host (a kernel would read garbage
    lengths or scatter out of range); the check comes before the one for the device, so it runs here."""
    from bergson_amd import ops

    dev = torch.device("cpu")
    ok_l, ok_r = torch.zeros(3, dtype=torch.int32), torch.zeros(3, dtype=torch.int64)
    with pytest.raises(ValueError, match="lengths must be a contiguous int32"):
        ops._check_batch_vectors(ok_r, None, 3, dev)
    with pytest.raises(ValueError, match="offsets must be a contiguous int64"):
        ops._check_batch_vectors(None, ok_l, 3, dev)
    with pytest.raises(ValueError, match="N=4"):
        ops._check_batch_vectors(ok_l, None, 4, dev)
    with pytest.raises(ValueError, match="contiguous"):
        ops._check_batch_vectors(torch.zeros(6, dtype=torch.int32)[::2], None, 3, dev)
    with pytest.raises(ValueError, match="vector"):
        ops._check_batch_vectors(torch.zeros(3, 1, dtype=torch.int32), None, 3, dev)
    with pytest.raises(RuntimeError, match="no CPU path"):   # well-formed vectors: only then the device matters
        ops._check_batch_vectors(ok_l, ok_r, 3, dev)
    ops._check_batch_vectors(None, None, 3, dev)


def test_product_does_not_import_the_oracle():
    import pathlib
    import re

    root = pathlib.Path(__file__).resolve().parent.parent / "bergson_amd"
    for f in root.rglob("*.py"):
        assert not re.search(r"^\s*(from|import)\s+oracle\b", f.read_text(), re.M), f


class _ToyLM(nn.Module):
    """Two target layers in sequence behind an embedding, shaped [N, S, *] like a language model."""

    def __init__(self, inplace: bool = False):
        super().__init__()
        self.emb = nn.Embedding(11, 8)
        self.fc1 = nn.Linear(8, 16)
        self.fc2 = nn.Linear(16, 8, bias=False)
        self.inplace = inplace
        self.device = torch.device("cpu")

    def forward(self, x):
        h = self.fc1(self.emb(x))
        if self.inplace:
            h.mul_(2.0)
        return self.fc2(torch.tanh(h))


def _logging_stub(model):
    from bergson_amd import GradientProcessor, HookCollectorBase

    class Log(HookCollectorBase):
        def setup(self):
            self.seen = []
            self.batches = []

        def teardown(self): ...

        def backward_hook(self, module, g):
            self.seen.append((module._name, module._inputs.clone(), g.clone(), self._current_collection_mask))

        def process_batch(self, indices, **k):
            self.batches.append((list(indices), k["losses"].clone(), len(self.seen)))

    return Log(model=model, processor=GradientProcessor(projection_dim=4, projection_type="normal"))


def test_recorded_backward_matches_tensor_hooks():
    """`begin_recording` + `torch.autograd.grad` + `replay_backward` hands `backward_hook` the same modules,
    inputs and output gradients, in the same order, as the tensor hooks of a plain backward pass."""
    torch.manual_seed(0)
    m = _ToyLM()
    x = torch.randint(0, 11, (3, 5))
    mask = torch.ones(3, 5, dtype=torch.bool)
    c = _logging_stub(m)
    with c.with_batch(mask):
        m(x).square().sum().backward()
    plain, c.seen = c.seen, []
    assert [n for n, *_ in plain] == ["fc2", "fc1"]
    m.zero_grad()

    with c:
        rec = c.begin_recording(mask)
        loss = m(x).square().sum()
        c.end_recording()
        assert len(rec.entries) == 2 and not c.seen
        grads = torch.autograd.grad(loss, rec.outputs(), allow_unused=True)
        c.replay_backward(rec, grads)
    assert [n for n, *_ in c.seen] == [n for n, *_ in plain]
    for (_, a0, g0, m0), (_, a1, g1, m1) in zip(plain, c.seen):
        assert torch.equal(a0, a1) and torch.equal(g0, g1) and m1 is mask
    assert not hasattr(m.fc1, "_inputs") and not rec.entries
    assert all(p.grad is None for p in m.fc1.parameters())  # autograd.grad accumulates nothing


def test_recorded_backward_refuses_outputs_modified_in_place():
    m = _ToyLM(inplace=True)
    c = _logging_stub(m)
    with c:
        rec = c.begin_recording(None)
        m(torch.randint(0, 11, (2, 4))).sum()
        c.end_recording()
        with pytest.raises(RuntimeError, match="modified in place"):
            rec.outputs()


@pytest.mark.parametrize("embedding_root", [False, True])
def test_overlapped_steps_equal_the_plain_loop(embedding_root):
    """`OverlappedSteps` (backward pass of batch i on a helper thread beside the forward pass of batch i+1)
    gives every batch the hook calls and losses of the plain loop, batch by batch, in order."""
    from bergson_amd import IndexConfig
    from bergson_amd.collector import CollectorComputer

    class LM(_ToyLM):
        def forward(self, x):
            out = super().forward(x)
            logits = torch.cat([out, out.flip(-1)[..., :3]], -1)  # 11 "vocabulary" entries
            return type("O", (), {"logits": logits})()

    if embedding_root:  # the backward pass then stops at the embedding's output instead of the parameters
        LM.get_input_embeddings = lambda self: self.emb

    class Data:
        docs = [[1, 2, 3, 4], [5, 6, 7], [8, 9, 10, 1, 2], [3, 4], [6, 5, 4, 3, 2, 1]]

        def __len__(self):
            return len(self.docs)

        def __getitem__(self, idx):
            return {"input_ids": [self.docs[i] for i in idx]}

    torch.manual_seed(1)
    m = LM()
    m.dtype = torch.float32
    batches = [[0, 1], [2], [3, 4]]
    cfg = IndexConfig(run_path="", projection_dim=4, projection_type="normal")
    logs = []
    for overlap in (False, True):
        c = _logging_stub(m)
        CollectorComputer(model=m, data=Data(), collector=c, batches=batches, cfg=cfg,
                          overlap_backward=overlap).run_with_collector_hooks()
        logs.append(c)
    plain, over = logs
    assert [b[0] for b in over.batches] == batches and [b[2] for b in over.batches] == [b[2] for b in plain.batches]
    for (_, l0, _), (_, l1, _) in zip(plain.batches, over.batches):
        assert torch.equal(l0, l1)
    assert len(plain.seen) == len(over.seen) == 6
    m.zero_grad()
    c = _logging_stub(m)
    CollectorComputer(model=m, data=Data(), collector=c, batches=batches, cfg=cfg,
                      overlap_backward=True).run_with_collector_hooks()
    assert all(q.grad is None for q in m.parameters())  # the overlapped loop leaves nothing in .grad
    assert not m.emb._forward_hooks  # and no hook behind on the embedding
    for (n0, a0, g0, m0), (n1, a1, g1, m1) in zip(plain.seen, over.seen):
        assert n0 == n1 and torch.equal(a0, a1) and torch.equal(g0, g1) and torch.equal(m0, m1)


@pytest.mark.parametrize("unit", [False, True])
@pytest.mark.parametrize("agg", ["none", "mean", "sum"])
@pytest.mark.parametrize("norm_agg", [False, True])
def test_query_normalisation_and_aggregation(unit, agg, norm_agg):
    """`normalize_and_aggregate_grads` against the oracle's restatement and against the formulas in float64."""
    import numpy as np
    from bergson_amd import normalize_and_aggregate_grads, normalize_flat_grad
    from oracle import scan as oscan

    gen = torch.Generator().manual_seed(4)
    grads = {"b": torch.randn(5, 7, generator=gen).to(torch.float16), "a": torch.randn(5, 3, generator=gen).to(torch.float16)}
    names = ["a", "b"]
    got = normalize_and_aggregate_grads(grads, names, unit, torch.device("cpu"), agg, norm_agg)
    want = oscan.normalize_and_aggregate_queries(grads, names, unit_normalize=unit, aggregation=agg,
                                                 normalize_aggregated=norm_agg)
    assert list(got) == names
    for n in names:
        assert got[n].shape == want[n].shape and got[n].dtype == want[n].dtype
        assert torch.allclose(got[n].float(), want[n].float(), rtol=1e-6, atol=1e-7)
    m = np.concatenate([grads["a"].double().numpy(), grads["b"].double().numpy()], axis=1)
    if unit or agg != "none":
        if unit:
            m = m / np.sqrt((m ** 2).sum(1, keepdims=True))
        if agg == "mean":
            m = m.mean(0, keepdims=True)
        elif agg == "sum":
            m = m.sum(0, keepdims=True)
        if norm_agg:
            m = m / np.sqrt((m ** 2).sum())
    flat = torch.cat([got["a"], got["b"]], dim=1).double().numpy()
    assert np.allclose(flat, m, rtol=1e-5, atol=1e-7)
    v = normalize_flat_grad(grads["b"], torch.device("cpu"))
    assert v.dtype == torch.float16 and abs(float(v.float().norm()) - 1.0) < 1e-3
    with pytest.warns(UserWarning):
        assert not normalize_flat_grad(torch.zeros(4), torch.device("cpu")).any()
    with pytest.raises(ValueError):
        normalize_and_aggregate_grads(grads, names, True, torch.device("cpu"), "median")


def test_overlapped_steps_keep_foreign_hooks_on_the_embedding_firing():
    """Someone else's hook on the input embedding's weight gradient (or on the module): the overlapped loop then
    runs the backward pass down to the parameters, as `backward()` does, so the hook fires once per batch
    with the gradient the plain loop gives it."""
    from bergson_amd import IndexConfig
    from bergson_amd.collector import CollectorComputer, OverlappedSteps

    class LM(_ToyLM):
        def forward(self, x):
            out = super().forward(x)
            return type("O", (), {"logits": torch.cat([out, out.flip(-1)[..., :3]], -1)})()

        def get_input_embeddings(self):
            return self.emb

    class Data:
        docs = [[1, 2, 3, 4], [5, 6, 7], [8, 9, 10, 1, 2]]

        def __len__(self):
            return len(self.docs)

        def __getitem__(self, idx):
            return {"input_ids": [self.docs[i] for i in idx]}

    torch.manual_seed(2)
    m = LM()
    m.dtype = torch.float32
    cfg = IndexConfig(run_path="", projection_dim=4, projection_type="normal")
    assert not OverlappedSteps._has_foreign_hooks(m.emb)
    seen = {False: [], True: []}
    for overlap in (False, True):
        handle = m.emb.weight.register_hook(lambda g, overlap=overlap: seen[overlap].append(g.clone()))
        assert OverlappedSteps._has_foreign_hooks(m.emb)
        CollectorComputer(model=m, data=Data(), collector=_logging_stub(m), batches=[[0, 1], [2]], cfg=cfg,
                          overlap_backward=overlap).run_with_collector_hooks()
        handle.remove()
    assert len(seen[False]) == len(seen[True]) == 2
    for g0, g1 in zip(seen[False], seen[True]):
        assert torch.equal(g0, g1)
    handle = m.emb.register_full_backward_hook(lambda mod, gi, go: None)
    assert OverlappedSteps._has_foreign_hooks(m.emb)
    handle.remove()
