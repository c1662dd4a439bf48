"""The reference-shaped classes (Scorer, Attributor, InMemoryCollector, head splitting, Builder options)
on the GPU against the CPU oracle."""
import json

import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import hooks as ohooks
from oracle import loop as oloop
from oracle import scan as oscan
from oracle import store as ostore
from oracle.projection import module_projections, projection_matrix

pytestmark = pytest.mark.gpu


def _proc(p, normalizers=None):
    from bergson_amd import GradientProcessor

    return GradientProcessor(normalizers=normalizers or {}, projection_dim=p, projection_type="normal")


def _setup(device, lengths, layers=2, seed=11):
    from bergson_amd import allocate_batches
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    docs = random_docs(lengths, seed=seed)
    batches = allocate_batches(lengths, 96)
    cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=layers)
    gpu = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=layers)
    return docs, ListDataset(docs), batches, cpu, gpu


def test_in_memory_collector_and_unit_normalize(device):
    from bergson_amd import IndexConfig, InMemoryCollector, PreprocessConfig
    from bergson_amd.collector import CollectorComputer

    lengths = [40, 22, 31, 17, 48]
    docs, data, batches, cpu, gpu = _setup(device, lengths)
    want, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16, unit_normalize=True)
    cfg = IndexConfig(projection_dim=16, projection_type="normal")
    col = InMemoryCollector(model=gpu.base_model, cfg=cfg, data=data, processor=_proc(16),
                            preprocess_cfg=PreprocessConfig(unit_normalize=True))
    CollectorComputer(model=gpu, data=data, collector=col, batches=batches, cfg=cfg).run_with_collector_hooks()
    assert list(col.gradients) == list(oloop.target_linears(cpu.base_model))
    got = torch.cat([col.gradients[n] for n in col.gradients], 1)
    assert got.shape == want.shape
    torch.testing.assert_close(got.norm(dim=1), torch.ones(5), rtol=1e-4, atol=1e-4)
    assert rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("aggregation", ["mean", "sum"])
def test_aggregated_store(device, tmp_path, aggregation):
    from bergson_amd import IndexConfig, PreprocessConfig, collect_gradients, load_gradients

    lengths = [40, 22, 31, 17]
    docs, data, batches, cpu, gpu = _setup(device, lengths)
    rows, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
    want = rows.sum(0, keepdim=True) if aggregation == "sum" else rows.mean(0, keepdim=True)
    cfg = IndexConfig(run_path=str(tmp_path / "agg"), projection_dim=16, projection_type="normal")
    collect_gradients(gpu, data, _proc(16), cfg, batches=batches,
                      preprocess_cfg=PreprocessConfig(aggregation=aggregation))
    info = json.loads((cfg.partial_run_path / "info.json").read_text())
    assert info["num_grads"] == 1 and info["base_dtype"] == "float32"
    got = torch.from_numpy(np.array(load_gradients(cfg.partial_run_path)))
    assert rel_l2(got, want) <= 1e-3


def test_attention_head_split(device):
    """Per-head rows: each head projects its slice of g with its own left matrix and shares the
    parent's input-side matrix; with Adafactor its row factor uses the mean over its own rows."""
    from bergson_amd import AdafactorNormalizer, AttentionConfig, GradientCollector, IndexConfig
    from bergson_amd.collector import CollectorComputer

    lengths = [30, 30]
    docs, data, batches, cpu, gpu = _setup(device, lengths, layers=1)
    name = "layers.0.attention.dense"
    heads, hs = 4, 32
    gen = torch.Generator().manual_seed(0)
    row, colm = torch.rand(128, generator=gen) + 0.1, torch.rand(128, generator=gen) + 0.1
    cap = {}
    mod = gpu.base_model.get_submodule(name)
    h1 = mod.register_forward_hook(lambda m, i, o: cap.__setitem__("a", i[0].detach().cpu()))
    h2 = mod.register_full_backward_hook(lambda m, gi, go: cap.__setitem__("g", go[0].detach().cpu()))
    cfg = IndexConfig(projection_dim=16, projection_type="normal")
    col = GradientCollector(model=gpu.base_model, cfg=cfg, data=data, target_modules={name},
                            processor=_proc(16, {name: AdafactorNormalizer(row.to(device), colm.to(device))}),
                            attention_cfgs={name: AttentionConfig(heads, hs, 2)})
    assert list(col.shapes()) == [f"{name}.head_{h}" for h in range(heads)]
    CollectorComputer(model=gpu, data=data, collector=col, batches=[[0, 1]], cfg=cfg).run_with_collector_hooks()
    h1.remove(), h2.remove()
    got = torch.from_numpy(np.array(col.builder.grad_buffer))
    assert got.shape == (2, heads * 256)
    a, g = cap["a"], cap["g"]
    right = projection_matrix(f"{name}/right", 16, 128, torch.float32)
    stash = ohooks.forward_hook(a, ohooks.Adafactor(row, colm), right)
    for h in range(heads):
        left = projection_matrix(f"{name}.head_{h}/left", 16, hs, torch.float32)
        norm_h = ohooks.Adafactor(row[h * hs:(h + 1) * hs], colm)
        want = ohooks.backward_hook(stash, g[:, :, h * hs:(h + 1) * hs], norm_h, left, right)
        assert rel_l2(got[:, h * 256:(h + 1) * 256], want) <= 1e-4


@pytest.mark.parametrize("attribute_tokens", [False, True])
def test_attention_head_split_adam(device, attribute_tokens):
    """With an Adam normalizer a head is projected on BOTH sides under its own name (the reference's Adam
    branch calls double_sided_projection with the head's name, bergson/collector/collector.py:545-550,
    :626-644), and its second moments are the head's rows of the module's."""
    from bergson_amd import AdamNormalizer, AttentionConfig, GradientCollector, IndexConfig
    from bergson_amd.collector import CollectorComputer

    lengths = [30, 21]
    docs, data, batches, cpu, gpu = _setup(device, lengths, layers=1)
    name = "layers.0.attention.dense"
    heads, hs = 4, 32
    gen = torch.Generator().manual_seed(1)
    v = torch.rand(128, 128, generator=gen) * 1e-4 + 1e-8
    cap = {}
    mod = gpu.base_model.get_submodule(name)
    h1 = mod.register_forward_hook(lambda m, i, o: cap.__setitem__("a", i[0].detach().cpu()))
    h2 = mod.register_full_backward_hook(lambda m, gi, go: cap.__setitem__("g", go[0].detach().cpu()))
    cfg = IndexConfig(projection_dim=16, projection_type="normal", attribute_tokens=attribute_tokens)
    col = GradientCollector(model=gpu.base_model, cfg=cfg, data=data, target_modules={name},
                            processor=_proc(16, {name: AdamNormalizer(v.to(device))}),
                            attention_cfgs={name: AttentionConfig(heads, hs, 2)})
    CollectorComputer(model=gpu, data=data, collector=col, batches=[[0, 1]], cfg=cfg).run_with_collector_hooks()
    h1.remove(), h2.remove()
    got = torch.from_numpy(np.array(col.builder.grad_buffer))
    a, g = cap["a"], cap["g"]
    mask = (torch.arange(30).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    assert got.shape == (int(mask.sum()) if attribute_tokens else 2, heads * 256)
    for h in range(heads):
        left = projection_matrix(f"{name}.head_{h}/left", 16, hs, torch.float32)
        right = projection_matrix(f"{name}.head_{h}/right", 16, 128, torch.float32)
        want = ohooks.module_gradient(a, g[:, :, h * hs:(h + 1) * hs], ohooks.Adam(v[h * hs:(h + 1) * hs]), left,
                                      right, attribute_tokens=attribute_tokens,
                                      collection_mask=mask if attribute_tokens else None)
        assert rel_l2(got[:, h * 256:(h + 1) * 256], want) <= 1e-4, h
    # the parent's matrix is another one: sharing it would not pass
    assert not torch.equal(projection_matrix(f"{name}/right", 16, 128, torch.float32),
                           projection_matrix(f"{name}.head_0/right", 16, 128, torch.float32))


def test_scorer_on_the_fly_matches_oracle(device, tmp_path):
    from bergson_amd import IndexConfig, Scorer, collect_gradients
    from bergson_amd.data import load_scores
    from bergson_amd.score_writer import MemmapSequenceScoreWriter

    lengths = [40, 22, 31, 17, 48, 12]
    docs, data, batches, cpu, gpu = _setup(device, lengths)
    rows, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
    mods = list(oloop.target_linears(cpu.base_model))
    sizes = {m: 256 for m in mods}
    cols = ostore.column_offsets(sizes)
    index = {m: rows[:, lo:hi] for m, (lo, hi) in cols.items()}
    gen = torch.Generator().manual_seed(5)
    queries = {m: torch.randn(3, 256, generator=gen) for m in mods}
    qn = oscan.normalize_and_aggregate_queries(queries, mods, unit_normalize=True)
    want = oscan.scorer_score(index, qn, mods, unit_normalize=True)
    want_near = oscan.scorer_score(index, qn, mods, unit_normalize=True, score_mode="nearest")

    for mode, ref, width in (("individual", want, 3), ("nearest", want_near, 1)):
        path = tmp_path / mode
        writer = MemmapSequenceScoreWriter(path, len(docs), width)
        scorer = Scorer(qn, mods, writer, device, torch.float32, unit_normalize=True, score_mode=mode)
        cfg = IndexConfig(projection_dim=16, projection_type="normal")
        collect_gradients(gpu, data, _proc(16), cfg, batches=batches, scorer=scorer)
        writer.flush()
        sc = load_scores(path)
        assert sc.is_written()
        got = torch.from_numpy(np.array(sc[:]))
        assert got.shape == ref.shape
        assert (got - ref).abs().max().item() <= 1e-3


def test_attributor_search_and_trace(device, tmp_path):
    from bergson_amd import Attributor, IndexConfig, collect_gradients

    lengths = [40, 22, 31, 17, 48, 12, 25, 36]
    docs, data, batches, cpu, gpu = _setup(device, lengths)
    cfg = IndexConfig(run_path=str(tmp_path / "idx"), projection_dim=16, projection_type="normal")
    collect_gradients(gpu, data, _proc(16), cfg, batches=batches)
    rows, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
    mods = list(oloop.target_linears(cpu.base_model))
    cols = ostore.column_offsets({m: 256 for m in mods})
    index = {m: rows[:, lo:hi] for m, (lo, hi) in cols.items()}

    attr = Attributor(cfg.partial_run_path, device="cuda:0", unit_norm=True)
    assert attr.N == len(docs) and attr.ordered_modules == mods
    queries = {m: index[m][[1, 6]] for m in mods}
    vals, idx = attr.search({m: q.to(device) for m, q in queries.items()}, k=3)
    ref_v, ref_i = oscan.attributor_search(index, queries, mods, 3, unit_norm=True)
    assert idx[:, 0].tolist() == [1, 6] and (vals[:, 0] > 0.999).all()
    assert torch.equal(idx.cpu(), ref_i)
    assert (vals.cpu() - ref_v).abs().max().item() <= 1e-3
    rv, ri = attr.search({m: q.to(device) for m, q in queries.items()}, k=2, reverse=True)
    ref_rv, ref_ri = oscan.attributor_search(index, queries, mods, 2, unit_norm=True, reverse=True)
    assert torch.equal(ri.cpu(), ref_ri) and (rv.cpu() - ref_rv).abs().max().item() <= 1e-3
    # a subset of modules: the other modules' query columns do not contribute
    sub = set(mods[:3])
    sv, si = attr.search({m: q.to(device) for m, q in queries.items()}, k=4, modules=sub)
    norm_i = oscan.attributor_normalize_index({m: index[m] for m in mods}, mods)
    qcat = torch.cat([queries[m] for m in mods], 1)
    qnorm = {m: queries[m] / (qcat.norm(dim=1, keepdim=True) + torch.finfo(torch.float32).eps) for m in mods}
    ref_sub = sum(qnorm[m] @ norm_i[m].T for m in mods[:3])
    rsv, rsi = torch.topk(ref_sub, 4, dim=1)
    assert torch.equal(si.cpu(), rsi) and (sv.cpu() - rsv).abs().max().item() <= 1e-3

    # trace(): the gradient of document 3's loss finds document 3
    from bergson_amd import pad_and_tensor
    with attr.trace(gpu.base_model, 2) as result:
        x, y, _, _ = pad_and_tensor([docs[3]], device=device, sync_max_len=False)
        logits = gpu(x).logits[:, :-1]
        loss = torch.nn.functional.cross_entropy(logits.reshape(-1, logits.size(-1)), y[:, 1:].flatten(), reduction="sum")
        loss.backward()
        gpu.zero_grad()
    assert result.indices[0, 0].item() == 3 and result.scores[0, 0].item() > 0.99


def test_attributor_searches_again_and_notices_a_changed_store(device, tmp_path):
    """The row norms are formed once when the index is loaded and serve every search: a search with 4 queries
    and one with 300 (another kernel) against the oracle's search, and -- the norms being a cache of `store` --
    rows edited in place or a replaced store are seen by the next search."""
    from bergson_amd import Attributor, ops
    from bergson_amd.data import create_index
    from bergson_amd.gradients import GradientProcessor

    gen = torch.Generator().manual_seed(11)
    n, sizes = 6000, {"a": 256, "b": 128, "c": 128}
    rows = torch.randn(n, 512, generator=gen) * (torch.rand(n, 1, generator=gen) * 3 + 0.1)
    path = tmp_path / "idx"
    mm = create_index(path, num_grads=n, grad_sizes=sizes, dtype="float16")
    mm[:] = rows.to(torch.float16).numpy()
    mm.flush()
    GradientProcessor(projection_dim=16).save(path)
    stored = torch.from_numpy(np.array(mm)).float()
    index = {"a": stored[:, :256], "b": stored[:, 256:384], "c": stored[:, 384:]}
    attr = Attributor(path, device="cuda:0", unit_norm=True)
    assert attr._row_sumsq is not None   # formed at load time, before any search
    assert torch.equal(attr._row_sumsq, ops.row_sumsq(attr.store))
    for Q in (4, 300, 4):
        picks = torch.randint(0, n, (Q,), generator=gen)
        noisy = stored[picks] + 0.3 * torch.randn(Q, 512, generator=gen) * stored[picks].norm(dim=1, keepdim=True) / 512 ** 0.5
        queries = {"a": noisy[:, :256], "b": noisy[:, 256:384], "c": noisy[:, 384:]}
        vals, idx = attr.search({m: q.to(device) for m, q in queries.items()}, k=5)
        ref_v, ref_i = oscan.attributor_search(index, queries, ["a", "b", "c"], 5, unit_norm=True)
        assert (idx[:, 0].cpu() == picks).all()
        assert (vals.cpu() - ref_v).abs().max().item() <= 1e-3
        assert (idx.cpu() == ref_i).float().mean().item() >= 0.98   # neighbours within the tolerance may swap
    # an in-place edit: row 17 becomes a scaled copy of the first query, and must now be its best match
    first = torch.cat([queries[m][0] for m in ("a", "b", "c")])
    attr.store[17] = (first * 100).to(torch.float16).to(device)
    vals, idx = attr.search({m: q.to(device) for m, q in queries.items()}, k=2)
    assert idx[0, 0].item() == 17 and abs(vals[0, 0].item() - 1.0) <= 1e-3
    # a replaced store
    attr.store = attr.store[:100].clone()
    attr.N = 100
    vals, idx = attr.search({m: q.to(device) for m, q in queries.items()}, k=2)
    assert attr._row_sumsq.shape == (100,) and idx[0, 0].item() == 17


def test_include_bias_end_to_end(device):
    """include_bias=True through the collector: every module's block against the oracle on captured (a, g)."""
    from bergson_amd import GradientCollector, GradientProcessor, IndexConfig
    from bergson_amd.collector import CollectorComputer

    lengths = [30, 22]
    docs, data, batches, cpu, gpu = _setup(device, lengths, layers=1)
    names = list(oloop.target_linears(cpu.base_model))
    captured = {}
    handles = []
    for name in names:
        mod = gpu.base_model.get_submodule(name)
        handles.append(mod.register_forward_hook(
            lambda m, inp, out, name=name: captured.setdefault(name, {}).__setitem__("a", inp[0].detach().cpu())))
        handles.append(mod.register_full_backward_hook(
            lambda m, gin, gout, name=name: captured[name].__setitem__("g", gout[0].detach().cpu())))
    cfg = IndexConfig(projection_dim=16, projection_type="normal", include_bias=True)
    proc = GradientProcessor(projection_dim=16, projection_type="normal", include_bias=True)
    col = GradientCollector(model=gpu.base_model, cfg=cfg, data=data, processor=proc)
    CollectorComputer(model=gpu, data=data, collector=col, batches=[[0, 1]], cfg=cfg).run_with_collector_hooks()
    for h in handles:
        h.remove()
    got = torch.from_numpy(np.array(col.builder.grad_buffer))
    for b, name in enumerate(names):
        a, g = captured[name]["a"], captured[name]["g"]
        left, right = module_projections(name, 16, g.shape[-1], a.shape[-1], torch.float32, collect_bias=True)
        want = ohooks.module_gradient(a, g, None, left, right, collect_bias=True)
        assert rel_l2(got[:, b * 256:(b + 1) * 256], want) <= 1e-4, name


def test_build_then_score_entry_points(device, tmp_path):
    """`build` a query store and a training store, then `score_dataset` on the fly: the scores equal the
    oracle's scorer applied to the oracle's rows; query slices give the same file."""
    from bergson_amd import IndexConfig, PreprocessConfig, ScoreConfig, build, load_gradients, score_dataset
    from bergson_amd.data import load_scores
    from bergson_amd.synthetic import ListDataset, random_docs

    lengths = [40, 22, 31, 17, 48, 12]
    docs, data, batches, cpu, gpu = _setup(device, lengths)
    qlengths = [20, 35, 28]
    qdocs = random_docs(qlengths, seed=77)
    qdata = ListDataset(qdocs)

    qcfg = IndexConfig(run_path=str(tmp_path / "query"), projection_dim=16, projection_type="normal",
                       token_batch_size=96)
    build(qcfg, model=gpu, data=qdata)
    assert (tmp_path / "query" / "gradients.bin").exists() and not (tmp_path / "query.part").exists()
    assert (tmp_path / "query" / "processor_config.yaml").exists()
    qrows = torch.from_numpy(np.array(load_gradients(tmp_path / "query")))
    qwant, _ = oloop.collect(cpu, cpu.base_model, qdocs, oloop.allocate_batches(qlengths, 96), p=16)
    assert rel_l2(qrows, qwant) <= 1e-3

    rows, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
    mods = list(oloop.target_linears(cpu.base_model))
    cols = ostore.column_offsets({m: 256 for m in mods})
    index = {m: rows[:, lo:hi] for m, (lo, hi) in cols.items()}
    queries = {m: qwant[:, lo:hi] for m, (lo, hi) in cols.items()}
    qn = oscan.normalize_and_aggregate_queries(queries, mods, unit_normalize=True)
    want = oscan.scorer_score(index, qn, mods, unit_normalize=True)

    for name, qbs in (("scores_all", None), ("scores_sliced", 2)):
        icfg = IndexConfig(run_path=str(tmp_path / name), projection_dim=16, projection_type="normal",
                           token_batch_size=96)
        scfg = ScoreConfig(query_path=str(tmp_path / "query"), query_batch_size=qbs)
        score_dataset(icfg, scfg, PreprocessConfig(unit_normalize=True), model=gpu, data=data)
        sc = load_scores(tmp_path / name)
        assert sc.is_written() and sc.num_scores == 3
        got = torch.from_numpy(np.array(sc[:]))
        assert (got - want).abs().max().item() <= 1e-3


@pytest.mark.parametrize("unit_norm", [True, False])
def test_attributor_streams_a_store_that_does_not_fit(device, tmp_path, unit_norm):
    """A store larger than the device budget stays mapped on the host and is searched in slabs of rows: the
    resident store's values to fp32 rounding (a slab of 700 rows and a store of 5000 go to different kernels,
    which add up over D in different orders), the same rows up to swaps of scores that close, row numbers counted
    over the whole store; k above a slab's row count and a second search (the slabs' row norms are kept)
    included."""
    from bergson_amd import Attributor, GradientProcessor
    from bergson_amd.data import create_index

    n, sizes = 5000, {"a": 192, "b": 64}
    gen = torch.Generator().manual_seed(21)
    rows = torch.randn(n, 256, generator=gen) * (torch.rand(n, 1, generator=gen) * 2 + 0.2)
    path = tmp_path / "slabs"
    mm = create_index(path, n, sizes, "float16")
    mm[:] = rows.to(torch.float16).numpy()
    mm.flush()
    GradientProcessor(projection_dim=None).save(path)
    resident = Attributor(path, device="cuda:0", unit_norm=unit_norm)
    streamed = Attributor(path, device="cuda:0", unit_norm=unit_norm, device_store_bytes=700 * 256 * 2)
    assert resident.store is not None and streamed.store is None and streamed._slab_rows == 700
    with pytest.raises(RuntimeError, match="slabs"):
        streamed.grads
    picks = torch.tensor([3, 699, 700, 2500, 4999])
    q = rows[picks] + 0.05 * torch.randn(5, 256, generator=gen)
    queries = {"a": q[:, :192].to(device), "b": q[:, 192:].to(device)}
    for k in (1, 10, 900, 10):
        v0, i0 = resident.search(queries, k)
        v1, i1 = streamed.search(queries, k)
        assert v1.shape == (5, k) and torch.allclose(v0, v1, rtol=1e-5, atol=2e-5)
        assert (i0 == i1).float().mean().item() >= 0.98
        assert not unit_norm or (i1[:, 0].cpu() == picks).all()  # by cosine a noisy copy finds its original
    assert sorted(streamed._slab_sumsq) == (list(range(0, n, 700)) if unit_norm else [])
    rv0, ri0 = resident.search(queries, 4, reverse=True)
    rv1, ri1 = streamed.search(queries, 4, reverse=True)
    assert torch.allclose(rv0, rv1, rtol=1e-5, atol=2e-5) and (ri0 == ri1).float().mean().item() >= 0.9


def test_attributor_full_ranking_beyond_the_fused_top_k(device, tmp_path):
    """k = None ranks the whole store (attributor.py:229-235 with k = None -> N); past the fused selection's
    2048 entries the scan writes every score and the ranking is torch.topk's."""
    from bergson_amd import Attributor, GradientProcessor
    from bergson_amd.data import create_index

    n, sizes = 2500, {"a": 48, "b": 80}
    gen = torch.Generator().manual_seed(9)
    rows = torch.randn(n, 128, generator=gen)
    path = tmp_path / "big"
    mm = create_index(path, n, sizes, np.float32)
    mm[:] = rows.numpy()
    mm.flush()
    GradientProcessor(projection_dim=None).save(path)
    attr = Attributor(path, device="cuda:0", unit_norm=True)
    q = rows[[7, 1900]]
    vals, idx = attr.search({"a": q[:, :48].to(device), "b": q[:, 48:].to(device)}, k=None)
    assert vals.shape == (2, n) and idx.shape == (2, n)
    index = {"a": rows[:, :48], "b": rows[:, 48:]}
    ref_v, ref_i = oscan.attributor_search(index, {"a": q[:, :48], "b": q[:, 48:]}, ["a", "b"], n, unit_norm=True)
    assert idx[:, 0].tolist() == [7, 1900]
    assert (vals.cpu() - ref_v).abs().max().item() <= 1e-3
    assert (idx.cpu() == ref_i).float().mean().item() > 0.99  # neighbours closer than the tolerance may swap
    assert all(sorted(r.tolist()) == list(range(n)) for r in idx.cpu())


@pytest.mark.parametrize("store_dtype", ["bfloat16", "float16"])
def test_attributor_on_16_bit_stores_against_fp32_search(device, tmp_path, store_dtype):
    """The reference scores a 16-bit store in fp32 against fp32 queries (attributor.py:137-167, dtype default);
    here the scan multiplies the store by queries rounded to the store dtype, so a score can be off by
    2^-9 |g||q| (bf16) or 2^-12 |g||q| (fp16) in the worst case and by 1 / sqrt(D) of that typically.
    Pinned with an explicit tolerance: values within 2e-3 / 1e-3 of the fp32 search over the same stored
    values, planted self-matches first, and every reported row scoring within that tolerance of the k-th
    best fp32 score."""
    from bergson_amd import Attributor, GradientProcessor
    from bergson_amd.data import create_index
    from bergson_amd.utils import tensor_to_numpy

    n, sizes, k = 3000, {"a": 96, "b": 160}, 50
    tdt = torch.bfloat16 if store_dtype == "bfloat16" else torch.float16
    tol = 2e-3 if store_dtype == "bfloat16" else 1e-3
    gen = torch.Generator().manual_seed(21)
    rows = torch.randn(n, 256, generator=gen).to(tdt)
    path = tmp_path / store_dtype
    mm = create_index(path, n, sizes, store_dtype)
    mm[:] = tensor_to_numpy(rows)
    mm.flush()
    GradientProcessor(projection_dim=None).save(path)
    attr = Attributor(path, device="cuda:0", unit_norm=True)
    q = torch.randn(6, 256, generator=gen)
    q[:2] = rows[[11, 2222]].float() + 0.01 * torch.randn(2, 256, generator=gen)
    vals, idx = attr.search({"a": q[:, :96].to(device), "b": q[:, 96:].to(device)}, k=k)
    stored = rows.float()
    index = {"a": stored[:, :96], "b": stored[:, 96:]}
    ref_v, ref_i = oscan.attributor_search(index, {"a": q[:, :96], "b": q[:, 96:]}, ["a", "b"], k, unit_norm=True)
    assert idx[:2, 0].tolist() == [11, 2222]
    assert (vals.cpu() - ref_v).abs().max().item() <= tol
    # the fp32 score of every reported row reaches the k-th best fp32 score up to the tolerance
    full_v, _ = oscan.attributor_search(index, {"a": q[:, :96], "b": q[:, 96:]}, ["a", "b"], n, unit_norm=True)
    _, order = oscan.attributor_search(index, {"a": q[:, :96], "b": q[:, 96:]}, ["a", "b"], n, unit_norm=True)
    score_of = torch.empty(6, n)
    score_of.scatter_(1, order, full_v)
    reported = score_of.gather(1, idx.cpu())
    assert bool((reported >= ref_v[:, -1:] - tol).all())
    assert (idx.cpu() == ref_i).float().mean().item() > 0.9


@pytest.mark.parametrize("attribute_tokens", [False, True])
def test_builder_flushes_only_changed_rows(device, tmp_path, attribute_tokens):
    """Device-resident store: rows reach the file at flush(), run by run of changed rows; a second flush after
    more batches adds exactly those; rows never written stay zero; the memory map sees what was written."""
    from bergson_amd import Builder, PreprocessConfig, load_gradients
    from bergson_amd.builder import RowBlock
    from bergson_amd.synthetic import ListDataset

    lengths = [5, 3, 9, 2, 7, 4, 6, 8, 3, 5, 2, 9] * 20
    data = ListDataset([[1] * l for l in lengths])
    sizes = {"a": 64, "b": 32}
    b = Builder(data, sizes, torch.float16, PreprocessConfig(), attribute_tokens=attribute_tokens,
                path=tmp_path / "store", device=torch.device(device))
    assert b.direct and b.device_rows is not None
    n_rows = b.device_rows.shape[0]
    want = torch.zeros((n_rows, 96), dtype=torch.float16)
    gen = torch.Generator().manual_seed(3)

    def write(docs):
        if attribute_tokens:
            rows = torch.cat([torch.arange(int(b.offsets[i]), int(b.offsets[i + 1])) for i in docs])
        else:
            rows = torch.tensor(docs)
        vals = torch.randn(len(rows), 96, generator=gen).to(torch.float16)
        want[rows] = vals
        b.device_rows[rows.to(device)] = vals.to(device)      # what the collection kernel does on the direct path
        block = RowBlock()
        block.committed = True
        b(docs, block)

    write([0, 1, 2, 200, 201])
    write([77])
    runs = b._dirty_runs()
    assert 2 <= len(runs) <= 3 and all(lo < hi for lo, hi in runs)
    b.flush()
    assert b._dirty_runs() == []
    assert torch.equal(torch.from_numpy(np.array(b.grad_buffer)), want)          # through the memory map
    assert torch.equal(torch.from_numpy(np.array(load_gradients(tmp_path / "store"))), want)  # through the file
    write([5, 6, 239, 100])
    b.teardown()
    got = torch.from_numpy(np.array(load_gradients(tmp_path / "store")))
    assert torch.equal(got, want)
    assert (got.abs().sum(1) == 0).sum() >= n_rows // 2    # most rows were never written and are still zero
