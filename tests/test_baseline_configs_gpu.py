"""The five benchmark configurations as parity cases.

Where the CPU oracle finishes in seconds the kernels are compared with it at the configuration's real
module shapes (on a few tokens); at the configurations' full sizes they are checked through properties
that do not depend on the size: linearity over tokens, batch-composition invariance, self-match,
pass-size invariance, agreement of the reported top-k values with a dense rescoring of the reported rows.

Tolerances: rel-L2 <= 1e-2 for bf16 inputs; scores within 1e-3 absolute cosine.
"""
import pytest
import torch

from helpers import TOL, rel_l2
from oracle import hooks as ohooks
from oracle.projection import module_projections

pytestmark = pytest.mark.gpu


def _case(N, S, I, O, p, dtype, seed, kind, name, g_scale=0.05):
    gen = torch.Generator().manual_seed(seed)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * g_scale).to(dtype)
    left, right = module_projections(name, p, O, I, dtype)
    if kind == "adafactor":  # second moments |N(0,1)| * 1e-4
        norm = ohooks.Adafactor(row=torch.randn(O, generator=gen).abs() * 1e-4 + 1e-12,
                                col=torch.randn(I, generator=gen).abs() * 1e-4 + 1e-12)
    elif kind == "adam":  # |N(0,1)| * 1e-5
        norm = ohooks.Adam(torch.randn(O, I, generator=gen).abs() * 1e-5 + 1e-12)
    else:
        norm = None
    return a, g, left, right, norm


def _collect_seq(device, cases, p, out_dtype, lengths=None):
    from bergson_amd import ops

    mods, col = [], 0
    for a, g, left, right, norm in cases:
        rs = cs = None
        if norm is not None:
            rs, cs = ops.adafactor_scales(norm.row.to(device), norm.col.to(device), a.dtype)
        mods.append(ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right.to(device), r_out=left.to(device),
                                    out_col=col, col_scale=cs, row_scale=rs))
        col += p * p
    out = torch.zeros(cases[0][0].shape[0], col, dtype=out_dtype, device=device)
    ldev = None if lengths is None else torch.tensor(lengths, dtype=torch.int32, device=device)
    ops.collect_seq(mods, p, out, lengths=ldev, lo=torch.finfo(out_dtype).min, hi=torch.finfo(out_dtype).max)
    torch.cuda.synchronize()
    return out


# ---- configuration 5: Llama-3-8B module shapes, p = 16, Adafactor, bf16 -> fp16 store ------------------
@pytest.mark.parametrize("shape", [(4096, 14336), (14336, 4096), (4096, 1024), (4096, 4096)])
def test_llama8b_module_shapes_against_oracle(device, shape):
    I, O = shape
    # output gradients of a realistic size keep the normalised values inside the fp16 range
    a, g, left, right, norm = _case(2, 96, I, O, 16, torch.bfloat16, 70, "adafactor", "layers.0.mlp.up_proj",
                                    g_scale=1e-4)
    want = ohooks.module_gradient(a, g, norm, left, right).float().clamp(-65504, 65504)
    assert want.abs().max() < 65504
    got = _collect_seq(device, [(a, g, left, right, norm)], 16, torch.float16).float().cpu()
    assert torch.isfinite(got).all()
    assert rel_l2(got, want) <= TOL[torch.bfloat16]


# ---- configuration 4: Pythia-410m module shapes, p = 32, Adam, per token ---------------------------------
@pytest.mark.parametrize("shape", [(1024, 3072), (1024, 1024), (1024, 4096), (4096, 1024)])
def test_pythia410m_adam_per_token_against_oracle(device, shape):
    from bergson_amd import ops

    I, O = shape
    N, S, p = 2, 9, 32
    lengths = [9, 6]
    a, g, left, right, norm = _case(N, S, I, O, p, torch.bfloat16, 71, "adam", "layers.3.mlp.dense_h_to_4h")
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
    prep = ops.AdamPrepared(right.to(device), left.to(device), norm.weight_avg_sq.to(device), 0)
    counts = [l - 1 for l in lengths]
    out = torch.zeros(sum(counts), p * p, dtype=torch.bfloat16, device=device)
    ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=True,
                     lengths=torch.tensor(lengths, dtype=torch.int32, device=device),
                     rows=torch.tensor([0, counts[0]], dtype=torch.int64, device=device),
                     lo=torch.finfo(torch.bfloat16).min, hi=torch.finfo(torch.bfloat16).max)
    torch.cuda.synchronize()
    assert rel_l2(out.cpu(), want) <= TOL[torch.bfloat16]


def _adam_closed_form_fp64(a_t, g_t, v, left, right):
    """P_t = L (g_t a_t^T / (sqrt(v) + 1e-8)) R^T for one token in float64, from the formula
    (bergson/gradients.py:380-388 applied to the outer product of collector.py:611-612)."""
    full = torch.outer(g_t.double(), a_t.double()) / (v.double().sqrt() + 1e-8)
    return (left.double() @ full @ right.double().T).flatten()


@pytest.mark.parametrize("shape", [(1024, 3072), (1024, 1024), (1024, 4096), (4096, 1024)])
def test_pythia410m_adam_per_token_whole_tiles_sampled_against_oracle(device, shape):
    """The configuration's production route -- whole 256-token tiles on the four-wave fused kernel -- held to the
    oracle directly: per-token rows do not depend on each other, so the oracle and the float64 closed form are
    evaluated on a sample of the tokens of a full launch (first and last token of every tile, the last valid
    token of each sequence, random interior ones).  Two sequences of 512, the second ragged."""
    from bergson_amd import _lib, ops

    I, O = shape
    N, S, p = 2, 512, 32
    lengths = [512, 389]
    a, g, left, right, norm = _case(N, S, I, O, p, torch.bfloat16, 72, "adam", "layers.5.mlp.dense_4h_to_h")
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    prep = ops.AdamPrepared(right.to(device), left.to(device), norm.weight_avg_sq.to(device), 0)
    counts = [l - 1 for l in lengths]
    offs = [0, counts[0]]

    def run(out_dtype, per_token=True):
        out = torch.zeros(sum(counts) if per_token else N, p * p, dtype=out_dtype, device=device)
        ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=per_token,
                         lengths=torch.tensor(lengths, dtype=torch.int32, device=device),
                         rows=torch.tensor(offs if per_token else [0, 1], dtype=torch.int64, device=device),
                         lo=torch.finfo(out_dtype).min, hi=torch.finfo(out_dtype).max)
        torch.cuda.synchronize()
        return out.cpu()

    got = run(torch.bfloat16)
    assert _lib.last_kernel(_lib.FAMILY_ADAM) == "adam_fused_wide"   # no switch set: this is the default route
    got32 = run(torch.float32)
    assert torch.isfinite(got32).all()
    gen = torch.Generator().manual_seed(5)
    for n in range(N):
        last = counts[n] - 1
        idx = {0, 255, 256, last, last - 1, 1, 254, 257}
        idx |= {t for t in (511, 510) if t <= last}
        idx |= set(torch.randint(2, last, (12,), generator=gen).tolist())
        idx = sorted(idx)
        ones = torch.ones(1, len(idx), dtype=torch.bool)
        want = ohooks.module_gradient(a[n:n + 1, idx], g[n:n + 1, idx], norm, left, right, attribute_tokens=True,
                                      collection_mask=ones)
        rows = torch.tensor(idx) + offs[n]
        assert rel_l2(got[rows], want) <= TOL[torch.bfloat16]
        for j, t in enumerate(idx):   # each sampled token on its own, so one wrong row cannot hide in the norm
            assert rel_l2(got[rows[j]], want[j]) <= 2 * TOL[torch.bfloat16], (n, t)
        for t in idx[:6] + idx[-3:]:
            exact = _adam_closed_form_fp64(a[n, t], g[n, t], norm.weight_avg_sq, left, right)
            assert rel_l2(got32[offs[n] + t], exact) <= TOL[torch.bfloat16], (n, t)
    # the per-sequence rows of the same inputs against the sum of the per-token rows
    seq = run(torch.float32, per_token=False)
    for n in range(N):
        assert rel_l2(seq[n], got32[offs[n]:offs[n] + counts[n]].sum(0)) <= TOL[torch.bfloat16]


def test_pythia410m_width_two_layers_adam_per_token_through_the_model(device):
    """Two layers at the Pythia-410m widths (1024 / 4096, 16 heads), bf16, Adam second moments, p = 32, per-token
    rows, two documents of 512 and 389 tokens in one batch through the product loop; every module's block of
    sampled tokens against the oracle on the (a, g) the hooks saw."""
    import numpy as np
    from bergson_amd import AdamNormalizer, GradientCollector, GradientProcessor, IndexConfig
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [512, 389]
    p = 32
    docs = random_docs(lengths, seed=23)
    model = make_gpt_neox("pythia-410m", torch.bfloat16, device, seed=0, layers=2)
    gen = torch.Generator().manual_seed(9)
    moments, captured, handles = {}, {}, []
    for name, mod in model.base_model.named_modules():
        if isinstance(mod, torch.nn.Linear):
            moments[name] = torch.randn(mod.weight.shape, generator=gen).abs() * 1e-5 + 1e-12
            handles.append(mod.register_forward_hook(
                lambda m, inp, out, name=name: captured.setdefault(name, {}).__setitem__("a", inp[0].detach().cpu())))
            handles.append(mod.register_full_backward_hook(
                lambda m, gin, gout, name=name: captured[name].__setitem__("g", gout[0].detach().cpu())))
    names = list(moments)
    assert len(names) == 8
    normalizers = {n: AdamNormalizer(weight_avg_sq=v.to(device)) for n, v in moments.items()}
    cfg = IndexConfig(run_path="", projection_dim=p, projection_type="normal", attribute_tokens=True)
    col = GradientCollector(model=model.base_model, cfg=cfg, data=ListDataset(docs),
                            processor=GradientProcessor(normalizers=normalizers, projection_dim=p,
                                                        projection_type="normal"))
    CollectorComputer(model=model, data=ListDataset(docs), collector=col, batches=[[0, 1]], cfg=cfg
                      ).run_with_collector_hooks()
    torch.cuda.synchronize()
    for h in handles:
        h.remove()
    assert col.builder.base_dtype == "bfloat16"   # the model's gradient dtype; numpy maps it as uint16 bit patterns
    got = torch.from_numpy(np.array(col.builder.grad_buffer).view(np.int16)).view(torch.bfloat16).float()
    counts = [l - 1 for l in lengths]
    assert got.shape == (sum(counts), 8 * p * p) and torch.isfinite(got).all()
    sample = {0: [0, 1, 255, 256, 300, 509, 510], 1: [0, 17, 255, 256, 386, 387]}
    for name in names:
        a, g = captured[name]["a"], captured[name]["g"]
        left, right = module_projections(name, p, g.shape[-1], a.shape[-1], torch.bfloat16)
        b = names.index(name)
        for n, idx in sample.items():
            ones = torch.ones(1, len(idx), dtype=torch.bool)
            want = ohooks.module_gradient(a[n:n + 1, idx], g[n:n + 1, idx], ohooks.Adam(moments[name]), left, right,
                                          attribute_tokens=True, collection_mask=ones).float()
            rows = torch.tensor(idx) + (0 if n == 0 else counts[0])
            block = got[rows, b * p * p:(b + 1) * p * p]
            assert want.abs().max() > 0
            assert rel_l2(block, want) <= TOL[torch.bfloat16], (name, n)


# ---- configuration 2 at full size: 4096-token batch, all 48 Pythia-160m modules ----------------------------
def _pythia160m_modules(N, S, seed):
    d = 768
    cases = []
    for layer in range(12):
        for j, (I, O) in enumerate([(d, 3 * d), (d, d), (d, 4 * d), (4 * d, d)]):
            cases.append(_case(N, S, I, O, 16, torch.bfloat16, seed + 4 * layer + j, "adafactor",
                               f"layers.{layer}.m{j}"))
    return cases


def test_pythia160m_full_batch_properties(device):
    """One 4096-token batch over 48 modules (1.2 GB of a and g): (i) the rows do not depend on how the
    documents are batched, (ii) the per-token rows of a document sum to its per-sequence row, (iii) skipping
    the padding of a causal batch changes nothing, (iv) one module against the oracle."""
    from bergson_amd import ops

    N, S, p = 4, 1024, 16
    lengths = [1024, 700, 1024, 129]
    cases = _pythia160m_modules(N, S, seed=100)
    for a, g, *_ in cases:
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0  # what a causal model with right padding produces
    full = _collect_seq(device, cases, p, torch.float32)
    assert full.shape == (N, 48 * 256) and torch.isfinite(full).all()

    # (i) documents 0,1 and 2,3 in separate launches, the second pair trimmed to its own padded length
    first = _collect_seq(device, [(a[:2], g[:2], l, r, nm) for a, g, l, r, nm in cases], p, torch.float32)
    assert rel_l2(first.cpu(), full[:2].cpu()) <= 1e-6
    one = _collect_seq(device, [(a[3:, :192].contiguous(), g[3:, :192].contiguous(), l, r, nm)
                                for a, g, l, r, nm in cases], p, torch.float32)
    assert rel_l2(one.cpu(), full[3:].cpu()) <= 1e-5

    # (iii) lengths given: padded positions are not read
    skipped = _collect_seq(device, cases, p, torch.float32, lengths=lengths)
    assert rel_l2(skipped.cpu(), full.cpu()) <= 1e-6

    # (ii) per-token rows of every document sum to its per-sequence row
    mods, col = [], 0
    for a, g, left, right, norm in cases:
        rs, cs = ops.adafactor_scales(norm.row.to(device), norm.col.to(device), a.dtype)
        mods.append(ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right.to(device), r_out=left.to(device),
                                    out_col=col, col_scale=cs, row_scale=rs))
        col += p * p
    counts = [l - 1 for l in lengths]
    offs = [sum(counts[:n]) for n in range(N)]
    tok = torch.zeros(sum(counts), col, dtype=torch.float32, device=device)
    ops.collect_tok(mods, p, tok, lengths=torch.tensor(lengths, dtype=torch.int32, device=device),
                    row_offsets=torch.tensor(offs, dtype=torch.int64, device=device))
    torch.cuda.synchronize()
    for n in range(N):
        assert rel_l2(tok[offs[n]:offs[n] + counts[n]].sum(0).cpu(), full[n].cpu()) <= 1e-4

    # (iv) the widest module against the oracle
    a, g, left, right, norm = cases[3]
    want = ohooks.module_gradient(a, g, norm, left, right).float()
    assert rel_l2(full[:, 3 * 256:4 * 256].cpu(), want) <= TOL[torch.bfloat16]


# ---- configuration 3 at full size: 10^6 x 12288 fp16 rows, 1024 queries, k = 100 ---------------------------
def test_store_scan_full_size_properties(device):
    from bergson_amd import ops

    n, D, Q, k = 1_000_000, 12288, 1024, 100
    free, _ = torch.cuda.mem_get_info()
    if free < 40 * 2**30:
        pytest.skip("needs 40 GB of free HBM")
    gen = torch.Generator(device=device).manual_seed(1)
    store = torch.empty((n, D), dtype=torch.float16, device=device)
    for lo in range(0, n, 65536):
        hi = min(n, lo + 65536)
        blk = torch.randn((hi - lo, D), generator=gen, device=device)
        heavy = torch.rand((hi - lo, 1), generator=gen, device=device) < 0.05
        store[lo:hi] = (blk * torch.where(heavy, 10.0, 1.0)).to(torch.float16)
    q = torch.randn((Q, D), generator=gen, device=device)
    # the first 64 queries are noisy copies of known store rows, so their best match is known
    planted = torch.randint(0, n, (64,), generator=gen, device=device)
    q[:64] = store[planted].float() + 0.05 * q[:64] * store[planted].float().norm(dim=1, keepdim=True) / D ** 0.5
    q = q / q.norm(dim=1, keepdim=True)
    qd = (q * 64.0).to(torch.float16)

    res = ops.scan(store, qd, unit_norm=True, k=k, query_scale=1.0 / 64.0, want_row_max=True, want_row_mean=True)
    torch.cuda.synchronize()
    vals, idx = res.topk_values, res.topk_indices
    assert (idx[:64, 0] == planted).all() and (vals[:64, 0] > 0.99).all()
    assert (vals[:, :-1] >= vals[:, 1:]).all()
    assert int(idx.min()) >= 0 and int(idx.max()) < n
    assert all(len(set(r.tolist())) == k for r in idx[:32].cpu())

    # the reported values are the cosines of the reported rows (dense fp32 rescoring of 16 queries)
    qn = (qd.float() / 64.0)
    for qi in (0, 63, 64, 500, 1023):
        rows = store[idx[qi]].float()
        cos = (rows @ qn[qi]) / rows.norm(dim=1)
        assert (cos - vals[qi]).abs().max().item() <= 1e-3

    # nothing outside the reported set beats its k-th value: dense scores of a 50 000-row slice
    sl = store[300_000:350_000].float()
    dense = (sl @ qn[:128].T) / sl.norm(dim=1, keepdim=True)  # [rows, 128]
    assert (dense.max(0).values <= vals[:128, 0] + 1e-3).all()
    in_slice = (idx[:128] >= 300_000) & (idx[:128] < 350_000)
    beat = (dense > (vals[:128, -1] + 1e-3).unsqueeze(0)).sum(0)
    assert (beat <= in_slice.sum(1)).all()
    # row max / mean over the queries on the same slice
    dense_all = (sl[:2000] @ qn.T) / sl[:2000].norm(dim=1, keepdim=True)
    assert (res.row_max[300_000:302_000] - dense_all.max(1).values).abs().max().item() <= 1e-3
    assert (res.row_mean[300_000:302_000] - dense_all.mean(1)).abs().max().item() <= 1e-3

    # the size of the internal passes changes nothing
    res2 = ops.scan(store, qd[:256].contiguous(), unit_norm=True, k=k, query_scale=1.0 / 64.0, chunk_rows=200_000)
    torch.cuda.synchronize()
    # selection is exact on (score, row) keys and a row's score does not depend on the pass it is in
    assert torch.equal(res2.topk_values, vals[:256])
    assert torch.equal(res2.topk_indices, idx[:256])


# ---- configuration 1 at its stated size: Pythia-14m fp32, 64 x 256 tokens, 2048-token batches ------------------
def test_pythia14m_config1_full_size_against_cpu_loop(device):
    """The reference's own CPU-runnable case in full: 64 documents of 256 uniform token ids, batches of 8
    (token_batch_size 2048), p = 16, no normalizer, per sequence, sum reduction -- the product loop on the GPU
    against the oracle's loop on the CPU (rel-L2 <= 1e-3: the model's own fp32 forward/backward differs
    between the devices at rounding level)."""
    import numpy as np
    from bergson_amd import GradientProcessor, IndexConfig, allocate_batches, collect_gradients
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs
    from oracle import loop as oloop

    lengths = [256] * 64
    docs = random_docs(lengths, seed=0)
    batches = allocate_batches(lengths, 2048)
    assert len(batches) == 8 and all(len(b) == 8 for b in batches)
    cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0)
    want, want_losses = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
    gpu = make_gpt_neox("pythia-14m", torch.float32, device, seed=0)
    cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal")
    col = collect_gradients(gpu, ListDataset(docs), GradientProcessor(projection_dim=16, projection_type="normal"),
                            cfg, batches=batches)
    torch.cuda.synchronize()
    got = torch.from_numpy(np.array(col.builder.grad_buffer))
    assert got.shape == want.shape == (64, 24 * 256)
    assert rel_l2(got, want) <= 1e-3
    for m in range(24):  # every module on its own
        assert rel_l2(got[:, m * 256:(m + 1) * 256], want[:, m * 256:(m + 1) * 256]) <= 2e-3, m
    assert torch.allclose(col.per_doc_losses.cpu(), want_losses, rtol=1e-4)
    assert int(col.total_processed) == 64 * 255


# ---- configuration 5 through a model: Llama-3-8B-shaped decoder, bf16, Adafactor, fp16 store -----------------
def _run_llama(device, layers, lengths, vocab, capture):
    """Collects from a Llama-shaped model; returns (store rows, {name: (a, g)} for the modules in `capture`
    -- a predicate on the module name --, moments, names)."""
    import numpy as np
    from bergson_amd import AdafactorNormalizer, GradientCollector, GradientProcessor, IndexConfig
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, adafactor_moments, make_llama, random_docs

    docs = random_docs(lengths, vocab=vocab, seed=21)
    model = make_llama(torch.bfloat16, device, layers=layers, vocab=vocab, seed=0)
    moments = adafactor_moments(model.base_model, seed=0)
    names = list(moments)
    normalizers = {n: AdafactorNormalizer(row=r.to(device), col=c.to(device)) for n, (r, c) in moments.items()}
    captured, handles = {}, []
    for name, mod in model.base_model.named_modules():
        if isinstance(mod, torch.nn.Linear) and capture(name):
            handles.append(mod.register_forward_hook(
                lambda m, inp, out, name=name: captured.setdefault(name, {}).__setitem__("a", inp[0].detach().cpu())))
            handles.append(mod.register_full_backward_hook(
                lambda m, gin, gout, name=name: captured[name].__setitem__("g", gout[0].detach().cpu())))
    cfg = IndexConfig(run_path="", projection_dim=16, projection_type="normal")
    col = GradientCollector(model=model.base_model, cfg=cfg, data=ListDataset(docs), store_dtype=torch.float16,
                            processor=GradientProcessor(normalizers=normalizers, projection_dim=16,
                                                        projection_type="normal"))
    assert list(col.shapes()) == names
    CollectorComputer(model=model, data=ListDataset(docs), collector=col, batches=[list(range(len(docs)))], cfg=cfg
                      ).run_with_collector_hooks()
    torch.cuda.synchronize()
    for h in handles:
        h.remove()
    assert col.builder.base_dtype == "float16"
    got = torch.from_numpy(np.array(col.builder.grad_buffer).astype(np.float32))
    return got, captured, moments, names


def _check_llama_blocks(got, captured, moments, names):
    assert torch.isfinite(got).all()
    for name, ag in captured.items():
        a, g = ag["a"], ag["g"]
        row, col = moments[name]
        left, right = module_projections(name, 16, g.shape[-1], a.shape[-1], torch.bfloat16)
        want = ohooks.module_gradient(a, g, ohooks.Adafactor(row=row, col=col), left, right).float().clamp(-65504, 65504)
        b = names.index(name)
        block = got[:, b * 256:(b + 1) * 256]
        assert want.abs().max() > 0
        assert rel_l2(block, want) <= TOL[torch.bfloat16], name


def test_llama8b_two_layers_through_the_model(device):
    """Two layers at the full Llama-3-8B widths (4096 / 14336, 32 query and 8 key-value heads): target discovery
    on a Llama model, bias-less modules, q/k/v and gate/up sharing one input tensor, the grouped-query widths
    (k_proj, v_proj 4096 -> 1024), ragged documents, modules too wide for their projections to stay on chip --
    every module's block against the oracle on the (a, g) the hooks saw."""
    lengths = [150, 97]
    got, captured, moments, names = _run_llama(device, 2, lengths, 32000, lambda name: True)
    assert len(names) == 14 and got.shape == (2, 14 * 256)
    assert [n.split(".", 2)[2] for n in names[:7]] == ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj",
                                                       "self_attn.o_proj", "mlp.gate_proj", "mlp.up_proj",
                                                       "mlp.down_proj"]
    assert captured["layers.0.self_attn.k_proj"]["g"].shape[-1] == 1024
    assert captured["layers.1.mlp.down_proj"]["a"].shape[-1] == 14336
    _check_llama_blocks(got, captured, moments, names)


def test_llama8b_full_depth_224_modules(device):
    """The whole configuration-5 model shape (32 layers, 224 hooked modules, rows of 57 344 values) in one
    launch per batch; three layers' modules are checked against the oracle on the (a, g) the hooks saw."""
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * 2**30:
        pytest.skip("needs 60 GB of free HBM")
    lengths = [96, 61]
    picked = ("layers.0.", "layers.17.", "layers.31.")
    got, captured, moments, names = _run_llama(device, 32, lengths, 128256, lambda name: name.startswith(picked))
    assert len(names) == 224 and got.shape == (2, 57344) and len(captured) == 21
    _check_llama_blocks(got, captured, moments, names)
    norms = got.view(2, 224, 256).norm(dim=2)
    assert (norms > 0).all()  # every module wrote its block
