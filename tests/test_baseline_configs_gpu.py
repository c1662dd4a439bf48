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
