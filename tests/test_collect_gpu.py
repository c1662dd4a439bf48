"""HIP collection kernels against the CPU oracle (the reference's op sequence).

Tolerances: relative L2 <= 1e-5 for fp32 inputs, <= 1e-2 for bf16 / fp16 inputs.
"""
import pytest
import torch

from helpers import TOL, rel_l2
from oracle import hooks as ohooks
from oracle.projection import module_projections

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["streamed", "persistent", "grid"], autouse=True)
def kernel_variant(request, bgx_env):
    """Every case runs three times: with the persistent collection kernel and its streamed loads where they
    apply (the default), with the persistent kernel's direct fragment loads, and with the
    one-workgroup-per-tile kernel, the latter two forced through the library's environment switches."""
    bgx_env("BGX_COLLECT_PERSIST", "0" if request.param == "grid" else None)
    bgx_env("BGX_COLLECT_STAGED", "0" if request.param == "persistent" else None)
    return request.param


def make_case(N, S, I, O, p, dtype, seed, normalizer=None, name="layers.0.mlp.dense_h_to_4h"):
    gen = torch.Generator().manual_seed(seed)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    left, right = module_projections(name, p, O, I, dtype)
    norm = None
    if normalizer == "adafactor":
        row = torch.randn(O, generator=gen).abs() * 1e-4
        col = torch.randn(I, generator=gen).abs() * 1e-4
        norm = ohooks.Adafactor(row=row, col=col)
    return a, g, left, right, norm


def run_kernel(device, cases, p, out_dtype, *, lengths=None, per_token=False, row_offsets=None, n_rows=None,
               out_rows=None, lo=float("-inf"), hi=float("inf")):
    from bergson_amd import ops

    mods = []
    col = 0
    for a, g, left, right, norm in cases:
        cs = rs = None
        if norm is not None:
            rs, cs = ops.adafactor_scales(norm.row.to(device), norm.col.to(device), a.dtype)
        mods.append(ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right.to(device), r_out=left.to(device),
                                    out_col=col, col_scale=cs, row_scale=rs))
        col += p * p
    N = cases[0][0].shape[0]
    rows = n_rows if n_rows is not None else N
    out = torch.zeros(rows, col, dtype=out_dtype, device=device)
    ldev = None if lengths is None else torch.tensor(lengths, dtype=torch.int32, device=device)
    if per_token:
        ops.collect_tok(mods, p, out, lengths=ldev, row_offsets=torch.tensor(row_offsets, dtype=torch.int64, device=device),
                        lo=lo, hi=hi)
    else:
        odev = None if out_rows is None else torch.tensor(out_rows, dtype=torch.int64, device=device)
        ops.collect_seq(mods, p, out, lengths=ldev, out_rows=odev, lo=lo, hi=hi)
    torch.cuda.synchronize()
    return out.cpu()


def oracle_rows(cases, out_dtype, **kw):
    lo, hi = torch.finfo(out_dtype).min, torch.finfo(out_dtype).max
    outs = [ohooks.module_gradient(a, g, norm, left, right, lo=lo, hi=hi, **kw).to(out_dtype)
            for a, g, left, right, norm in cases]
    return torch.cat(outs, dim=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 64, 128, 384, 16), (3, 100, 256, 128, 16), (1, 7, 64, 64, 16),
                                   (2, 130, 128, 128, 32), (2, 70, 96, 160, 8), (2, 33, 64, 32, 5),
                                   (1, 65, 128, 64, 48)])
def test_seq_no_normalizer(device, dtype, shape):
    N, S, I, O, p = shape
    case = make_case(N, S, I, O, p, dtype, seed=1)
    out_dtype = dtype
    got = run_kernel(device, [case], p, out_dtype, lo=torch.finfo(out_dtype).min, hi=torch.finfo(out_dtype).max)
    want = oracle_rows([case], out_dtype)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_seq_unaligned_features(device, dtype):
    # odd feature counts take the element-wise loader
    case = make_case(2, 50, 100, 37, 16, dtype, seed=2)
    got = run_kernel(device, [case], 16, dtype)
    want = oracle_rows([case], dtype)
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_seq_adafactor(device, dtype):
    a, g, left, right, norm = make_case(3, 150, 256, 512, 16, dtype, seed=3, normalizer="adafactor")
    case = (a, g * 1e-3, left, right, norm)  # keeps every value inside the fp16 range of the store
    out_dtype = torch.float16 if dtype == torch.bfloat16 else dtype
    lo, hi = torch.finfo(out_dtype).min, torch.finfo(out_dtype).max
    got = run_kernel(device, [case], 16, out_dtype, lo=lo, hi=hi)
    want = oracle_rows([case], out_dtype)
    assert torch.isfinite(got.float()).all()
    assert rel_l2(got, want) <= TOL[dtype]


def test_seq_adafactor_matches_closed_form_fp32(device):
    # independent of the hook formulation: L @ normalize_weight(G^T A) @ R^T per sequence
    a, g, left, right, norm = make_case(2, 40, 64, 96, 16, torch.float32, seed=4, normalizer="adafactor")
    got = run_kernel(device, [(a, g, left, right, norm)], 16, torch.float32)
    full = g.mT.double() @ a.double()  # [N, O, I]
    r = norm.row.double() + 1e-30
    c = norm.col.double() + 1e-30
    full = full * (r.mean().sqrt() * r.rsqrt())[:, None] * c.rsqrt()[None, :]
    want = (left.double() @ full @ right.double().T).flatten(1)
    assert rel_l2(got, want) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_seq_multi_module_and_lengths(device, dtype):
    N, S = 4, 200
    lengths = [200, 131, 64, 2]
    cases = []
    for i, (I, O) in enumerate([(128, 384), (128, 128), (128, 512), (512, 128)]):
        a, g, left, right, norm = make_case(N, S, I, O, 16, dtype, seed=10 + i, normalizer="adafactor",
                                            name=f"layers.{i}.x")
        # a causal model with right padding yields an exactly-zero g from position len-1 on
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        cases.append((a, g, left, right, norm))
    out_rows = [5, 0, 3, 1]
    got = run_kernel(device, cases, 16, dtype, lengths=lengths, out_rows=out_rows, n_rows=6)
    want = oracle_rows(cases, dtype)
    assert rel_l2(got[out_rows], want) <= TOL[dtype]
    assert got[[2, 4]].abs().sum() == 0
    # without lengths the padded positions are read and contribute exactly zero
    got_dense = run_kernel(device, cases, 16, dtype)
    assert rel_l2(got_dense, want) <= TOL[dtype]


def test_seq_bf16_to_fp16_store_saturates_finite(device):
    # A bf16 model writing an fp16 store: the kernel clamps in fp32 at +-65504 and stays finite.  (The
    # reference's clamp_ runs on the bf16 tensor, where the bound rounds up to 65536 and the cast gives inf.)
    a, g, left, right, norm = make_case(2, 128, 256, 256, 16, torch.bfloat16, seed=6, normalizer="adafactor")
    hi = torch.finfo(torch.float16).max
    got = run_kernel(device, [(a, g, left, right, norm)], 16, torch.float16, lo=-hi, hi=hi)
    want = ohooks.module_gradient(a, g, norm, left, right).float()
    assert torch.isfinite(got.float()).all()
    big = want.abs() > 7e4
    assert big.any() and (got.float().abs()[big] == hi).all()
    small = want.abs() < 6e4
    assert rel_l2(got.float()[small], want[small]) <= 1e-2


def test_seq_clamp_to_store_dtype(device):
    a, g, left, right, _ = make_case(1, 64, 64, 64, 16, torch.float32, seed=5)
    g = g * 1e6
    lo, hi = torch.finfo(torch.float16).min, torch.finfo(torch.float16).max
    got = run_kernel(device, [(a, g, left, right, None)], 16, torch.float16, lo=lo, hi=hi)
    want = ohooks.module_gradient(a, g, None, left, right, lo=lo, hi=hi).to(torch.float16)
    assert torch.isfinite(got.float()).all()
    assert (got.float().abs() == hi).any()
    assert rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("per_token", [False, True])
def test_many_tiles_across_modules(device, dtype, per_token):
    """More (module, tile) items than the GPU has CUs, modules of different widths and ragged lengths: a
    persistent workgroup then walks several tiles and crosses module and sequence boundaries."""
    N, S, p = 8, 640, 16
    lengths = [640, 513, 129, 128, 400, 2, 77, 639]
    shapes = [(64, 192), (128, 64), (64, 64), (256, 64), (64, 256), (128, 128), (192, 64), (64, 128)]
    cases = []
    for i, (I, O) in enumerate(shapes):
        a, g, left, right, norm = make_case(N, S, I, O, p, dtype, seed=40 + i, normalizer="adafactor" if i % 2 else None,
                                            name=f"layers.{i}.z")
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        cases.append((a, g, left, right, norm))
    if not per_token:
        got = run_kernel(device, cases, p, dtype, lengths=lengths)
        want = oracle_rows(cases, dtype)
    else:
        counts = [l - 1 for l in lengths]
        row_offsets = [sum(counts[:n]) for n in range(N)]
        mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        got = run_kernel(device, cases, p, dtype, lengths=lengths, per_token=True, row_offsets=row_offsets,
                         n_rows=sum(counts))
        want = oracle_rows(cases, dtype, attribute_tokens=True, collection_mask=mask)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("per_token", [False, True])
def test_long_item_ranges_with_odd_widths(device, dtype, per_token):
    """Several tiles per workgroup, module widths that are odd multiples of the streamed kernel's 128-byte
    unit (so the last block of a segment is partial), sequences shorter than a tile (waves without tokens),
    all-padding tiles in the middle of a range: the input stream runs ahead across all of these."""
    N, S, p = 6, 1536, 16
    lengths = [1536, 1, 700, 1409, 130, 1025]
    unit = 64 if dtype == torch.bfloat16 else 32
    shapes = [(5 * unit, 7 * unit), (unit, 9 * unit), (3 * unit, unit), (6 * unit, 2 * unit), (4 * unit, 11 * unit),
              (13 * unit, 5 * unit), (unit, unit), (10 * unit, 3 * unit)]
    cases = []
    for i, (I, O) in enumerate(shapes):
        a, g, left, right, norm = make_case(N, S, I, O, p, dtype, seed=140 + i, normalizer="adafactor" if i % 3 else None,
                                            name=f"layers.{i}.w")
        for n, l in enumerate(lengths):
            g[n, max(l - 1, 0):] = 0
        cases.append((a, g, left, right, norm))
    if not per_token:
        got = run_kernel(device, cases, p, dtype, lengths=lengths)
        want = oracle_rows(cases, dtype)
    else:
        counts = [l - 1 for l in lengths]
        row_offsets = [sum(counts[:n]) for n in range(N)]
        mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        got = run_kernel(device, cases, p, dtype, lengths=lengths, per_token=True, row_offsets=row_offsets,
                         n_rows=sum(counts))
        want = oracle_rows(cases, dtype, attribute_tokens=True, collection_mask=mask)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("p", [5, 8, 13])
def test_seq_small_projection_dims(device, dtype, p):
    """p < 16: the unused rows / columns of the 16 x 16 MFMA tiles must not leak into the p x p block."""
    cases = [make_case(3, 150, 96, 160, p, dtype, seed=45 + p, normalizer="adafactor" if p != 8 else None)]
    got = run_kernel(device, cases, p, dtype)
    assert got.shape == (3, p * p)
    assert rel_l2(got, oracle_rows(cases, dtype)) <= TOL[dtype]


@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_wide_modules(device, dtype, per_token):
    """I + O too wide for the projection fragments to fit in LDS: the streamed kernel reads them from a table in
    global memory (the default variant), or the launch falls back to the tile kernel (the other two).  Several
    tiles per workgroup, ragged lengths, a narrow module in the same launch."""
    N, S, p = 3, 400, 16
    lengths = [400, 130, 2]
    wide = 4096 if dtype == torch.bfloat16 else 2048
    shapes = [(wide, 1024), (512, wide + 512), (64, 64)]
    cases = []
    for i, (I, O) in enumerate(shapes):
        a, g, left, right, norm = make_case(N, S, I, O, p, dtype, seed=50 + i, normalizer="adafactor" if i != 1 else None,
                                            name=f"layers.{i}.wide")
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        cases.append((a, g, left, right, norm))
    if not per_token:
        got = run_kernel(device, cases, p, dtype, lengths=lengths)
        want = oracle_rows(cases, dtype)
    else:
        counts = [l - 1 for l in lengths]
        row_offsets = [sum(counts[:n]) for n in range(N)]
        mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        got = run_kernel(device, cases, p, dtype, lengths=lengths, per_token=True, row_offsets=row_offsets,
                         n_rows=sum(counts))
        want = oracle_rows(cases, dtype, attribute_tokens=True, collection_mask=mask)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("p,S", [(32, 512), (32, 300), (20, 257), (64, 500), (50, 130)])
def test_seq_wide_projections(device, dtype, p, S, kernel_variant):
    """p > 16: per-sequence rows come from the streamed kernel with two or four blocks of 16 projection columns per
    k-step (the default variant; tiles of 256 tokens where the sequence length wastes little of them, else of 128),
    or from the tile kernel (the other two).  Ragged lengths, a projection dimension that is no multiple of 16, a
    normalizer folded into the fragments, out_rows."""
    from bergson_amd import _lib

    N = 4
    lengths = [S, (2 * S) // 3, 65, 2]
    cases = []
    for i, (I, O) in enumerate([(256, 768), (64, 64), (384, 128)]):
        a, g, left, right, norm = make_case(N, S, I, O, p, dtype, seed=70 + i, normalizer="adafactor" if i == 0 else None,
                                            name=f"layers.{i}.p{p}")
        if norm is not None:
            g = g * 1e-3  # keeps every value inside the fp16 range of the store
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        cases.append((a, g, left, right, norm))
    out_rows = [3, 0, 4, 1]
    got = run_kernel(device, cases, p, dtype, lengths=lengths, out_rows=out_rows, n_rows=5)
    assert _lib.last_kernel(_lib.FAMILY_COLLECT) == ("collect_persist_table" if kernel_variant == "streamed" else "collect_tile")
    want = oracle_rows(cases, dtype)
    assert rel_l2(got[out_rows], want) <= TOL[dtype]
    assert got[2].abs().sum() == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("p,S", [(32, 300), (64, 200), (24, 129), (40, 70), (20, 90)])
def test_tok_wide_projections(device, dtype, p, S, kernel_variant):
    """Per-token rows at p > 16: with p a multiple of 8 the streamed kernel leaves every token's a', g' (32 or 64
    columns each) in the workspace and token_rows_kernel writes the rows (the default variant); other p, and the other
    two variants, take the tile kernel.  Ragged lengths, two modules."""
    from bergson_amd import _lib

    N = 3
    lengths = [S, S // 2 + 1, 2]
    cases = []
    for i, (I, O) in enumerate([(128, 256), (64, 64)]):
        a, g, left, right, norm = make_case(N, S, I, O, p, dtype, seed=80 + i, normalizer="adafactor" if i == 1 else None,
                                            name=f"layers.{i}.tok{p}")
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        cases.append((a, g, left, right, norm))
    counts = [l - 1 for l in lengths]
    row_offsets = [sum(counts[:n]) for n in range(N)]
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    got = run_kernel(device, cases, p, dtype, lengths=lengths, per_token=True, row_offsets=row_offsets, n_rows=sum(counts))
    streamed = kernel_variant == "streamed" and p % 8 == 0
    assert _lib.last_kernel(_lib.FAMILY_COLLECT) == ("collect_persist_table" if streamed else "collect_tile")
    want = oracle_rows(cases, dtype, attribute_tokens=True, collection_mask=mask)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [16, 32, 8])
def test_tok(device, dtype, p):
    N, S = 3, 90
    lengths = [90, 33, 70]
    cases = []
    for i, (I, O) in enumerate([(128, 256), (256, 64)]):
        cases.append(make_case(N, S, I, O, p, dtype, seed=20 + i, normalizer="adafactor" if i else None,
                               name=f"layers.{i}.y"))
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    # documents are stored in a different order than they sit in the batch
    counts = [l - 1 for l in lengths]
    doc_order = [2, 0, 1]
    offs = {}
    r = 0
    for d in doc_order:
        offs[d] = r
        r += counts[d]
    row_offsets = [offs[n] for n in range(N)]
    got = run_kernel(device, cases, p, dtype, lengths=lengths, per_token=True, row_offsets=row_offsets, n_rows=r)
    want_batch_order = oracle_rows(cases, dtype, attribute_tokens=True, collection_mask=mask)
    want = torch.zeros_like(want_batch_order)
    src = 0
    for n in range(N):
        want[row_offsets[n]:row_offsets[n] + counts[n]] = want_batch_order[src:src + counts[n]]
        src += counts[n]
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("p", [16, 8])
def test_two_step_token_rows_equal_the_one_step_rows_bitwise(device, out_dtype, p, bgx_env, kernel_variant):
    """Per-token rows at p = 8 / 16 are written in two steps by default (the collection kernel leaves every token's
    a', g' in the workspace, a second kernel writes the store rows whole); BGX_COLLECT_TWO_STEP_OFF makes the
    collection kernel write them itself.  Same arithmetic, same bits -- on ragged lengths, documents stored out of
    batch order, several tiles per sequence, and a clamp that bites."""
    N, S = 4, 300
    lengths = [300, 2, 131, 257]
    cases = []
    for i, (I, O) in enumerate([(128, 256), (256, 64), (64, 192)]):
        a, g, left, right, norm = make_case(N, S, I, O, p, torch.bfloat16, seed=220 + i,
                                            normalizer="adafactor" if i == 1 else None, name=f"layers.{i}.w")
        cases.append((a, g * (30.0 if i == 2 else 1.0), left, right, norm))
    counts = [l - 1 for l in lengths]
    order = [3, 1, 0, 2]
    offs, r = {}, 0
    for d in order:
        offs[d] = r
        r += counts[d]
    kw = dict(lengths=lengths, per_token=True, row_offsets=[offs[n] for n in range(N)], n_rows=r, lo=-2.0, hi=2.0)
    two = run_kernel(device, cases, p, out_dtype, **kw)
    bgx_env("BGX_COLLECT_TWO_STEP_OFF", "1")
    one = run_kernel(device, cases, p, out_dtype, **kw)
    bgx_env("BGX_COLLECT_TWO_STEP_OFF", None)
    assert torch.equal(two, one)
    assert two.abs().max().item() == 2.0 and (two != 0).any(dim=1).all()   # the clamp bit; every row was written


def test_two_step_token_rows_of_wide_modules_equal_the_one_step_rows_bitwise(device, bgx_env, kernel_variant):
    """The same for modules whose projections do not fit LDS (fragments from the table in global memory, shared by the
    workgroup's waves): several tiles per sequence, ragged lengths, waves without tokens in the last tile."""
    from bergson_amd import _lib

    N, S, p = 3, 330, 16
    lengths = [330, 3, 140]
    cases = []
    for i, (I, O) in enumerate([(4096, 1024), (512, 4608)]):
        a, g, left, right, norm = make_case(N, S, I, O, p, torch.bfloat16, seed=230 + i,
                                            normalizer="adafactor" if i == 0 else None, name=f"layers.{i}.wide")
        cases.append((a, g, left, right, norm))
    counts = [l - 1 for l in lengths]
    kw = dict(lengths=lengths, per_token=True, row_offsets=[sum(counts[:n]) for n in range(N)], n_rows=sum(counts))
    two = run_kernel(device, cases, p, torch.bfloat16, **kw)
    route = _lib.last_kernel(_lib.FAMILY_COLLECT)
    bgx_env("BGX_COLLECT_TWO_STEP_OFF", "1")
    one = run_kernel(device, cases, p, torch.bfloat16, **kw)
    bgx_env("BGX_COLLECT_TWO_STEP_OFF", None)
    assert route == ("collect_persist_table" if kernel_variant == "streamed" else "collect_tile")
    assert torch.equal(two, one)
    assert (two != 0).any(dim=1).all()


def test_tok_rows_sum_to_seq_row(device):
    # sum over tokens of the per-token rows equals the per-sequence row (fp32)
    N, S, p = 2, 77, 16
    lengths = [77, 40]
    a, g, left, right, _ = make_case(N, S, 128, 64, p, torch.float32, seed=30)
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    case = (a, g, left, right, None)
    seq = run_kernel(device, [case], p, torch.float32, lengths=lengths)
    tok = run_kernel(device, [case], p, torch.float32, lengths=lengths, per_token=True, row_offsets=[0, 76], n_rows=76 + 39)
    assert rel_l2(tok[:76].sum(0), seq[0]) <= 1e-5
    assert rel_l2(tok[76:].sum(0), seq[1]) <= 1e-5


def test_noncontiguous_views(device):
    # g arriving as a slice of a wider tensor (fused qkv) keeps its strides
    from bergson_amd import ops

    N, S, I, O, p = 2, 64, 128, 128, 16
    a, g_full, left, right, _ = make_case(N, S, I, 3 * O, p, torch.bfloat16, seed=40)
    left = left[:, :O].contiguous()
    gd = g_full.to(device)[:, :, O:2 * O]
    assert not gd.is_contiguous()
    out = torch.zeros(N, p * p, dtype=torch.bfloat16, device=device)
    ops.collect_seq([ops.ModuleInput(a=a.to(device), g=gd, r_in=right.to(device), r_out=left.to(device), out_col=0)],
                    p, out)
    want = ohooks.module_gradient(a, g_full[:, :, O:2 * O], None, left, right)
    assert rel_l2(out.cpu(), want) <= 1e-2


def test_rejects_cpu_tensors():
    from bergson_amd import ops

    a = torch.zeros(1, 4, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.collect_seq([ops.ModuleInput(a=a, g=a, r_in=torch.zeros(16, 8), r_out=torch.zeros(16, 8), out_col=0)], 16,
                        torch.zeros(1, 256))


# ---- Adam second-moment normaliser -----------------------------------------------------------------------

def _adam_case(N, S, I, O, p, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    left, right = module_projections("layers.1.attention.dense", p, O, I, dtype)
    v = (torch.randn(O, I, generator=gen).abs() * 1e-5) + 1e-9
    return a, g, left, right, ohooks.Adam(weight_avg_sq=v)


def _run_adam(device, case, p, out_dtype, *, per_token=False, lengths=None, row_offsets=None, n_rows=None,
              chunk_tokens=0, out_col=0, width=None):
    from bergson_amd import ops

    a, g, left, right, norm = case
    prep = ops.AdamPrepared(right.to(device), left.to(device), norm.weight_avg_sq.to(device), out_col)
    rows = n_rows if n_rows is not None else a.shape[0]
    out = torch.zeros(rows, width or p * p, dtype=out_dtype, device=device)
    ldev = None if lengths is None else torch.tensor(lengths, dtype=torch.int32, device=device)
    rdev = None if row_offsets is None else torch.tensor(row_offsets, dtype=torch.int64, device=device)
    ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=per_token, lengths=ldev, rows=rdev,
                     lo=torch.finfo(out_dtype).min, hi=torch.finfo(out_dtype).max, chunk_tokens=chunk_tokens)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 40, 64, 96, 16), (3, 70, 128, 64, 32), (1, 33, 96, 40, 8)])
@pytest.mark.parametrize("chunk_tokens", [0, 64])
def test_adam_seq(device, dtype, shape, chunk_tokens):
    """chunk_tokens = 0: the normalisation is applied to the summed gradient (batched GEMM, then the
    collection kernel over output features); 64: the per-token formulation in several internal passes."""
    N, S, I, O, p = shape
    case = _adam_case(N, S, I, O, p, dtype, seed=50)
    got = _run_adam(device, case, p, dtype, chunk_tokens=chunk_tokens)
    a, g, left, right, norm = case
    want = ohooks.module_gradient(a, g, norm, left, right)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[dtype]
    if dtype == torch.float32:
        # and against the closed form L @ (G^T A / (sqrt(v) + 1e-8)) @ R^T in fp64
        full = (g.mT.double() @ a.double()) / (norm.weight_avg_sq.double().sqrt() + 1e-8)
        assert rel_l2(got, (left.double() @ full @ right.double().T).flatten(1)) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_adam_tok(device, dtype):
    N, S, I, O, p = 3, 50, 64, 96, 16
    lengths = [50, 21, 37]
    case = _adam_case(N, S, I, O, p, dtype, seed=51)
    a, g, left, right, norm = case
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    counts = [l - 1 for l in lengths]
    offs = [0, counts[0], counts[0] + counts[1]]
    got = _run_adam(device, case, p, dtype, per_token=True, lengths=lengths, row_offsets=offs, n_rows=sum(counts),
                    chunk_tokens=64, out_col=256, width=768)
    want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
    assert rel_l2(got[:, 256:512], want) <= TOL[dtype]
    assert got[:, :256].abs().sum() == 0 and got[:, 512:].abs().sum() == 0


# ---- bias column -------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("normalizer", [None, "adafactor"])
@pytest.mark.parametrize("per_token", [False, True])
def test_bias_column(device, dtype, normalizer, per_token):
    from bergson_amd import ops

    N, S, I, O, p = 2, 90, 96, 64, 16
    gen = torch.Generator().manual_seed(60)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    lengths = [90, 47]
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    left, right = module_projections("layers.0.mlp.dense_4h_to_h", p, O, I, dtype, collect_bias=True)
    assert right.shape == (p, I + 1)
    norm = None
    rs = cs = bs = None
    if normalizer:
        # second moments in the model dtype, as the reference's arithmetic needs for a bias with a 16-bit model
        row = (torch.rand(O, generator=gen) + 0.1).to(dtype)
        col = (torch.rand(I, generator=gen) + 0.1).to(dtype)
        bsq = (torch.rand(O, generator=gen) + 0.1).to(dtype)
        norm = ohooks.Adafactor(row=row, col=col, bias_avg_sq=bsq)
        rs, cs = ops.adafactor_scales(row.to(device), col.to(device), dtype)
        bs = (bsq.to(device).float() + 1e-8).rsqrt().contiguous()
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    want = ohooks.module_gradient(a, g, norm, left, right, collect_bias=True, attribute_tokens=per_token,
                                  collection_mask=mask if per_token else None)
    mi = ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right[:, :I].contiguous().to(device),
                         r_out=left.to(device), out_col=0, col_scale=cs, row_scale=rs,
                         bias_col=right[:, I].float().contiguous().to(device), bias_scale=bs)
    if per_token:
        out = torch.zeros(sum(l - 1 for l in lengths), p * p, dtype=dtype, device=device)
        ops.collect_tok([mi], p, out, lengths=torch.tensor(lengths, dtype=torch.int32, device=device),
                        row_offsets=torch.tensor([0, lengths[0] - 1], dtype=torch.int64, device=device))
    else:
        out = torch.zeros(N, p * p, dtype=dtype, device=device)
        ops.collect_seq([mi], p, out)
    torch.cuda.synchronize()
    assert out.shape == want.shape
    assert rel_l2(out.cpu(), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("wide", [False, True])
def test_bias_column_without_a_factor_on_the_streamed_kernels(device, dtype, per_token, wide, kernel_variant):
    """A bias column with no factor of its own (no normalizer, or none on the bias) is a constant added to every
    token's projected activation, which the streamed kernels do in registers; the launch mixes a module with the column
    and one without, ragged lengths, and (wide) a module whose projections come from the table in global memory."""
    from bergson_amd import _lib, ops

    N, S, p = 3, 200, 16
    lengths = [200, 77, 2]
    shapes = [(128, 192, True), (64, 64, False)]
    if wide:
        shapes.append((4096 if dtype == torch.bfloat16 else 2048, 1024, True))
    gen = torch.Generator().manual_seed(61)
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    mods, wants, col = [], [], 0
    for i, (I, O, bias) in enumerate(shapes):
        a = torch.randn(N, S, I, generator=gen).to(dtype)
        g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        left, right = module_projections(f"layers.{i}.b", p, O, I, dtype, collect_bias=bias)
        wants.append(ohooks.module_gradient(a, g, None, left, right, collect_bias=bias, attribute_tokens=per_token,
                                            collection_mask=mask if per_token else None))
        mods.append(ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right[:, :I].contiguous().to(device),
                                    r_out=left.to(device), out_col=col,
                                    bias_col=right[:, I].float().contiguous().to(device) if bias else None))
        col += p * p
    want = torch.cat(wants, dim=1)
    ldev = torch.tensor(lengths, dtype=torch.int32, device=device)
    if per_token:
        counts = [l - 1 for l in lengths]
        out = torch.zeros(sum(counts), col, dtype=dtype, device=device)
        ops.collect_tok(mods, p, out, lengths=ldev,
                        row_offsets=torch.tensor([sum(counts[:n]) for n in range(N)], dtype=torch.int64, device=device))
    else:
        out = torch.zeros(N, col, dtype=dtype, device=device)
        ops.collect_seq(mods, p, out, lengths=ldev)
    torch.cuda.synchronize()
    route = _lib.last_kernel(_lib.FAMILY_COLLECT)
    assert route == {"streamed": "collect_persist_table" if wide else "collect_persist_lds"}.get(kernel_variant, "collect_tile")
    assert out.shape == want.shape
    assert rel_l2(out.cpu(), want) <= TOL[dtype]


@pytest.mark.parametrize("per_token", [False, True])
def test_adam_with_bias(device, per_token):
    from bergson_amd import ops

    N, S, I, O, p = 2, 40, 64, 48, 16
    lengths = [40, 19]
    gen = torch.Generator().manual_seed(70)
    a = torch.randn(N, S, I, generator=gen)
    g = torch.randn(N, S, O, generator=gen) * 0.1
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    left, right = module_projections("layers.2.attention.dense", p, O, I, torch.float32, collect_bias=True)
    norm = ohooks.Adam(weight_avg_sq=torch.rand(O, I, generator=gen) * 1e-4 + 1e-8,
                       bias_avg_sq=torch.rand(O, generator=gen) * 1e-4 + 1e-8)
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    want = ohooks.module_gradient(a, g, norm, left, right, collect_bias=True, attribute_tokens=per_token,
                                  collection_mask=mask if per_token else None)
    prep = ops.AdamPrepared(right[:, :I].contiguous().to(device), left.to(device), norm.weight_avg_sq.to(device), 0,
                            bias_col=right[:, I].to(device), bias_avg_sq=norm.bias_avg_sq.to(device))
    ldev = torch.tensor(lengths, dtype=torch.int32, device=device)
    if per_token:
        out = torch.zeros(sum(l - 1 for l in lengths), p * p, device=device)
        ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=True, lengths=ldev,
                         rows=torch.tensor([0, lengths[0] - 1], dtype=torch.int64, device=device), lo=-3e38, hi=3e38)
    else:
        out = torch.zeros(N, p * p, device=device)
        ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=False, lengths=None, rows=None, lo=-3e38,
                         hi=3e38)
    torch.cuda.synchronize()
    assert rel_l2(out.cpu(), want) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("shape", [(2, 300, 128, 320, 32), (1, 512, 256, 1000, 32), (2, 70, 200, 256, 16),
                                   (3, 40, 96, 40, 8), (1, 256, 1024, 768, 32)])
def test_adam_fused_kernels_take_any_width_and_the_bias(device, dtype, bias, per_token, shape):
    """16-bit models with p <= 32 stay on the fused per-token kernels whatever the module's widths: O that is no
    multiple of 256 (320, 1000, 40), I that is no multiple of 64 (200, 96), and the bias column, which travels as one
    more input feature.  Rows against the oracle, and the route asserted from what the library ran."""
    from bergson_amd import _lib, ops

    N, S, I, O, p = shape
    gen = torch.Generator().manual_seed(300 + O + I)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    lengths = [S, max(2, S // 3), max(2, S - 9)][:N]
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    left, right = module_projections("layers.4.mlp.dense_h_to_4h", p, O, I, dtype, collect_bias=bias)
    # second moments bounded away from zero keep R / sqrt(v) inside fp16's range; in the model dtype where the
    # bias is collected, as the reference's arithmetic needs there
    v = torch.rand(O, I, generator=gen) * 1e-3 + 1e-4
    bsq = (torch.rand(O, generator=gen) * 1e-3 + 1e-4) if bias else None
    norm = ohooks.Adam(weight_avg_sq=v.to(dtype) if bias else v, bias_avg_sq=None if bsq is None else bsq.to(dtype))
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    want = ohooks.module_gradient(a, g, norm, left, right, collect_bias=bias, attribute_tokens=per_token,
                                  collection_mask=mask if per_token else None).float()
    r_in = right[:, :I].contiguous() if bias else right
    prep = ops.AdamPrepared(r_in.to(device), left.to(device), norm.weight_avg_sq.float().to(device), 0,
                            bias_col=right[:, I].to(device) if bias else None,
                            bias_avg_sq=norm.bias_avg_sq.float().to(device) if bias else None)
    ldev = torch.tensor(lengths, dtype=torch.int32, device=device)
    counts = [l - 1 for l in lengths]
    if per_token:
        out = torch.zeros(sum(counts), p * p, dtype=torch.float32, device=device)
        offs = torch.tensor([sum(counts[:n]) for n in range(N)], dtype=torch.int64, device=device)
        ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=True, lengths=ldev, rows=offs, lo=-3e38,
                         hi=3e38)
        torch.cuda.synchronize()
        assert _lib.last_kernel(_lib.FAMILY_ADAM).startswith("adam_fused")
    else:
        out = torch.zeros(N, p * p, dtype=torch.float32, device=device)
        ops.collect_adam(prep, a.to(device), g.to(device), out, per_token=False, lengths=ldev, rows=None, lo=-3e38,
                         hi=3e38)
        torch.cuda.synchronize()
    assert out.shape == want.shape and torch.isfinite(out).all()
    assert rel_l2(out.cpu(), want) <= TOL[dtype]
    if per_token and S * N <= 600:   # every row on its own, so that a wrong padded column cannot hide in the norm
        live = want.norm(dim=1) > 1e-3 * want.norm(dim=1).max()
        per_row = (out.cpu() - want).norm(dim=1) / want.norm(dim=1).clamp_min(1e-30)
        assert per_row[live].max().item() <= 4 * TOL[dtype]


# ---- weight-shaped (unprojected) gradients ----------------------------------------------------------
def _full_case(N, S, I, O, dtype, kind, bias, seed):
    gen = torch.Generator().manual_seed(seed)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    norm = None
    if kind == "adafactor":
        norm = ohooks.Adafactor(torch.rand(O, generator=gen) + 0.1, torch.rand(I, generator=gen) + 0.1,
                                torch.rand(O, generator=gen) + 0.1 if bias else None)
    elif kind == "adam":
        norm = ohooks.Adam(torch.rand(O, I, generator=gen) + 0.1, torch.rand(O, generator=gen) + 0.1 if bias else None)
    return a, g, norm


def _full_module(device, a, g, norm, bias, out_col):
    from bergson_amd import ops

    O, I = g.shape[2], a.shape[2]
    mod = ops.FullGradModule(O=O, I=I, out_col=out_col, collect_bias=bias)
    if isinstance(norm, ohooks.Adafactor):
        mod.row_scale, mod.col_scale = ops.adafactor_scales(norm.row.to(device), norm.col.to(device), a.dtype)
        if bias:
            mod.bias_scale = norm.bias_avg_sq.to(device).add(1e-8).rsqrt()
    elif isinstance(norm, ohooks.Adam):
        mod.adam_v = norm.weight_avg_sq.to(device).contiguous()
        if bias:
            mod.bias_scale = (norm.bias_avg_sq.to(device).sqrt() + 1e-8).reciprocal()
    return mod


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", [None, "adafactor", "adam"])
@pytest.mark.parametrize("bias", [False, True])
def test_fullgrad_seq(device, dtype, kind, bias):
    from bergson_amd import ops

    N, S, I, O = 3, 37, 24, 40
    a, g, norm = _full_case(N, S, I, O, dtype, kind, bias, seed=60)
    lo, hi = torch.finfo(dtype).min, torch.finfo(dtype).max
    want = ohooks.module_gradient(a, g, norm, None, None, collect_bias=bias, lo=lo, hi=hi)
    width = O * (I + int(bias))
    out = torch.zeros(5, 7 + width, dtype=dtype, device=device)
    rows = torch.tensor([4, 0, 2], dtype=torch.int64, device=device)
    ops.full_gradient(_full_module(device, a, g, norm, bias, 7), a.to(device), g.to(device), out, per_token=False,
                      lengths=None, rows=rows, lo=lo, hi=hi)
    torch.cuda.synchronize()
    got = out.cpu()
    assert rel_l2(got[[4, 0, 2], 7:], want) <= TOL[dtype]
    assert got[:, :7].abs().sum() == 0 and got[[1, 3]].abs().sum() == 0


def _wgrad_reference(a, g, lengths):
    """sum_s g[n, s, :] (x) a[n, s, :] over the tokens s < lengths[n] - 1, in float64."""
    a64, g64 = a.double(), g.double().clone()
    if lengths is not None:
        for n, l in enumerate(lengths):
            g64[n, max(l - 1, 0):] = 0
    return torch.einsum("nso,nsi->noi", g64, a64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [
    (3, 37, 24, 40),       # one ragged 64-wide tile, tokens not a multiple of a stage
    (2, 130, 200, 136),    # several 64-wide tiles with ragged edges
    (3, 96, 1024, 1024),   # whole 64-wide tiles, many of them
    (16, 520, 1024, 1024), # 128-wide tiles (long sequences, 64 tiles x 16 sequences: two rounds of the chip)
    (29, 530, 700, 650),   # 128-wide tiles with ragged edges and rows that are not whole 16-byte pieces
    (1, 70, 70, 61),       # odd widths: pieces of 16 bytes cannot be loaded whole
    (4, 1, 64, 64),        # a single token
])
def test_fullgrad_seq_gemm_against_float64(device, dtype, shape):
    """The fused GEMM-over-tokens kernel alone (no normaliser): every tile variant and edge against the float64
    contraction, with lengths that cut sequences short (one of them to nothing) and scattered output rows."""
    from bergson_amd import ops

    N, S, I, O = shape
    gen = torch.Generator().manual_seed(91)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    lengths = [[S + 1, max(1, S // 2), 1, S][n % 4] for n in range(N)]
    want = _wgrad_reference(a, g, lengths).reshape(N, O * I)
    out = torch.full((N + 1, 3 + O * I), 7.0, dtype=torch.float32, device=device)
    rows = torch.tensor(list(range(N, 0, -1)), dtype=torch.int64, device=device)
    mod = ops.FullGradModule(O=O, I=I, out_col=3)
    ops.full_gradient(mod, a.to(device), g.to(device), out, per_token=False,
                      lengths=torch.tensor(lengths, dtype=torch.int32, device=device), rows=rows, lo=-3e38, hi=3e38)
    torch.cuda.synchronize()
    got = out.cpu()
    assert bool((got[0] == 7).all()) and bool((got[:, :3] == 7).all())
    assert rel_l2(got[list(range(N, 0, -1)), 3:].double(), want) <= TOL[dtype]
    if N >= 3:
        assert got[N - 2, 3:].abs().sum() == 0  # the sequence of length 1 has no labelled token


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind,bias", [(None, False), ("adam", True), ("adafactor", True)])
def test_fullgrad_seq_gemm_128_tiles_equal_64_tiles_bitwise(device, dtype, kind, bias, monkeypatch):
    """Modules with enough 128 x 128 tiles to go round take them (wgrad_seq_128); every element is the same
    sequence of MFMAs over the tokens as on 64 x 64 tiles, the normalisation behind it is the same code: identical
    bits, ragged edges and short sequences included.  (The bias column is a plain sum over the tokens, added up by
    four threads per feature on the small tiles and two on the large ones: equal to rounding.)"""
    from bergson_amd import _lib, ops

    N, S, I, O = 52, 600, 520, 392
    a, g, norm = _full_case(N, S, I, O, dtype, kind, bias, seed=97)
    mod = _full_module(device, a, g, norm, bias, 5)
    a, g = a.to(device), g.to(device)
    lengths = torch.tensor([S + 1, 77, 1, S, 2, 65, 64, 130, 17, S, S, 533, 100] * 4, dtype=torch.int32, device=device)
    lo, hi = torch.finfo(dtype).min, torch.finfo(dtype).max
    outs = {}
    for tiles in ("wgrad_seq_128", "wgrad_seq_64"):
        if tiles == "wgrad_seq_64":
            monkeypatch.setenv("BGX_WGRAD_BIG_OFF", "1")
            _lib.reload_switches()
        out = torch.zeros(N, 5 + mod.width, dtype=dtype, device=device)
        ops.full_gradient(mod, a, g, out, per_token=False, lengths=lengths, rows=None, lo=lo, hi=hi)
        torch.cuda.synchronize()
        assert _lib.last_kernel(_lib.FAMILY_FULLGRAD) == tiles
        outs[tiles] = out
    monkeypatch.delenv("BGX_WGRAD_BIG_OFF")
    _lib.reload_switches()
    Iw = I + int(bias)
    big, small = (outs[t][:, 5:].reshape(N, O, Iw) for t in ("wgrad_seq_128", "wgrad_seq_64"))
    assert torch.equal(big[:, :, :I], small[:, :, :I]) and torch.equal(outs["wgrad_seq_128"][:, :5], outs["wgrad_seq_64"][:, :5])
    if bias:
        assert rel_l2(big[:, :, I].float().cpu(), small[:, :, I].float().cpu()) <= 1e-6 + TOL[dtype] / 10
    assert big[0].abs().sum() > 0 and big[2].abs().sum() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fullgrad_seq_gemm_strided_operands(device, dtype):
    """Operands that are views: token rows wider than the features used, sequences far apart, and a g whose first
    element is not 16-byte aligned (the element-wise loader)."""
    from bergson_amd import ops

    N, S, I, O = 2, 45, 72, 88
    gen = torch.Generator().manual_seed(92)
    a_big = torch.randn(N, S + 3, I + 24, generator=gen).to(dtype).to(device)
    g_big = (torch.randn(N, S, O + 9, generator=gen) * 0.1).to(dtype).to(device)
    a = a_big[:, 1:S + 1, 8:8 + I]
    g = g_big[:, :, 3:3 + O]
    want = _wgrad_reference(a.cpu(), g.cpu(), None).reshape(N, O * I)
    out = torch.zeros(N, O * I, dtype=torch.float32, device=device)
    ops.full_gradient(ops.FullGradModule(O=O, I=I, out_col=0), a, g, out, per_token=False, lengths=None, rows=None,
                      lo=-3e38, hi=3e38)
    torch.cuda.synchronize()
    assert rel_l2(out.cpu().double(), want) <= TOL[dtype]


@pytest.mark.parametrize("kind", [None, "adafactor", "adam"])
def test_fullgrad_two_step_entries_agree_with_fused(device, kind):
    """bgx_token_sum + bgx_fullgrad_seq behind a caller's own GEMM (the entries a C caller with its own BLAS uses)
    give the rows of the fused entry: same rounding points, sums in another order."""
    from bergson_amd import _lib, ops
    from bergson_amd.ops import _ptr, _stream, dtype_code

    N, S, I, O = 3, 64, 96, 80
    dtype = torch.bfloat16
    a, g, norm = _full_case(N, S, I, O, dtype, kind, True, seed=93)
    mod = _full_module(device, a, g, norm, True, 0)
    a, g = a.to(device), g.to(device)
    fused = torch.zeros(N, mod.width, dtype=dtype, device=device)
    ops.full_gradient(mod, a, g, fused, per_token=False, lengths=None, rows=None, lo=-3e38, hi=3e38)
    lib = _lib.load()
    P = torch.einsum("nso,nsi->noi", g.float(), a.float()).to(dtype).contiguous()
    bias_sum = torch.empty(N, O, dtype=torch.float32, device=device)
    code = dtype_code(dtype)
    _lib.check(lib.bgx_token_sum(_ptr(g), g.stride(0), g.stride(1), N, S, O, code, _ptr(bias_sum), _stream()), "sum")
    two = torch.zeros_like(fused)
    _lib.check(lib.bgx_fullgrad_seq(_ptr(P), N, O, I, code, _ptr(mod.row_scale), _ptr(mod.col_scale),
                                    _ptr(mod.adam_v), _ptr(bias_sum), _ptr(mod.bias_scale), None, _ptr(two),
                                    two.stride(0), 0, code, -3e38, 3e38, _stream()), "fullgrad_seq")
    torch.cuda.synchronize()
    assert rel_l2(fused.cpu(), two.cpu()) <= 4e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(3, 40 * 24, 16), (70, 5000, 40), (2, 393216, 32), (33, 1001, 100), (1, 7, 1)])
def test_project_rows_against_float64(device, dtype, shape):
    """The global projection's contraction (rows [M, W] times a [P, W] block, added to an fp32 accumulator):
    few and many rows, widths that are no multiple of a k-step (and of nothing: the element-wise loader), more
    columns than one workgroup takes, a second call adding to the first, and the same bits on a repeat."""
    from bergson_amd import ops

    M, W, P = shape
    gen = torch.Generator().manual_seed(95)
    rows = (torch.randn(M, W, generator=gen) * 0.1).to(dtype)
    proj = (torch.randn(P, W, generator=gen) / W ** 0.5).to(dtype)
    want = rows.double() @ proj.double().T
    acc = torch.zeros(M, P, dtype=torch.float32, device=device)
    ops.project_rows(rows.to(device), proj.to(device), acc)
    torch.cuda.synchronize()
    first = acc.clone()
    assert rel_l2(first.cpu().double(), want) <= (1e-5 if dtype == torch.float32 else 1e-4)  # exact products, fp32 sums
    ops.project_rows(rows.to(device), proj.to(device), acc)
    again = torch.zeros_like(first)
    ops.project_rows(rows.to(device), proj.to(device), again)
    torch.cuda.synchronize()
    assert torch.equal(again, first)
    assert rel_l2(acc.cpu().double(), 2 * want) <= (1e-5 if dtype == torch.float32 else 1e-4)


def test_project_rows_strided_rows(device):
    """Rows that are a column slice of a wider buffer (row stride above the width, first element off a 16-byte
    boundary)."""
    from bergson_amd import ops

    gen = torch.Generator().manual_seed(96)
    big = (torch.randn(9, 700, generator=gen) * 0.1).to(torch.bfloat16).to(device)
    rows = big[:, 3:3 + 640]
    proj = (torch.randn(24, 640, generator=gen) / 25).to(torch.bfloat16).to(device)
    acc = torch.zeros(9, 24, dtype=torch.float32, device=device)
    ops.project_rows(rows, proj, acc)
    torch.cuda.synchronize()
    assert rel_l2(acc.cpu().double(), rows.cpu().double() @ proj.cpu().double().T) <= 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", [None, "adafactor", "adam"])
@pytest.mark.parametrize("bias", [False, True])
def test_fullgrad_tok(device, dtype, kind, bias):
    from bergson_amd import ops

    N, S, I, O = 3, 21, 24, 20
    lengths = [21, 2, 10]
    a, g, norm = _full_case(N, S, I, O, dtype, kind, bias, seed=61)
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    lo, hi = torch.finfo(dtype).min, torch.finfo(dtype).max
    want = ohooks.module_gradient(a, g, norm, None, None, collect_bias=bias, attribute_tokens=True,
                                  collection_mask=mask, lo=lo, hi=hi)
    counts = [l - 1 for l in lengths]
    offs = [sum(counts[:n]) for n in range(N)]
    out = torch.zeros(sum(counts), O * (I + int(bias)), dtype=dtype, device=device)
    ops.full_gradient(_full_module(device, a, g, norm, bias, 0), a.to(device), g.to(device), out, per_token=True,
                      lengths=torch.tensor(lengths, dtype=torch.int32, device=device),
                      rows=torch.tensor(offs, dtype=torch.int64, device=device), lo=lo, hi=hi)
    torch.cuda.synchronize()
    assert rel_l2(out.cpu(), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("shape", [(3, 150, 192, 256, 16), (4, 70, 200, 330, 32), (2, 130, 77, 61, 7),
                                   (5, 64, 64, 64, 32), (2, 300, 1024, 520, 16),
                                   (16, 520, 1024, 1024, 32), (29, 530, 700, 650, 16)])  # the last two: 128 x 128 tiles
def test_adam_seq_projected_in_the_tile_kernel(device, dtype, bias, shape):
    """Per-sequence Adam on 16-bit models: the weight-shaped gradient is formed tile by tile and projected where
    it is (bgx_collect_seq_weight).  Against the oracle's op sequence, and against the route through memory
    (bgx_fullgrad_seq_gemm + bgx_collect_seq: the same rounding of the normalised gradient, the projections summed
    in another order); ragged tiles, odd widths, short and empty sequences, scattered rows, the bias column."""
    from bergson_amd import _lib, ops

    N, S, I, O, p = shape
    gen = torch.Generator().manual_seed(77)
    a = torch.randn(N, S, I, generator=gen).to(dtype)
    g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
    lengths = [[S + 1, max(2, S // 3), 1, S, 2][n % 5] for n in range(N)]
    gz = g.clone()
    for n, l in enumerate(lengths):
        gz[n, max(l - 1, 0):] = 0
    left, right = module_projections("layers.1.mlp.dense_h_to_4h", p, O, I, dtype, collect_bias=bias)
    # second moments bounded away from zero keep the normalised gradient inside fp16's range; in the model dtype
    # where the bias is collected, as the reference's arithmetic needs there
    v = torch.rand(O, I, generator=gen) * 1e-3 + 1e-4
    bsq = (torch.rand(O, generator=gen) * 1e-3 + 1e-4) if bias else None
    norm = ohooks.Adam(weight_avg_sq=v.to(dtype) if bias else v, bias_avg_sq=None if bsq is None else bsq.to(dtype))
    want = ohooks.module_gradient(a, gz, norm, left, right, collect_bias=bias)
    kw = dict(bias_col=right[:, I].to(device), bias_avg_sq=norm.bias_avg_sq.float().to(device)) if bias else {}
    prep = ops.AdamPrepared(right[:, :I].contiguous().to(device), left.to(device),
                            norm.weight_avg_sq.float().to(device), 3, **kw)
    ldev = torch.tensor(lengths, dtype=torch.int32, device=device)
    rows = torch.tensor(list(range(N, 0, -1)), dtype=torch.int64, device=device)
    lo, hi = torch.finfo(dtype).min, torch.finfo(dtype).max
    outs = []
    for through_memory in (False, True):
        out = torch.full((N + 1, 3 + p * p + 2), 5.0, dtype=dtype, device=device)
        ops._collect_adam_seq(prep, a.to(device), g.to(device), out, ldev, rows, lo, hi, through_memory=through_memory)
        torch.cuda.synchronize()
        if not through_memory:
            big = -(-O // 128) * -(-I // 128) * N >= 1024 and S >= 512
            assert _lib.last_kernel(_lib.FAMILY_FULLGRAD) == ("wgrad_seq_projected_128" if big else "wgrad_seq_projected_64")
        outs.append(out.cpu())
    got = outs[0]
    assert bool((got[0] == 5).all()) and bool((got[:, :3] == 5).all()) and bool((got[:, 3 + p * p:] == 5).all())
    block = got[list(range(N, 0, -1)), 3:3 + p * p].float()
    assert rel_l2(block, want.float()) <= TOL[dtype]
    assert rel_l2(block, outs[1][list(range(N, 0, -1)), 3:3 + p * p].float()) <= TOL[dtype] / 2
    if N >= 3:
        assert block[2].abs().sum() == 0  # the sequence of length 1 has no labelled token


def test_adam_seq_with_lengths_and_rows(device):
    """Per-sequence Adam with positions past each document's last label skipped and rows scattered."""
    N, S, I, O, p = 3, 48, 64, 96, 16
    lengths = [48, 20, 33]
    case = _adam_case(N, S, I, O, p, torch.float32, seed=52)
    a, g, left, right, norm = case
    gz = g.clone()
    for n, l in enumerate(lengths):
        gz[n, l - 1:] = 0
    want = ohooks.module_gradient(a, gz, norm, left, right)
    # g itself is NOT zeroed: the lengths must do it
    got = _run_adam(device, case, p, torch.float32, lengths=lengths, row_offsets=[2, 0, 1], n_rows=4)
    assert rel_l2(got[[2, 0, 1]], want) <= 1e-5
    assert got[3].abs().sum() == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("p", [16, 32])
@pytest.mark.parametrize("per_token", [False, True])
def test_adam_fused_path(device, dtype, p, per_token, bgx_env):
    """Shapes the fused Adam kernel takes (16-bit, O % 256 == 0, I % 64 == 0, p <= 32): several token tiles,
    two chunks of output features, ragged lengths; against the oracle and against the two-kernel path."""
    N, S, I, O = 3, 200, 128, 512
    lengths = [200, 77, 130]
    case = _adam_case(N, S, I, O, p, dtype, seed=53)
    a, g, left, right, norm = case
    g = g.clone()
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    case = (a, g, left, right, norm)
    if per_token:
        mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        counts = [l - 1 for l in lengths]
        offs = [sum(counts[:n]) for n in range(N)]
        want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
        kw = dict(per_token=True, lengths=lengths, row_offsets=offs, n_rows=sum(counts))
    else:
        want = ohooks.module_gradient(a, g, norm, left, right)
        kw = dict(chunk_tokens=256)  # the per-token formulation, summed per sequence
    got = _run_adam(device, case, p, dtype, **kw)
    assert rel_l2(got, want) <= TOL[dtype]
    bgx_env("BGX_ADAM_FUSED_OFF", "1")
    other = _run_adam(device, case, p, dtype, **kw)
    assert rel_l2(got, other) <= TOL[dtype]


@pytest.mark.parametrize("ttx", [None, 2, 8])
def test_adam_fused_xcd_order(device, ttx, bgx_env):
    """A grid of 256 workgroups (8 token tiles x 32 columns): the fused kernel then deals (token tile, column)
    pairs to the workgroups so that those sharing an XCD share operands.  Every pair must still be taken exactly
    once: the rows equal those of the plain order bit for bit, and the oracle's within tolerance."""
    N, S, I, O, p = 2, 1024, 64, 256, 32
    case = _adam_case(N, S, I, O, p, torch.bfloat16, seed=61)
    a, g, left, right, norm = case
    lengths = [1024, 700]
    g = g.clone()
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    case = (a, g, left, right, norm)
    counts = [l - 1 for l in lengths]
    offs = [0, counts[0]]
    kw = dict(per_token=True, lengths=lengths, row_offsets=offs, n_rows=sum(counts))
    if ttx is not None:
        bgx_env("BGX_ADAM_TTX", str(ttx))
    got = _run_adam(device, case, p, torch.bfloat16, **kw)
    bgx_env("BGX_ADAM_TTX", "0")
    plain = _run_adam(device, case, p, torch.bfloat16, **kw)
    assert torch.equal(got, plain)
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
    assert rel_l2(got, want) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 256, 256, 256, 32), (2, 512, 320, 512, 32), (1, 768, 1024, 768, 16),
                                   (3, 256, 512, 1024, 8), (1, 256, 1024, 4096, 32), (1, 512, 4096, 1024, 32)])
def test_adam_wide_tiles_equal_the_eight_wave_kernel_bitwise(device, dtype, shape, bgx_env):
    """Whole 256-token tiles with I >= 256 run on four waves per workgroup (one per SIMD, 128 x 128 per wave); the
    sums are formed in the same order as on eight waves, so the rows are the same bits.  Shapes: the smallest the
    kernel takes (four K tiles, one chunk), a K count that is not a power of two, several chunks, p below 32,
    ragged lengths, the widest modules of a Pythia-410m layer; and against the oracle where that is quick."""
    N, S, I, O, p = shape
    case = _adam_case(N, S, I, O, p, dtype, seed=97)
    a, g, left, right, norm = case
    norm = ohooks.Adam(weight_avg_sq=norm.weight_avg_sq * 100 + 1e-6)
    lengths = [S, max(2, S // 3), max(2, S - 41)][:N]
    g = g.clone()
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    case = (a, g, left, right, norm)
    counts = [l - 1 for l in lengths]
    offs = [sum(counts[:n]) for n in range(N)]
    kw = dict(per_token=True, lengths=lengths, row_offsets=offs, n_rows=sum(counts))
    got = _run_adam(device, case, p, dtype, **kw)
    bgx_env("BGX_ADAM_WIDE_OFF", "1")
    eight = _run_adam(device, case, p, dtype, **kw)
    assert torch.equal(got, eight)
    assert bool(torch.isfinite(got.float()).all())
    if I * O * N * S <= 256 * 256 * 512:
        mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
        assert rel_l2(got, want) <= TOL[dtype]
    # per-sequence rows are sums of the same per-token results
    seq = _run_adam(device, case, p, dtype)
    bgx_env("BGX_ADAM_WIDE_OFF", None)
    assert torch.equal(_run_adam(device, case, p, dtype), seq)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 700, 256, 512, 32), (1, 1024, 1024, 1024, 32), (3, 300, 192, 768, 16)])
def test_adam_direct_tiles_against_oracle_and_two_kernel_path(device, dtype, shape, bgx_env):
    """The eight-wave fused Adam kernel (partial token tiles, or fewer than four K tiles) on shapes with several K
    tiles, several chunks of output features and ragged lengths: per-token rows against the oracle on a sample of
    each sequence's tokens (rows do not depend on each other), and every row against the path that materialises H
    (BGX_ADAM_FUSED_OFF), an independent implementation of the same sums."""
    from bergson_amd import _lib

    N, S, I, O, p = shape
    case = _adam_case(N, S, I, O, p, dtype, seed=83)
    a, g, left, right, norm = case
    # second moments bounded away from zero: the table entries R / sqrt(v) stay inside fp16's range
    norm = ohooks.Adam(weight_avg_sq=norm.weight_avg_sq * 100 + 1e-6)
    lengths = [S, max(2, S // 3), max(2, S - 41)][:N]
    g = g.clone()
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    case = (a, g, left, right, norm)
    counts = [l - 1 for l in lengths]
    offs = [sum(counts[:n]) for n in range(N)]
    kw = dict(per_token=True, lengths=lengths, row_offsets=offs, n_rows=sum(counts))
    got = _run_adam(device, case, p, dtype, **kw)
    assert _lib.last_kernel(_lib.FAMILY_ADAM) in ("adam_fused_direct", "adam_fused_wide")
    bgx_env("BGX_ADAM_FUSED_OFF", "1")
    two = _run_adam(device, case, p, dtype, **kw)
    assert _lib.last_kernel(_lib.FAMILY_ADAM) == "adam_two_kernel"
    assert rel_l2(got, two) <= TOL[dtype]
    assert bool(torch.isfinite(got.float()).all())
    gen = torch.Generator().manual_seed(1)
    for n in range(N):
        last = counts[n] - 1
        idx = sorted({0, last, last // 2, min(255, last), min(256, last)} | set(torch.randint(0, last + 1, (6,), generator=gen).tolist()))
        ones = torch.ones(1, len(idx), dtype=torch.bool)
        want = ohooks.module_gradient(a[n:n + 1, idx], g[n:n + 1, idx], norm, left, right, attribute_tokens=True,
                                      collection_mask=ones)
        assert rel_l2(got[torch.tensor(idx) + offs[n]], want) <= TOL[dtype], n


@pytest.mark.parametrize("view", ["g_slice_of_qkv", "a_offset_by_one", "g_sequences_apart"])
def test_adam_fused_kernels_take_odd_views(device, view):
    """Operands the fused kernels cannot load in 16-byte pieces from uniformly strided rows -- g as a slice of a
    wider tensor at an odd offset, a starting one element into its storage, sequences of g that lie apart -- are
    brought into shape by the call itself and stay on the fused kernels."""
    from bergson_amd import _lib, ops

    N, S, I, O, p = 2, 256, 128, 256, 16
    a, g, left, right, norm = _adam_case(N, S, I, O, p, torch.bfloat16, seed=91)
    norm = ohooks.Adam(weight_avg_sq=norm.weight_avg_sq * 100 + 1e-6)
    lengths = [256, 100]
    for n, l in enumerate(lengths):
        g[n, l - 1:] = 0
    ad, gd = a.to(device), g.to(device)
    if view == "g_slice_of_qkv":
        wide = torch.zeros(N, S, 3 * O + 3, dtype=torch.bfloat16, device=device)
        wide[:, :, O + 3:2 * O + 3] = gd
        gd = wide[:, :, O + 3:2 * O + 3]
    elif view == "a_offset_by_one":
        flat = torch.zeros(N * S * I + 1, dtype=torch.bfloat16, device=device)
        flat[1:] = ad.flatten()
        ad = flat[1:].view(N, S, I)
    else:
        apart = torch.zeros(N, S + 5, O, dtype=torch.bfloat16, device=device)
        apart[:, :S] = gd
        gd = apart[:, :S]
    prep = ops.AdamPrepared(right.to(device), left.to(device), norm.weight_avg_sq.to(device), 0)
    counts = [l - 1 for l in lengths]
    out = torch.zeros(sum(counts), p * p, dtype=torch.float32, device=device)
    ops.collect_adam(prep, ad, gd, out, per_token=True, lengths=torch.tensor(lengths, dtype=torch.int32, device=device),
                     rows=torch.tensor([0, counts[0]], dtype=torch.int64, device=device), lo=-3e38, hi=3e38)
    torch.cuda.synchronize()
    assert _lib.last_kernel(_lib.FAMILY_ADAM).startswith("adam_fused")
    mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
    want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
    assert rel_l2(out.cpu(), want) <= TOL[torch.bfloat16]


def test_adam_seq_many_short_sequences(device):
    """Many short sequences of a fused-eligible shape: the per-sequence rows come from the per-token kernel."""
    N, S, I, O, p = 40, 24, 128, 256, 16
    case = _adam_case(N, S, I, O, p, torch.bfloat16, seed=54)
    a, g, left, right, norm = case
    got = _run_adam(device, case, p, torch.bfloat16)
    assert rel_l2(got, ohooks.module_gradient(a, g, norm, left, right)) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("shape", [(1, 4, 768, 768, 16), (1, 2, 64, 256, 32), (2, 3, 128, 512, 8)])
def test_adam_fused_shapes_with_fewer_tokens_than_a_tile(device, per_token, shape):
    """A batch of a few tokens on a shape the fused Adam kernel takes: one pass of T tokens (a chunk size
    rounded down to whole 256-token tiles would be zero here)."""
    N, S, I, O, p = shape
    case = _adam_case(N, S, I, O, p, torch.bfloat16, seed=70)
    a, g, left, right, norm = case
    lengths = [S] * N
    g = g.clone()
    g[:, S - 1:] = 0
    case = (a, g, left, right, norm)
    if per_token:
        mask = (torch.arange(S).unsqueeze(0) + 1) < torch.tensor(lengths).unsqueeze(1)
        offs = [n * (S - 1) for n in range(N)]
        want = ohooks.module_gradient(a, g, norm, left, right, attribute_tokens=True, collection_mask=mask)
        got = _run_adam(device, case, p, torch.bfloat16, per_token=True, lengths=lengths, row_offsets=offs,
                        n_rows=N * (S - 1))
    else:
        want = ohooks.module_gradient(a, g, norm, left, right)
        got = _run_adam(device, case, p, torch.bfloat16)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= TOL[torch.bfloat16]


def test_adam_tables_stay_within_their_budget(device, monkeypatch):
    """The per-module Adam tables (p times the weight bytes each) are dropped least recently used first once
    together they exceed the budget, and rebuilt on demand with the same contents."""
    from bergson_amd import ops

    gen = torch.Generator().manual_seed(3)
    p, I, O = 16, 64, 256
    preps = []
    for k in range(3):
        left, right = module_projections(f"layers.{k}.mlp.dense_h_to_4h", p, O, I, torch.bfloat16)
        v = torch.rand(O, I, generator=gen) * 1e-5 + 1e-9
        preps.append(ops.AdamPrepared(right.to(device), left.to(device), v.to(device), 0))
    one = O * p * I * 2
    monkeypatch.setattr(ops, "adam_table_budget_bytes", 2 * one)
    first = preps[0].table.clone()
    assert preps[1].table is not None and preps[0]._table is not None
    preps[2].table  # the third table does not fit: the least recently used one goes
    torch.cuda.synchronize()
    assert preps[0]._table is None and preps[1]._table is not None and preps[2]._table is not None
    assert torch.equal(preps[0].table, first)  # rebuilt
    assert preps[1]._table is None


def test_full_gradient_refuses_malformed_lengths_and_rows(device):
    """Both branches of the unprojected path check lengths (int32 [N]) and rows (int64 [N]) before launching."""
    from bergson_amd import ops

    N, S, I, O = 2, 8, 16, 32
    a = torch.randn(N, S, I, device=device)
    g = torch.randn(N, S, O, device=device)
    mod = ops.FullGradModule(O=O, I=I, out_col=0)
    out = torch.zeros(N * S, O * I, device=device)
    good_l = torch.tensor([8, 5], dtype=torch.int32, device=device)
    good_r = torch.tensor([0, 7], dtype=torch.int64, device=device)
    for per_token in (False, True):
        for lengths, rows in ((good_l.long(), good_r), (good_l, good_r.int()), (good_l[:1], good_r), (good_l, good_r[:1]),
                              (good_l.cpu(), good_r)):
            with pytest.raises((ValueError, RuntimeError)):
                ops.full_gradient(mod, a, g, out, per_token=per_token, lengths=lengths, rows=rows, lo=-1e30, hi=1e30)
    ops.full_gradient(mod, a, g, out, per_token=True, lengths=good_l, rows=good_r, lo=-1e30, hi=1e30)
    ops.full_gradient(mod, a, g, out, per_token=False, lengths=good_l, rows=torch.tensor([0, 1], device=device),
                      lo=-1e30, hi=1e30)
    torch.cuda.synchronize()
    want = torch.einsum("so,si->oi", g[1, :4], a[1, :4]).flatten()
    assert torch.allclose(out[1], want, rtol=1e-4, atol=1e-4)
