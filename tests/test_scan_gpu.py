"""HIP store scan against the CPU oracle: scores within 1e-3 absolute cosine,
top-k indices identical except where scores tie within that tolerance."""
import pytest
import torch

from oracle import scan as oscan

pytestmark = pytest.mark.gpu

COS_TOL = 1e-3


def make_store(n, D, Q, dtype, seed, outliers=True):
    gen = torch.Generator().manual_seed(seed)
    store = torch.randn(n, D, generator=gen)
    if outliers:
        idx = torch.randperm(n, generator=gen)[: max(1, n // 20)]
        store[idx] *= 10
    queries = torch.randn(Q, D, generator=gen)
    return store.to(dtype), queries.to(dtype)


def unit_queries(queries, dtype):
    q = queries.float()
    q = q / (q.norm(dim=1, keepdim=True) + torch.finfo(torch.float32).eps)
    return q


def check_topk(vals, idx, ref_scores, k, tol=COS_TOL):
    """vals/idx [Q, k] from the kernel; ref_scores [Q, n] from the oracle."""
    ref_v, ref_i = torch.topk(ref_scores, k, dim=1)
    assert (vals - ref_v).abs().max().item() <= tol
    assert (vals[:, :-1] >= vals[:, 1:]).all(), "values must be sorted descending"
    # reported values are the scores of the reported rows
    assert (torch.gather(ref_scores, 1, idx) - vals).abs().max().item() <= tol
    for q in range(vals.shape[0]):
        got, want = set(idx[q].tolist()), set(ref_i[q].tolist())
        if got == want:
            continue
        kth = ref_v[q, -1].item()
        for r in got ^ want:  # may differ only among rows tied with the k-th score
            assert abs(ref_scores[q, r].item() - kth) <= tol, (q, r)
        assert len(got) == k


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(300, 256, 7, 10), (1000, 512, 40, 100), (5000, 1024, 130, 100)])
def test_scan_cosine_topk(device, dtype, shape):
    from bergson_amd import ops

    n, D, Q, k = shape
    store, queries = make_store(n, D, Q, dtype, seed=n)
    qn = unit_queries(queries, dtype)
    # the oracle scores what the kernel is given: store rows in `dtype`, unit queries rounded to `dtype`
    qd = qn.to(dtype)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True).T  # [Q, n]
    res = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=k, want_row_max=True, want_row_mean=True,
                   want_scores=True, want_sumsq=True, chunk_rows=1024)
    torch.cuda.synchronize()
    scores = res.scores.cpu().T
    assert (scores - ref).abs().max().item() <= COS_TOL
    # mean over queries: the mean of the scores, which by linearity is the score against the mean query
    # (how the reference gets it: aggregate the queries first, process_grads.py:166-182)
    assert (res.row_mean.cpu() - ref.mean(0)).abs().max().item() <= COS_TOL
    ref_mean_query = oscan.scorer_score({"m": store}, {"m": qd.float().mean(0, keepdim=True)}, ["m"],
                                        dtype=torch.float32, unit_normalize=True)[:, 0]
    assert (res.row_mean.cpu() - ref_mean_query).abs().max().item() <= COS_TOL
    assert torch.allclose(res.sumsq.cpu(), store.float().pow(2).sum(1), rtol=1e-4)
    assert (res.row_max.cpu() - ref.max(0).values).abs().max().item() <= COS_TOL
    check_topk(res.topk_values.cpu(), res.topk_indices.cpu(), ref, k)


def test_scan_matches_attributor_search(device):
    from bergson_amd import ops

    n, Q, k = 2000, 16, 50
    sizes = {"a": 256, "b": 256, "c": 512}
    gen = torch.Generator().manual_seed(7)
    index = {m: torch.randn(n, d, generator=gen).to(torch.float16) for m, d in sizes.items()}
    queries = {m: torch.randn(Q, d, generator=gen) for m, d in sizes.items()}
    mods = list(sizes)
    ref_v, ref_i = oscan.attributor_search(index, queries, mods, k, unit_norm=True)
    store = torch.cat([index[m] for m in mods], 1)
    qcat = torch.cat([queries[m] for m in mods], 1)
    qn = qcat / (qcat.norm(dim=1, keepdim=True) + torch.finfo(torch.float32).eps)
    res = ops.scan(store.to(device), qn.to(torch.float16).to(device), unit_norm=True, k=k)
    torch.cuda.synchronize()
    assert (res.topk_values.cpu() - ref_v).abs().max().item() <= COS_TOL
    same = (res.topk_indices.cpu() == ref_i).float().mean().item()
    assert same > 0.98  # neighbours closer than the tolerance may swap places


def test_scan_self_match_and_zero_rows(device):
    from bergson_amd import ops

    n, D = 700, 384
    store, _ = make_store(n, D, 1, torch.float16, seed=3)
    store[5] = 0  # documents with fewer than 2 tokens are stored as zero rows
    picks = [0, 5, 123, 699]
    q = store[picks].float()
    qn = q / (q.norm(dim=1, keepdim=True) + torch.finfo(torch.float32).eps)
    res = ops.scan(store.to(device), qn.to(torch.float16).to(device), unit_norm=True, k=3, want_scores=True)
    torch.cuda.synchronize()
    idx, vals, scores = res.topk_indices.cpu(), res.topk_values.cpu(), res.scores.cpu()
    assert torch.isfinite(scores).all()
    assert (scores[5] == 0).all()  # zero row scores 0 against everything
    for j, r in enumerate(picks):
        if r == 5:
            continue
        assert idx[j, 0].item() == r and vals[j, 0].item() > 0.99
        assert vals[j, 1].item() < 0.5


def test_scan_raw_inner_product_and_reverse(device):
    from bergson_amd import ops

    store, queries = make_store(900, 256, 5, torch.bfloat16, seed=11, outliers=False)
    ref = queries.float() @ store.float().T
    res = ops.scan(store.to(device), queries.to(device), unit_norm=False, k=20, want_scores=True)
    neg = ops.scan(store.to(device), (-queries).to(device), unit_norm=False, k=20)
    torch.cuda.synchronize()
    assert torch.allclose(res.scores.cpu().T, ref, rtol=1e-4, atol=1e-3)
    rv, ri = torch.topk(ref, 20, dim=1)
    assert torch.equal(res.topk_indices.cpu(), ri)
    lv, li = torch.topk(ref, 20, dim=1, largest=False)
    assert torch.equal(neg.topk_indices.cpu(), li)
    assert torch.allclose(-neg.topk_values.cpu(), lv, rtol=1e-4, atol=1e-3)


def test_scan_chunking_invariance(device):
    # the chunk size of the internal passes changes neither scores nor the selected rows
    from bergson_amd import ops

    store, queries = make_store(6000, 512, 33, torch.float16, seed=5)
    qd = unit_queries(queries, torch.float16).to(torch.float16)
    a = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=64, chunk_rows=512)
    b = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=64, chunk_rows=0)
    torch.cuda.synchronize()
    assert torch.equal(a.topk_indices.cpu(), b.topk_indices.cpu())
    assert torch.equal(a.topk_values.cpu(), b.topk_values.cpu())


def test_scan_ties_pick_lowest_rows(device):
    from bergson_amd import ops

    row = torch.randn(128)
    store = row.repeat(50, 1).to(torch.float16)
    res = ops.scan(store.to(device), row[None].to(torch.float16).to(device), unit_norm=True, k=10)
    torch.cuda.synchronize()
    assert res.topk_indices.cpu()[0].tolist() == list(range(10))


def test_scan_k_equals_rows_and_unaligned_dim(device):
    from bergson_amd import ops

    store, queries = make_store(37, 100, 3, torch.float32, seed=13, outliers=False)
    store = store[:, :99].contiguous()
    queries = queries[:, :99].contiguous()
    ref = queries @ store.T
    res = ops.scan(store.to(device), queries.to(device), unit_norm=False, k=37)
    torch.cuda.synchronize()
    rv, ri = torch.topk(ref, 37, dim=1)
    assert torch.equal(res.topk_indices.cpu(), ri)
    assert torch.allclose(res.topk_values.cpu(), rv, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("Q", [5, 48, 300])
def test_scan_row_mean_alone(device, Q):
    """Only the mean over queries is asked for (no top-k): several passes, every tile configuration."""
    from bergson_amd import ops

    n, D = 3000, 256
    store, queries = make_store(n, D, Q, torch.float16, seed=77)
    qd = unit_queries(queries, torch.float16).to(torch.float16)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True)  # [n, Q]
    res = ops.scan(store.to(device), qd.to(device), unit_norm=True, want_row_mean=True, chunk_rows=1024)
    torch.cuda.synchronize()
    assert res.topk_values is None
    assert (res.row_mean.cpu() - ref.mean(1)).abs().max().item() <= COS_TOL


# ---- few queries over a long store: the streaming kernel ------------------------------------------------
# At most 96 queries, a row length that is a multiple of two MFMA k-steps and at least two tiles of 256 rows
# per compute unit route the scan through the streaming kernel: a first pass of one tile per compute unit
# without thresholds (one candidate per row, cut down by the select kernel's sample bound), then the rest.
STREAM_ROWS = 2 * 256 * 256 + 9001  # past the minimum, with a ragged last tile


@pytest.mark.parametrize("dtype,D,Q", [(torch.float16, 128, 5), (torch.float16, 320, 32), (torch.bfloat16, 192, 16),
                                       (torch.bfloat16, 64, 23), (torch.float32, 96, 8), (torch.float32, 32, 32),
                                       (torch.float16, 128, 33), (torch.bfloat16, 192, 48), (torch.float32, 64, 41),
                                       (torch.float16, 192, 49), (torch.bfloat16, 128, 64), (torch.float32, 64, 70),
                                       (torch.float16, 64, 80), (torch.bfloat16, 320, 96), (torch.float32, 32, 91)])
def test_scan_streamed_few_queries(device, dtype, D, Q):
    from bergson_amd import _lib, ops

    n, k = STREAM_ROWS, 100
    store, queries = make_store(n, D, Q, dtype, seed=D + Q)
    store[12345] = 0  # a zero row scores 0 under unit norms
    qd = unit_queries(queries, dtype).to(dtype)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True).T  # [Q, n]
    dev_store, dev_q = store.to(device), qd.to(device)
    res = ops.scan(dev_store, dev_q, unit_norm=True, k=k, want_row_max=True, want_row_mean=True, want_scores=True,
                   want_sumsq=True)
    torch.cuda.synchronize()
    assert _lib.last_kernel(_lib.FAMILY_SCAN) == "scan_stream"
    assert (res.scores.cpu().T - ref).abs().max().item() <= COS_TOL
    assert res.scores[12345].abs().max().item() == 0
    assert (res.row_mean.cpu() - ref.mean(0)).abs().max().item() <= COS_TOL
    assert torch.allclose(res.sumsq.cpu(), store.float().pow(2).sum(1), rtol=1e-4)
    assert (res.row_max.cpu() - ref.max(0).values).abs().max().item() <= COS_TOL
    check_topk(res.topk_values.cpu(), res.topk_indices.cpu(), ref, k)
    # the tile kernel on the same inputs (passes too short for the streaming kernel) selects the same rows
    tiled = ops.scan(dev_store, dev_q, unit_norm=True, k=k, want_row_mean=True, chunk_rows=65536 - 256)
    torch.cuda.synchronize()
    check_topk(tiled.topk_values.cpu(), tiled.topk_indices.cpu(), ref, k)
    same = (tiled.topk_indices == res.topk_indices)
    assert (tiled.topk_values[same] - res.topk_values[same]).abs().max().item() <= 1e-5
    assert (tiled.row_mean - res.row_mean).abs().max().item() <= 1e-5


def test_scan_streamed_passes_and_short_tail(device):
    """Passes of exactly one tile per compute unit, then a tail too short for the streaming kernel."""
    from bergson_amd import ops

    n, D, Q, k = 2 * 65536 + 100, 128, 12, 300
    store, queries = make_store(n, D, Q, torch.float16, seed=3)
    store[-50:] *= 3.0
    ref = queries.to(torch.float16).float() @ store.float().T  # raw inner products
    res = ops.scan(store.to(device), queries.to(torch.float16).to(device), unit_norm=False, k=k, chunk_rows=65536,
                   want_row_mean=True)
    torch.cuda.synchronize()
    rv, ri = torch.topk(ref, k, dim=1)
    scale = ref.abs().max().item()
    assert (res.topk_values.cpu() - rv).abs().max().item() <= 2e-3 * scale
    agree = (res.topk_indices.cpu() == ri).float().mean().item()
    assert agree > 0.99  # rows may swap only where scores agree to rounding
    assert (res.row_mean.cpu() - ref.mean(0)).abs().max().item() <= 2e-3 * scale


def test_scan_streamed_without_topk(device):
    from bergson_amd import ops

    n, D, Q = STREAM_ROWS, 64, 9
    store, queries = make_store(n, D, Q, torch.bfloat16, seed=21)
    qd = unit_queries(queries, torch.bfloat16).to(torch.bfloat16)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True)  # [n, Q]
    res = ops.scan(store.to(device), qd.to(device), unit_norm=True, want_row_mean=True, want_row_max=True)
    torch.cuda.synchronize()
    assert res.topk_values is None
    assert (res.row_mean.cpu() - ref.mean(1)).abs().max().item() <= COS_TOL
    assert (res.row_max.cpu() - ref.max(1).values).abs().max().item() <= COS_TOL


def test_scan_streamed_ties_pick_lowest_rows(device):
    """Every row the same: every candidate of the first pass survives the sample bound's score, and the order
    among equal scores is by row number."""
    from bergson_amd import ops

    row = torch.randn(64, generator=torch.Generator().manual_seed(2))
    store = row.repeat(STREAM_ROWS, 1).to(torch.float16)
    res = ops.scan(store.to(device), row[None].to(torch.float16).to(device), unit_norm=True, k=150)
    torch.cuda.synchronize()
    assert res.topk_indices.cpu()[0].tolist() == list(range(150))


def test_scan_streamed_best_rows_last(device):
    """Scores that grow with the row number: the threshold of each pass is met by every later row."""
    from bergson_amd import ops

    n, D, k = STREAM_ROWS, 64, 64
    gen = torch.Generator().manual_seed(8)
    q = torch.randn(D, generator=gen)
    q = q / q.norm()
    ramp = torch.linspace(0.1, 4.0, n)[:, None]
    store = (q[None] * ramp + 0.01 * torch.randn(n, D, generator=gen)).to(torch.float16)
    qd = q[None].to(torch.float16)
    ref = qd.float() @ store.float().T
    res = ops.scan(store.to(device), qd.to(device), unit_norm=False, k=k)
    torch.cuda.synchronize()
    rv, ri = torch.topk(ref, k, dim=1)
    assert torch.allclose(res.topk_values.cpu(), rv, rtol=1e-3, atol=1e-3)
    assert len(set(res.topk_indices.cpu()[0].tolist()) & set(ri[0].tolist())) >= k - 2


# ---- many queries over a long 16-bit store: the tile kernel that loads straight into LDS ----------------
# At least 256 tiles of 256 rows x 256 queries, aligned fp16 / bf16 operands and D a multiple of 64 take the
# variant whose K tiles travel global -> LDS without registers (three row buffers, two query buffers); D of
# 64 to 320 covers its pipeline with one to five K tiles, rows and queries that do not fill the last tiles; at most
# 128 queries take its 128-query-wide form.
@pytest.mark.parametrize("dtype,D,Q", [(torch.float16, 64, 300), (torch.float16, 128, 257), (torch.bfloat16, 192, 300),
                                       (torch.float16, 256, 512), (torch.bfloat16, 320, 70), (torch.float16, 128, 128),
                                       (torch.float16, 64, 97)])
def test_scan_many_queries_direct_tiles(device, dtype, D, Q):
    from bergson_amd import ops

    n, k = 66_000 if Q > 256 else 131_000, 50
    store, queries = make_store(n, D, Q, dtype, seed=D + Q)
    store[777] = 0
    qd = unit_queries(queries, dtype).to(dtype)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True).T  # [Q, n]
    dev_store, dev_q = store.to(device), qd.to(device)
    res = ops.scan(dev_store, dev_q, unit_norm=True, k=k, want_row_max=True, want_row_mean=True, want_scores=True,
                   want_sumsq=True, chunk_rows=n)
    torch.cuda.synchronize()
    assert (res.scores.cpu().T - ref).abs().max().item() <= COS_TOL
    assert res.scores[777].abs().max().item() == 0
    assert (res.row_mean.cpu() - ref.mean(0)).abs().max().item() <= COS_TOL
    assert torch.allclose(res.sumsq.cpu(), store.float().pow(2).sum(1), rtol=1e-4)
    assert (res.row_max.cpu() - ref.max(0).values).abs().max().item() <= COS_TOL
    check_topk(res.topk_values.cpu(), res.topk_indices.cpu(), ref, k)
    # the same through passes too short for the large tiles (the 128-row tile kernel)
    small = ops.scan(dev_store, dev_q, unit_norm=True, k=k, chunk_rows=4096)
    torch.cuda.synchronize()
    same = small.topk_indices == res.topk_indices
    assert same.float().mean().item() > 0.99
    assert (small.topk_values[same] - res.topk_values[same]).abs().max().item() <= 1e-5


@pytest.mark.parametrize("dtype,D,Q", [(torch.float16, 192, 300), (torch.bfloat16, 128, 520), (torch.float16, 64, 1024),
                                       (torch.float16, 128, 200), (torch.bfloat16, 64, 129)])
def test_scan_wide_tiles_equal_the_256_tiles_bitwise(device, dtype, D, Q, bgx_env):
    """More than 128 queries over many rows: whole rounds of the chip (256 workgroups: 24 576 rows with four query
    tiles, 98 304 with one) run on the 384 x 256 tile kernel (one wave per SIMD, accumulators in both register
    files), the rest on the 256 x 256 kernels.  Every score is the
    same sequence of matrix instructions over D in both, and the row norms are summed in the same order: scores,
    norms, row maxima and the top-k must be the same bits with the wide kernel switched off; the row means add
    their per-wave partial sums in another order and agree to rounding.  Scores are also held to the oracle."""
    from bergson_amd import ops

    n, k = (4096 + 16384 + 2 * 24576 + 1500, 40) if Q > 256 else (4096 + 98304 + 11000, 40)
    store, queries = make_store(n, D, Q, dtype, seed=3 * D + Q)
    store[30_000] = 0
    qd = unit_queries(queries, dtype).to(dtype)
    dev_store, dev_q = store.to(device), qd.to(device)

    def run():
        r = ops.scan(dev_store, dev_q, unit_norm=True, k=k, want_row_max=True, want_row_mean=True, want_scores=True,
                     want_sumsq=True)
        torch.cuda.synchronize()
        return r

    wide = run()
    bgx_env("BGX_SCAN_WIDE_OFF", "1")
    narrow = run()
    assert torch.equal(wide.scores, narrow.scores)
    assert torch.equal(wide.sumsq, narrow.sumsq)
    assert torch.equal(wide.row_max, narrow.row_max)
    assert torch.equal(wide.topk_values, narrow.topk_values) and torch.equal(wide.topk_indices, narrow.topk_indices)
    assert (wide.row_mean - narrow.row_mean).abs().max().item() <= 1e-6
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True)  # [n, Q]
    assert (wide.scores.cpu() - ref).abs().max().item() <= COS_TOL
    assert wide.scores[30_000].abs().max().item() == 0
    check_topk(wide.topk_values.cpu(), wide.topk_indices.cpu(), ref.T, k)


def test_scan_with_known_row_norms_equals_the_plain_scan_bitwise(device):
    """bgx_scan_known_norms: the row sums of squares of one scan handed to the next.  With more than 256 queries the
    wide-tile kernel then leaves the norms out of its K loop; everything it reports is the same bits, and so it is
    for query counts whose kernels ignore the array."""
    from bergson_amd import ops

    gen = torch.Generator().manual_seed(77)
    n, D = 4096 + 24576 + 10240 + 300, 256  # the last pass: less than a round of the wide tiles, ragged end
    store = torch.randn(n, D, generator=gen).to(torch.float16).to(device)
    for Q in (1024, 300, 40):
        q = torch.randn(Q, D, generator=gen).to(torch.float16).to(device)
        plain = ops.scan(store, q, unit_norm=True, k=10, want_row_max=True, want_row_mean=True, want_sumsq=True)
        known = ops.scan(store, q, unit_norm=True, k=10, want_row_max=True, want_row_mean=True,
                         row_sumsq=plain.sumsq)
        torch.cuda.synchronize()
        assert torch.equal(plain.topk_values, known.topk_values)
        assert torch.equal(plain.topk_indices, known.topk_indices)
        assert torch.equal(plain.row_max, known.row_max)
        assert torch.equal(plain.row_mean, known.row_mean)
    with pytest.raises(ValueError):
        ops.scan(store, q, unit_norm=True, k=10, row_sumsq=plain.sumsq[:-1])


@pytest.mark.parametrize("n,D,Q", [(9000, 128, 5), (9000, 128, 48), (12000, 128, 300), (140000, 64, 8)])
def test_scan_rows_with_nan_scores_are_never_selected(device, n, D, Q):
    """A row whose score is NaN (a NaN or infinite element) is left out of the top-k whichever pass and kernel
    meets it -- inside the first, threshold-free pass (rows 7, 4000 of the tile scans' 4096; any row of the
    streaming scan's first 65 536) or beyond it -- so the result is the oracle's on the store without those
    rows.  The last shape runs the few-queries streaming kernel."""
    from bergson_amd import ops

    store, queries = make_store(n, D, Q, torch.float16, seed=n + Q, outliers=False)
    bad = [7, 4000, 4100, n - 3]
    store[bad[0], 3] = float("nan")
    store[bad[1], 5] = float("inf")
    store[bad[2], 0] = float("nan")
    store[bad[3], 9] = float("-inf")
    qd = unit_queries(queries, torch.float16).to(torch.float16)
    clean = store.clone()
    clean[bad] = 0
    ref = oscan.scorer_score({"m": clean}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True).T
    ref[:, bad] = float("-inf")
    for known in (False, True):
        res = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=50, want_sumsq=True)
        if known:
            res = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=50, row_sumsq=res.sumsq)
        torch.cuda.synchronize()
        idx = res.topk_indices.cpu()
        assert not set(idx.flatten().tolist()) & set(bad)
        assert torch.isfinite(res.topk_values).all()
        check_topk(res.topk_values.cpu(), idx, ref, 50)


def test_scan_fewer_selectable_rows_than_k(device):
    """Twenty rows of which fifteen score NaN, k = 10: the five real scores in order, then (-inf, -1)."""
    from bergson_amd import ops

    store, queries = make_store(20, 64, 3, torch.float32, seed=2, outliers=False)
    good = [1, 4, 9, 10, 17]
    for r in range(20):
        if r not in good:
            store[r, r % 64] = float("nan")
    res = ops.scan(store.to(device), queries.to(device), unit_norm=False, k=10)
    torch.cuda.synchronize()
    ref = queries @ store[good].T
    rv, ri = torch.topk(ref, 5, dim=1)
    assert torch.allclose(res.topk_values.cpu()[:, :5], rv, rtol=1e-5, atol=1e-5)
    assert torch.equal(res.topk_indices.cpu()[:, :5], torch.tensor(good)[ri])
    assert (res.topk_values.cpu()[:, 5:] == float("-inf")).all() and (res.topk_indices.cpu()[:, 5:] == -1).all()


@pytest.mark.parametrize("Q", [6, 70, 200])
def test_scan_passes_shorter_than_k(device, Q):
    """An explicit chunk_rows below k: the early passes hold fewer than k rows, no threshold exists until k
    scores have been seen, and the result is still the oracle's."""
    from bergson_amd import ops

    n, D, k = 3000, 256, 500
    store, queries = make_store(n, D, Q, torch.float16, seed=77)
    qd = unit_queries(queries, torch.float16).to(torch.float16)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True).T
    res = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=k, chunk_rows=256)
    torch.cuda.synchronize()
    check_topk(res.topk_values.cpu(), res.topk_indices.cpu(), ref, k)
    whole = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=k)
    torch.cuda.synchronize()
    assert torch.equal(whole.topk_indices, res.topk_indices) and torch.equal(whole.topk_values, res.topk_values)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,D", [(4096 + 24576 + 300, 256), (5000, 192), (1000, 12288), (777, 100)])
def test_row_sumsq_equals_the_sums_a_scan_forms(device, dtype, n, D):
    """bgx_row_sumsq, the one pass that stands for the reference's normalisation of an index at load time: against
    float64, and bit for bit against the `sumsq` output of scans on the tile kernels (256 x 256 register-staged,
    direct-to-LDS, 384 x 256 wide), whose order of additions it follows -- so a scan given these sums returns
    exactly what a scan that forms them returns."""
    from bergson_amd import ops

    gen = torch.Generator().manual_seed(n + D)
    store = (torch.randn(n, D, generator=gen) * torch.rand(n, 1, generator=gen) * 4).to(dtype)
    store[5] = 0
    dev_store = store.to(device)
    got = ops.row_sumsq(dev_store)
    torch.cuda.synchronize()
    want = store.double().pow(2).sum(1)
    assert torch.allclose(got.cpu().double(), want, rtol=2e-5, atol=0)  # fp32 running sums over up to 1536 K tiles
    assert got[5].item() == 0.0
    for Q in (300, 100):
        q = torch.randn(Q, D, generator=gen).to(dtype).to(device)
        plain = ops.scan(dev_store, q, unit_norm=True, k=10, want_sumsq=True, want_row_max=True)
        given = ops.scan(dev_store, q, unit_norm=True, k=10, row_sumsq=got, want_row_max=True)
        torch.cuda.synchronize()
        assert torch.equal(plain.sumsq, got), Q
        assert torch.equal(plain.topk_values, given.topk_values) and torch.equal(plain.topk_indices, given.topk_indices)
        assert torch.equal(plain.row_max, given.row_max)
    # a strided view (rows of a wider matrix) gives the same sums
    wide = torch.zeros(n, D + 24, dtype=dtype, device=device)
    wide[:, :D] = dev_store
    assert torch.equal(ops.row_sumsq(wide[:, :D]), got)


@pytest.mark.parametrize("n,D,Q,k,chunk", [(30000, 128, 5, 3000, 0), (30000, 128, 40, 5000, 4096),
                                           (40000, 64, 300, 2049, 0), (150000, 64, 3, 20000, 0),
                                           (9000, 64, 2, 9000, 1000)])
def test_scan_topk_beyond_2048(device, n, D, Q, k, chunk):
    """k above what one workgroup sorts on chip: the running top-k lives in the workspace, is cut to the k largest
    after every pass and sorted once at the end.  Against the oracle's scores and torch.topk; passes shorter and
    longer than k, every kernel family, and k = all rows."""
    from bergson_amd import ops

    store, queries = make_store(n, D, Q, torch.float16, seed=n + k)
    qd = unit_queries(queries, torch.float16).to(torch.float16)
    ref = oscan.scorer_score({"m": store}, {"m": qd}, ["m"], dtype=torch.float32, unit_normalize=True).T
    res = ops.scan(store.to(device), qd.to(device), unit_norm=True, k=k, chunk_rows=chunk)
    torch.cuda.synchronize()
    vals, idx = res.topk_values.cpu(), res.topk_indices.cpu()
    assert all(len(set(r.tolist())) == k for r in idx)
    check_topk(vals, idx, ref, k)
    with pytest.raises(Exception, match="k="):
        ops.scan(store.to(device), qd.to(device), unit_norm=True, k=65537 if n > 65537 else n + 1)


def test_attributor_topk_beyond_2048(device, tmp_path):
    """Attributor.search with k = 3000 runs on the fused selection and agrees with the oracle's search."""
    import numpy as np

    from bergson_amd import Attributor
    from bergson_amd.data import create_index
    from bergson_amd.gradients import GradientProcessor

    gen = torch.Generator().manual_seed(5)
    n = 8000
    rows = torch.randn(n, 256, generator=gen)
    path = tmp_path / "idx"
    mm = create_index(path, num_grads=n, grad_sizes={"a": 256}, dtype="float16")
    mm[:] = rows.to(torch.float16).numpy()
    mm.flush()
    GradientProcessor(projection_dim=16).save(path)
    stored = torch.from_numpy(np.array(mm)).float()
    q = torch.randn(3, 256, generator=gen)
    attr = Attributor(path, device="cuda:0", unit_norm=True)
    vals, idx = attr.search({"a": q.to(device)}, k=3000)
    ref_v, ref_i = oscan.attributor_search({"a": stored}, {"a": q}, ["a"], 3000, unit_norm=True)
    assert (vals.cpu() - ref_v).abs().max().item() <= 1e-3
    # with 3000 of 8000 random rows selected, neighbours closer than the 16-bit store's tolerance swap places and the
    # last few may differ: the sets agree almost entirely, the values throughout
    for qi in range(3):
        assert len(set(idx[qi].tolist()) & set(ref_i[qi].tolist())) >= 2985
    vals_all, idx_all = attr.search({"a": q.to(device)}, k=None)   # the full ranking
    assert idx_all.shape == (3, n) and sorted(idx_all[0].tolist()) == list(range(n))
