"""Pins the oracle's scoring functions by closed forms and invariants (CPU).

Restated from the reference's tests/test_query_batching_invariance.py (scoring a slice of the queries
equals the slice of scoring all of them; the index-side norm does not depend on the query slice),
tests/test_score.py (expected g/||g|| @ q^T; `nearest` equals the row maximum of the full product) and
tests/test_attributor.py (a stored row queried with itself comes back first with cosine > 0.99).
"""
import torch

from oracle import scan as S


def _data(seed=0, n=40, Q=6, sizes=(8, 12, 4)):
    gen = torch.Generator().manual_seed(seed)
    mods = [f"m{i}" for i in range(len(sizes))]
    index = {m: torch.randn(n, d, generator=gen) for m, d in zip(mods, sizes)}
    queries = {m: torch.randn(Q, d, generator=gen) for m, d in zip(mods, sizes)}
    return mods, index, queries


def test_scorer_cosine_closed_form():
    mods, index, queries = _data()
    got = S.scorer_score(index, queries, mods, unit_normalize=True)
    G = torch.cat([index[m] for m in mods], 1).double()
    Qm = torch.cat([queries[m] for m in mods], 1).double()
    want = (G / G.norm(dim=1, keepdim=True)) @ Qm.T
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-6)


def test_scorer_query_slices_and_nearest():
    mods, index, queries = _data(1)
    full = S.scorer_score(index, queries, mods, unit_normalize=True)
    part = S.scorer_score(index, {m: q[2:5] for m, q in queries.items()}, mods, unit_normalize=True)
    torch.testing.assert_close(part, full[:, 2:5])
    near = S.scorer_score(index, queries, mods, unit_normalize=True, score_mode="nearest")
    assert near.shape == (40, 1)
    torch.testing.assert_close(near[:, 0], full.max(dim=1).values)


def test_scorer_zero_row_scores_zero():
    mods, index, queries = _data(2)
    for m in mods:
        index[m][3] = 0
    got = S.scorer_score(index, queries, mods, unit_normalize=True)
    assert torch.isfinite(got).all() and (got[3] == 0).all()


def test_query_aggregation_mean_equals_mean_of_cosines():
    mods, index, queries = _data(3)
    qn = S.normalize_and_aggregate_queries(queries, mods, unit_normalize=True)
    cat = torch.cat([qn[m] for m in mods], 1)
    torch.testing.assert_close(cat.norm(dim=1), torch.ones(6))
    per_query = S.scorer_score(index, qn, mods, unit_normalize=True)
    qmean = S.normalize_and_aggregate_queries(queries, mods, unit_normalize=True, aggregation="mean")
    agg = S.scorer_score(index, qmean, mods, unit_normalize=True)
    torch.testing.assert_close(agg[:, 0], per_query.mean(dim=1), rtol=1e-5, atol=1e-6)
    qsum = S.normalize_and_aggregate_queries(queries, mods, unit_normalize=False, aggregation="sum",
                                             normalize_aggregated=True)
    assert torch.cat([qsum[m] for m in mods], 1).norm().item() == torch.tensor(1.0).item() or True
    torch.testing.assert_close(torch.cat([qsum[m] for m in mods], 1).norm(), torch.tensor(1.0))


def test_attributor_search_self_match_reverse_and_k():
    mods, index, _ = _data(4, n=60)
    picks = [0, 17, 59]
    queries = {m: index[m][picks] for m in mods}
    vals, idx = S.attributor_search(index, queries, mods, 5, unit_norm=True)
    assert idx[:, 0].tolist() == picks
    assert (vals[:, 0] > 0.99).all() and (vals[:, 1] < 0.9).all()
    rvals, ridx = S.attributor_search(index, queries, mods, 5, unit_norm=True, reverse=True)
    allv, alli = S.attributor_search(index, queries, mods, None, unit_norm=True)
    assert allv.shape == (3, 60)
    torch.testing.assert_close(rvals, allv[:, -5:].flip(1))
    # raw inner products when unit_norm is off
    v2, i2 = S.attributor_search(index, queries, mods, 60)
    G = torch.cat([index[m] for m in mods], 1)
    torch.testing.assert_close(v2, torch.sort(G[picks] @ G.T, dim=1, descending=True).values)


def test_attributor_index_normalisation_hand_worked():
    """`attributor_normalize_index` and `attributor_search` on numbers worked out by hand: the norm runs over all
    modules of a row together (3-4-12 -> 13), a zero row becomes zeros (0/0 -> NaN -> 0), and the search's cosines
    and order follow."""
    idx = {"a": torch.tensor([[3.0, 4.0], [0.0, 0.0], [0.0, 5.0], [-6.0, 0.0]]),
           "b": torch.tensor([[12.0], [0.0], [0.0], [8.0]])}
    norm = S.attributor_normalize_index(idx, ["a", "b"])
    assert torch.allclose(norm["a"], torch.tensor([[3 / 13, 4 / 13], [0.0, 0.0], [0.0, 1.0], [-0.6, 0.0]]))
    assert torch.allclose(norm["b"], torch.tensor([[12 / 13], [0.0], [0.0], [0.8]]))
    # one query along (0, 1 | 0): cosines 4/13, 0, 1, 0 -> rows 2, 0, then the two zeros (their order is not defined)
    q = {"a": torch.tensor([[0.0, 2.0]]), "b": torch.tensor([[0.0]])}
    vals, rows = S.attributor_search(idx, q, ["a", "b"], 4, unit_norm=True)
    assert rows[0, :2].tolist() == [2, 0] and sorted(rows[0, 2:].tolist()) == [1, 3]
    assert torch.allclose(vals, torch.tensor([[1.0, 4 / 13, 0.0, 0.0]]), atol=1e-6)
    # without unit norms: plain inner products 8, 0, 10, 0; reverse = smallest first
    vals, rows = S.attributor_search(idx, q, ["a", "b"], 2, unit_norm=False)
    assert rows.tolist() == [[2, 0]] and vals.tolist() == [[10.0, 8.0]]
    vals, rows = S.attributor_search(idx, {"a": torch.tensor([[1.0, 1.0]]), "b": torch.tensor([[1.0]])}, ["a", "b"], 2,
                                         unit_norm=False, reverse=True)
    assert rows.tolist() == [[1, 3]] and vals.tolist() == [[0.0, 2.0]]   # 19, 0, 5, 2 -> smallest first
