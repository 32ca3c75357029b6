"""Pins the oracle's ranking objectives and list metrics (LambdaRank gradients, MAP, NDCG) without running
the reference: closed forms for groups where the reference's loop leaves no freedom, invariants every pair
must satisfy, brute-force DCG differences, and hand-computed metric values."""
import os

import numpy as np
import pytest

import oracle_lib as O

HERE = os.path.dirname(os.path.abspath(__file__))


def _sigmoid_pair(s_hi, s_lo):
    rho = 1.0 / (1.0 + np.exp(np.float64(s_hi) - np.float64(s_lo)))
    return -rho, 2.0 * max(rho * (1.0 - rho), 1e-16)


def test_two_row_groups_closed_form():
    # A group of two rows with different labels leaves one possible pair; its lambda is -1 / (1 + e^(s_hi - s_lo)).
    rng = np.random.default_rng(0)
    n_g = 50
    y = np.zeros(2 * n_g, np.float32)
    hi_first = rng.random(n_g) < 0.5
    y[0::2] = hi_first
    y[1::2] = ~hi_first
    equal = rng.random(n_g) < 0.2  # some groups with equal labels: no pair, zero gradient
    y[0::2][equal] = 1
    y[1::2][equal] = 1
    s = rng.normal(size=2 * n_g).astype(np.float32)
    for seed in (0, 1, 12345):
        gh, order, pair = O.rank_gradient("rank:pairwise", y, s, [2] * n_g, seed)
        for g in range(n_g):
            a, b = 2 * g, 2 * g + 1
            if equal[g]:
                assert np.all(gh[a:b + 1] == 0)
                continue
            hi, lo = (a, b) if y[a] > y[b] else (b, a)
            lam, hess = _sigmoid_pair(s[hi], s[lo])
            np.testing.assert_allclose(gh[hi], [lam, hess], rtol=2e-6)
            np.testing.assert_allclose(gh[lo], [-lam, hess], rtol=2e-6)
            assert order[a] == hi and order[b] == lo
            assert pair[a] == b and pair[b] == -1  # only the first position of the label order draws


def _expected_order(y, s, groups):
    out = []
    start = 0
    for g in groups:
        rows = np.arange(start, start + g)
        # label descending, then score descending, then row ascending
        k = np.lexsort((rows, -s[rows].astype(np.float64), -y[rows].astype(np.float64)))
        out.append(rows[k])
        start += g
    return np.concatenate(out) if out else np.zeros(0, np.int64)


def _random_ranking_data(rng, groups, n_labels, tie_scores=False):
    n = int(np.sum(groups))
    y = rng.integers(0, n_labels, size=n).astype(np.float32)
    s = rng.normal(size=n).astype(np.float32)
    if tie_scores:
        s = np.round(s * 2) / 2
    return y, s


@pytest.mark.parametrize("tie_scores", [False, True])
def test_order_is_label_then_score_then_row(tie_scores):
    rng = np.random.default_rng(3)
    groups = [1, 7, 0, 40, 3, 129]
    y, s = _random_ranking_data(rng, groups, 4, tie_scores)
    _, order, _ = O.rank_gradient("rank:pairwise", y, s, groups, 5)
    assert np.array_equal(order, _expected_order(y, s, groups))


def test_drawing_positions_distinct_labels():
    # All labels of a group distinct: every run of equal labels has one row. The reference's loop handles
    # position 0, then steps over one position after every handled run (i = j; ++i), so exactly the even
    # positions draw, each from all other positions of the group.
    n = 11
    y = np.arange(n, dtype=np.float32)[::-1].copy()
    s = np.zeros(n, np.float32)
    seen_partners = set()
    for seed in range(200):
        _, order, pair = O.rank_gradient("rank:pairwise", y, s, [n], seed)
        assert np.array_equal(order, np.arange(n))
        for p in range(n):
            if p % 2 == 0:
                assert pair[p] >= 0 and pair[p] != p
                seen_partners.add((p, int(pair[p])))
            else:
                assert pair[p] == -1
    # the draw is uniform over the n - 1 other positions: every partner shows up for position 0 and 10
    assert {q for p, q in seen_partners if p == 0} == set(range(1, n))
    assert {q for p, q in seen_partners if p == 10} == set(range(0, 10))


def test_drawing_positions_binary_labels():
    # k relevant rows then the rest: positions [0, k) draw from [k, n); position k is stepped over; positions
    # [k + 1, n) draw from [0, k + 1) (which includes the stepped-over position k of their own label).
    n, k = 12, 4
    y = np.array([1] * k + [0] * (n - k), np.float32)
    s = -np.arange(n, dtype=np.float32)  # already in score order
    partners_low = set()
    for seed in range(300):
        _, order, pair = O.rank_gradient("rank:pairwise", y, s, [n], seed)
        assert np.array_equal(order, np.arange(n))
        assert np.all((pair[:k] >= k) & (pair[:k] < n))
        assert pair[k] == -1
        assert np.all((pair[k + 1:] >= 0) & (pair[k + 1:] <= k))
        partners_low.update(pair[k + 1:].tolist())
    assert partners_low == set(range(k + 1))


def _dcg(labels_in_order):
    pos = np.arange(len(labels_in_order), dtype=np.float64)
    return np.sum((2.0 ** np.asarray(labels_in_order, np.float64) - 1.0) / np.log2(pos + 2.0))


def _recompute(objective, y, s, groups, order, pair):
    """Gradients from the (order, pair) lists in float64; |delta NDCG| by brute force: the change of the
    group's DCG when the two positions swap their rows, divided by the ideal DCG."""
    n = len(y)
    acc = np.zeros((n, 2))
    start = 0
    for g in groups:
        labels = y[order[start:start + g]].astype(np.float64)
        ideal = _dcg(np.sort(labels)[::-1]) if g else 0.0
        for p in range(start, start + g):
            q = pair[p]
            if q < 0:
                continue
            hi, lo = (p, q) if p < q else (q, p)  # `high` is the position nearer the top of the label order
            if objective == "rank:ndcg":
                if ideal == 0:
                    dz = 0.0
                else:
                    swapped = labels.copy()
                    swapped[hi - start], swapped[lo - start] = swapped[lo - start], swapped[hi - start]
                    dz = abs(_dcg(labels) - _dcg(swapped)) / ideal
            else:
                dz = 1.0
            r_hi, r_lo = order[hi], order[lo]
            rho = 1.0 / (1.0 + np.exp(np.float64(s[r_hi]) - np.float64(s[r_lo])))
            lam = -dz * rho
            hess = 2.0 * max(dz * rho * (1.0 - rho), 1e-16)
            acc[r_hi] += [lam, hess]
            acc[r_lo] += [-lam, hess]
        start += g
    return acc


@pytest.mark.parametrize("objective", ["rank:pairwise", "rank:ndcg"])
def test_gradients_from_pairs_and_invariants(objective):
    rng = np.random.default_rng(11)
    groups = [5, 1, 33, 0, 64, 2, 17]
    y, s = _random_ranking_data(rng, groups, 5, tie_scores=True)
    for seed in (1, 99):
        gh, order, pair = O.rank_gradient(objective, y, s, groups, seed)
        exp = _recompute(objective, y, s, groups, order, pair)
        scale = np.abs(exp).max()
        assert np.abs(gh - exp).max() <= 2e-6 * scale
        start = 0
        for g in groups:
            rows = slice(start, start + g)
            assert abs(gh[rows, 0].astype(np.float64).sum()) <= 1e-5 * max(1.0, np.abs(gh[rows, 0]).sum())  # pairs cancel
            start += g
        assert np.all(gh[:, 1] >= 0)
        # a partner always lies outside the drawing position's own handled run: different label, or the
        # stepped-over first row of the run
        lab = y[order]
        gstart = np.repeat(np.cumsum([0] + groups[:-1]), groups)
        for p in np.nonzero(pair >= 0)[0]:
            q = pair[p]
            assert gstart[p] == gstart[q]  # same group
            if lab[p] == lab[q]:
                assert q < p and (q == gstart[q] or lab[q - 1] != lab[q])


def test_ndcg_gradient_zero_for_all_zero_labels():
    y = np.zeros(9, np.float32)
    s = np.linspace(-1, 1, 9).astype(np.float32)
    gh, _, _ = O.rank_gradient("rank:ndcg", y, s, [9], 3)
    assert np.all(gh == 0)  # one run of equal labels: nobody draws


def test_map_hand_values():
    # score order gives relevance 1,0,1,0 -> AP = (1/1 + 2/3) / 2; a group without relevant rows scores 1
    y = np.array([1, 0, 1, 0, 0, 0, 0], np.float32)
    s = np.array([4, 3, 2, 1, 0.3, 0.2, 0.1], np.float32)
    assert O.rank_metric("rank:pairwise", y, s, [4, 3]) == pytest.approx(((1 + 2 / 3) / 2 + 1) / 2, rel=1e-6)
    # worst order for two relevant rows out of four: AP = (1/3 + 2/4) / 2
    s2 = np.array([1, 3, 2, 4], np.float32)
    y2 = np.array([1, 0, 1, 0], np.float32)  # order by score: rows 3,1,2,0 -> 0,0,1,1
    assert O.rank_metric("rank:pairwise", y2, s2, [4]) == pytest.approx((1 / 3 + 2 / 4) / 2, rel=1e-6)
    # any non-zero label counts as a hit
    y3 = np.array([2, 0, -1, 0], np.float32)
    assert O.rank_metric("rank:pairwise", y3, s[:4], [4]) == pytest.approx((1 + 2 / 3) / 2, rel=1e-6)


def test_ndcg_values():
    rng = np.random.default_rng(5)
    groups = [6, 10, 3]
    y = rng.integers(0, 4, size=19).astype(np.float32)
    # a perfect ranking scores 1 in every group
    assert O.rank_metric("rank:ndcg", y, y + 0.0, groups) == pytest.approx(1.0, abs=1e-6)
    s = rng.normal(size=19).astype(np.float32)
    exp = 0.0
    start = 0
    for g in groups:
        rows = np.arange(start, start + g)
        k = np.argsort(-s[rows], kind="stable")
        ideal = _dcg(np.sort(y[rows])[::-1])
        exp += _dcg(y[rows][k]) / ideal if ideal else 1.0
        start += g
    assert O.rank_metric("rank:ndcg", y, s, groups) == pytest.approx(exp / 3, rel=1e-5)
    # all labels zero: IDCG = 0 and the group scores 1
    assert O.rank_metric("rank:ndcg", np.zeros(4, np.float32), s[:4], [4]) == 1.0
    # hand value: labels in score order 3,2,3,0,1,2 with gains (2^l - 1) / log2(i + 2)
    lab = np.array([3, 2, 3, 0, 1, 2], np.float32)
    sc = -np.arange(6, dtype=np.float32)
    dcg = 7 / 1 + 3 / np.log2(3) + 7 / 2 + 0 + 1 / np.log2(6) + 3 / np.log2(7)
    idcg = 7 / 1 + 7 / np.log2(3) + 3 / 2 + 3 / np.log2(5) + 1 / np.log2(6) + 0
    assert O.rank_metric("rank:ndcg", lab, sc, [6]) == pytest.approx(dcg / idcg, rel=1e-6)


def test_reference_group_fixture_covers_the_a1a_fixture():
    # the reference ships dataset/test_dataset.txt.group next to its a1a sample; sizes must add up to the rows
    sizes = [int(t) for t in open(os.path.join(HERE, "golden", "a1a_test_dataset.txt.group")).read().split()]
    rows = sum(1 for _ in open(os.path.join(HERE, "golden", "a1a_test_dataset.txt")))
    assert sizes == [100, 300, 400, 200, 605] and sum(sizes) == rows == 1605


def test_boosting_with_ranking_objective_improves_metric():
    rng = np.random.default_rng(2)
    groups = [30] * 20
    n = 600
    X = rng.normal(size=(n, 5)).astype(np.float32)
    rel = X[:, 0] + 0.5 * X[:, 1] + 0.3 * rng.normal(size=n)
    y = np.digitize(rel, [-0.5, 0.5, 1.2]).astype(np.float32)
    val, row_ptr, col = O.dense_to_csr(X)
    for objective in ("rank:pairwise", "rank:ndcg"):
        o = O.Oracle(val, row_ptr, col, y, depth=4, n_trees=10, learning_rate=0.3, objective=objective,
                     groups=groups).prepare()
        assert o.base_score == 0  # ObjectiveFunction::init_base_score is not overridden by LambdaRank
        first = o.metric()
        o.boost(10)
        log = o.metric_log()
        assert log[-1] > first + 0.02
        assert 0 < log[-1] <= 1
