"""GPU parity of the ranking objectives (rank:pairwise, rank:ndcg) and list metrics (MAP, NDCG) against the
CPU oracle: row order bit-exact, gradients / metrics within 1e-5, trees through the usual tree comparison."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import datasets as D
import oracle_lib as O
import parity as P

pytestmark = pytest.mark.gpu

LIBC = C.CDLL("libc.so.6")
LIBC.rand.restype = C.c_int


@pytest.fixture(scope="module")
def T():
    import thundergbm_amd
    L = thundergbm_amd.load()
    # the first GPU call of a process initialises the runtime (which may draw from rand() itself): do it here,
    # so that no test's random stream depends on which test runs first
    D.warm_up(thundergbm_amd)
    return thundergbm_amd


def _round_seed(seed):
    """The value the next rand() returns after srand(seed): what one gradient pass consumes."""
    LIBC.srand(seed)
    v = LIBC.rand()
    LIBC.srand(seed)
    return v


def _ranking_case(name):
    rng = np.random.default_rng(sum(map(ord, name)))
    if name == "small_mixed":
        groups = [5, 1, 33, 0, 64, 2, 17, 300]
        n_labels, F = 5, 6
    elif name == "tiny_groups":
        groups = [2] * 150 + [1] * 20 + [3] * 40
        n_labels, F = 2, 4
    elif name == "one_big_group":  # several radix tiles inside one group
        groups = [20000]
        n_labels, F = 4, 5
    elif name == "many_groups":
        groups = rng.integers(1, 200, size=400).tolist()
        n_labels, F = 5, 8
    elif name == "binary_relevance":
        groups = rng.integers(5, 60, size=120).tolist()
        n_labels, F = 2, 6
    else:
        raise KeyError(name)
    n = int(np.sum(groups))
    X = rng.normal(size=(n, F)).astype(np.float32)
    X[rng.random(X.shape) < 0.1] = 0  # some missing values
    rel = X[:, 0] + 0.5 * X[:, 1] - 0.25 * X[:, 2] + 0.5 * rng.normal(size=n)
    qs = np.quantile(rel, np.linspace(0, 1, n_labels + 1)[1:-1])
    y = np.digitize(rel, qs).astype(np.float32)
    return D.dense_to_csr(X), y, groups


CASES = ["small_mixed", "tiny_groups", "one_big_group", "many_groups", "binary_relevance"]


@pytest.mark.parametrize("objective", ["rank:pairwise", "rank:ndcg"])
@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("ties", [False, True])
def test_rank_gradient_and_metric_parity(T, objective, name, ties):
    (val, rp, col), y, groups = _ranking_case(name)
    n = len(y)
    s = T.Session(val, rp, col, y, depth=4, n_trees=2, objective=objective, groups=groups)
    assert s.base_score == 0
    rng = np.random.default_rng(len(name) + ties)
    for trial in range(3):
        score = rng.normal(size=n).astype(np.float32)
        if ties:
            score = (np.round(score * 2) / 2).astype(np.float32)  # many equal scores, some -0.0
            score[score == 0] = -0.0 if trial == 1 else 0.0
        if trial == 2 and not ties:
            score[:] = 0  # the first round of every training run: all scores equal
        s.set("y_pred", score)
        seed = 1000 + 17 * trial
        draw = _round_seed(seed)
        s.gradient()
        gh = s.gh()
        order = s.get("rank_order", np.int32)
        ogh, oorder, _ = O.rank_gradient(objective, y, score, groups, draw)
        assert np.array_equal(order, oorder)  # index work: bit-exact
        scale = max(np.abs(ogh).max(), 1e-30)
        assert np.abs(gh.astype(np.float64) - ogh).max() <= 1e-5 * scale
        # pairs cancel inside every group (exact in the fixed-point sums, float rounding once per row)
        start = 0
        for g in groups:
            seg = gh[start:start + g, 0].astype(np.float64)
            assert abs(seg.sum()) <= 1e-6 * max(1.0, np.abs(seg).sum())
            start += g
        m = s.metric()
        om = O.rank_metric(objective, y, score, groups)
        assert abs(m - om) <= 1e-5 * max(1.0, abs(om))
        # right after a metric pass the gradient re-sorts the metric's order by run id only: same bits
        _round_seed(seed)
        s.gradient()
        assert np.array_equal(s.get("rank_order", np.int32), order)
        assert np.array_equal(s.gh(), gh)
    s.close()


@pytest.mark.parametrize("sort", ["counting", "radix"])
def test_rank_full_size_parity(T, sort, monkeypatch):
    """About a million rows in 8 000 query groups (several thousand radix tiles, 40 000 label runs): order
    bit-exact, gradients and both metrics against the oracle, which handles this size in a second. Groups this
    short are ordered by counting; TGBM_RANK_SORT=radix sends them through the radix sort that longer groups take."""
    if sort == "radix":
        monkeypatch.setenv("TGBM_RANK_SORT", "radix")
    else:
        monkeypatch.delenv("TGBM_RANK_SORT", raising=False)
    rng = np.random.default_rng(17)
    groups = rng.integers(40, 200, size=8000)
    n = int(groups.sum())
    F = 6
    X = rng.normal(size=(n, F)).astype(np.float32)
    rel = X[:, 0] + 0.5 * X[:, 1] + rng.normal(size=n)
    y = np.digitize(rel, np.quantile(rel, [0.5, 0.75, 0.9, 0.97])).astype(np.float32)
    rp = np.arange(0, n * F + 1, F, dtype=np.int32)
    col = np.tile(np.arange(F, dtype=np.int32), n)
    for objective in ("rank:pairwise", "rank:ndcg"):
        s = T.Session(X.ravel(), rp, col, y, depth=6, n_trees=3, learning_rate=0.3, objective=objective,
                      groups=groups)
        LIBC.srand(9)
        s.boost(2)  # scores with many distinct values and, from the leaves, many ties
        score = s.y_pred()
        draw = _round_seed(31)
        s.gradient()
        gh, order = s.gh(), s.get("rank_order", np.int32)
        ogh, oorder, _ = O.rank_gradient(objective, y, score, groups, draw)
        assert np.array_equal(order, oorder)
        assert np.abs(gh.astype(np.float64) - ogh).max() <= 1e-5 * np.abs(ogh).max()
        assert abs(s.metric() - O.rank_metric(objective, y, score, groups)) <= 1e-5
        log = s.metric_log()
        assert log[1] > log[0]
        s.close()


def test_rank_gradient_is_bit_reproducible(T):
    (val, rp, col), y, groups = _ranking_case("many_groups")
    s = T.Session(val, rp, col, y, depth=4, n_trees=2, objective="rank:ndcg", groups=groups)
    score = np.random.default_rng(0).normal(size=len(y)).astype(np.float32)
    s.set("y_pred", score)
    outs = []
    for _ in range(3):
        LIBC.srand(77)
        s.gradient()
        outs.append(s.gh().copy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    LIBC.srand(78)  # another seed draws other partners
    s.gradient()
    assert not np.array_equal(outs[0], s.gh())
    s.close()


@pytest.mark.parametrize("objective", ["rank:pairwise", "rank:ndcg"])
@pytest.mark.parametrize("name", ["small_mixed", "many_groups"])
def test_rank_boosting_teacher_forced(T, objective, name):
    """Every round both sides start from the GPU's scores and draw the same partners (same rand() seed);
    gradients, trees, updated scores and the metric are compared round by round."""
    (val, rp, col), y, groups = _ranking_case(name)
    rounds = 6
    kw = dict(depth=5, n_trees=rounds, learning_rate=0.3, objective=objective, min_child_weight=0.1)
    s = T.Session(val, rp, col, y, groups=groups, **kw)
    o = O.Oracle(val, rp, col, y, debug=True, groups=groups, **kw).prepare()
    _, crp, _ = s.cuts()
    n = s.n
    present = np.zeros((n, s.F), bool)
    present[np.repeat(np.arange(n), np.diff(rp)), col] = True
    total_ties = 0
    metrics = []
    for r in range(rounds):
        yp = s.y_pred()
        o.set_y_pred(yp)
        LIBC.srand(500 + r)
        o.compute_gradient()
        ogh = o.gh()
        LIBC.srand(500 + r)
        s.gradient()  # the gradients the round is built from, for the comparison
        gh = s.gh()
        LIBC.srand(500 + r)
        s.boost(1)  # computes them again with the same draws
        scale = np.abs(ogh).max()
        assert np.abs(gh.astype(np.float64) - ogh).max() <= 1e-5 * scale
        o.set_gh(gh)
        o.build_tree(0)
        final_nid = o.nid()
        ghk = np.abs(gh.astype(np.float64)).sum(axis=0)
        d = P.compare_trees(s.model()[r, 0], o.nodes(), 1.0, crp=crp, orc_scores=o.tree_scores(), orc_dir_gaps=o.tree_dir_gaps(),
                            missing_rows=lambda x, f: int((~present[P.rows_in_node(final_nid, x), f]).sum()),
                            abs_scale=(ghk[0], ghk[1]), mcw=0.1)
        total_ties += len(d.near_ties)
        if not d.near_ties:
            tol = P.pred_tolerance(o.nodes(), final_nid, kw["learning_rate"], 1.0, (ghk[0], ghk[1]), o.y_pred())
            assert np.all(np.abs(s.y_pred().astype(np.float64) - o.y_pred()) <= tol)
        metrics.append(s.metric_log()[-1])
        # the metric of the GPU's own scores, recomputed by the oracle
        assert abs(metrics[-1] - O.rank_metric(objective, y, s.y_pred(), groups)) <= 1e-5
    # pairwise lambdas of equal scores repeat the same few values, so exact gain ties are common on small
    # groups; every accepted tie was checked to lie within the gain tolerance
    assert total_ties <= rounds
    assert metrics[-1] > metrics[0]
    s.close()


@pytest.mark.parametrize("layout", ["dense", "sparse"])
def test_rank_with_bagging_and_column_sampling(T, layout):
    """Everything that draws from rand() in one round, in the reference's order (booster.h:80-84 gradients,
    then bagging; tree_builder.cu:150-152 column sampling at the start of the tree building): the ranking
    partner seed, the bagging seed, the shuffle of the columns. Both sides start every round from the same
    srand() and must build the same trees."""
    os.environ["TGBM_LAYOUT"] = layout
    try:
        (val, rp, col), y, groups = _ranking_case("many_groups")
        rounds = 4
        kw = dict(depth=4, n_trees=rounds, learning_rate=0.3, objective="rank:ndcg", min_child_weight=0.05)
        s = T.Session(val, rp, col, y, groups=groups, **kw)
        o = O.Oracle(val, rp, col, y, debug=True, groups=groups, **kw).prepare()
        s.set_option("bagging", 1)
        s.set_option("column_sampling_rate", 0.5)
        o.set_bagging(True)
        o.set_column_sampling_rate(0.5)
        n = s.n
        ties = 0
        for r in range(rounds):
            o.set_y_pred(s.y_pred())
            LIBC.srand(900 + r)
            o.compute_gradient()
            o.sample_columns()
            ogh = o.gh()
            LIBC.srand(900 + r)
            s.gradient()
            gh = s.gh()
            assert np.abs(gh.astype(np.float64) - ogh).max() <= 1e-5 * np.abs(ogh).max()
            LIBC.srand(900 + r)
            s.boost(1)
            o.set_gh(gh)
            o.build_tree(0)
            ghk = np.abs(gh.astype(np.float64)).sum(axis=0)
            d = P.compare_trees(s.model()[r, 0], o.nodes(), 1.0, crp=s.cuts()[1], orc_scores=o.tree_scores(), orc_dir_gaps=o.tree_dir_gaps(),
                                abs_scale=(ghk[0], ghk[1]), mcw=0.05)
            ties += len(d.near_ties)
        assert ties <= rounds
        s.close()
    finally:
        os.environ.pop("TGBM_LAYOUT", None)


def test_ranker_through_the_c_abi(T, tmp_path):
    """sparse_train_scikit / sparse_predict_scikit with group sizes (scikit_tgbm.cpp:26-121 with the group and
    num_group arguments): the model ranks better than the constant score and predicts raw scores."""
    (val, rp, col), y, groups = _ranking_case("binary_relevance")
    import scipy.sparse as sp
    X = sp.csr_matrix((val, col, rp), shape=(len(y), int(col.max()) + 1))
    base_map = O.rank_metric("rank:pairwise", y, np.zeros(len(y), np.float32), groups)
    for objective in ("rank:pairwise", "rank:ndcg"):
        m = T.TGBMRegressor(depth=4, n_trees=15, learning_rate=0.3, objective=objective, verbose=0)
        LIBC.srand(3)
        m.fit(X, y, groups=groups)
        pred = np.asarray(m.predict(X, groups=groups), np.float32)
        assert pred.shape == (len(y),)
        assert O.rank_metric("rank:pairwise", y, pred, groups) > base_map + 0.1
        # raw scores: the sum of the leaf values, no transform, base score 0
        o = O.Oracle(val, rp, col, y, depth=4, n_trees=15, learning_rate=0.3, objective=objective,
                     groups=groups).prepare()
        LIBC.srand(3)
        o.boost(15)
        # free-running runs may part ways at a near tie; the first rounds agree and the quality is the same
        assert abs(O.rank_metric(objective, y, pred, groups) - o.metric_log()[-1]) < 0.02
        path = str(tmp_path / "rank.model")
        m.save_model(path)
        m2 = T.TGBMRegressor(objective=objective, verbose=0)
        m2.load_model(path)
        np.testing.assert_allclose(np.asarray(m2.predict(X), np.float32), pred, rtol=1e-6, atol=1e-7)


def test_ranking_needs_consistent_groups(T):
    """LambdaRank::configure checks that the groups cover the instances (ranking_obj.cpp:14-17); a mismatch
    is fatal. Checked in a child process because fatal errors abort."""
    code = (
        "import numpy as np, thundergbm_amd as T\n"
        "X = np.random.default_rng(0).normal(size=(50, 3)).astype(np.float32)\n"
        "y = (X[:, 0] > 0).astype(np.float32)\n"
        "import sys; sys.path.insert(0, %r)\n"
        "import datasets as D\n"
        "val, rp, col = D.dense_to_csr(X)\n"
        "T.Session(val, rp, col, y, objective='rank:pairwise', groups=%s)\n"
    )
    here = os.path.dirname(os.path.abspath(__file__))
    root = os.path.dirname(here)
    for groups in ("[20, 20]", "None"):
        out = subprocess.run(["python", "-c", code % (here, groups)], capture_output=True, text=True, cwd=root,
                             timeout=300)
        assert out.returncode != 0
        assert "FATAL" in out.stderr and "group" in out.stderr


def test_cli_ranking_on_reference_group_file(T, tmp_path):
    """thundergbm-train with objective=rank:pairwise loads <data>.group (dataset.cpp:302): the reference ships
    test_dataset.txt.group for its a1a sample. All a1a labels are non-zero, so MAP is 1 by definition; the run
    covers the loader, the LambdaRank rounds and the predictor's metric line."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    conf = tmp_path / "rank.conf"
    conf.write_text("data=%s\nobjective=rank:pairwise\nn_trees=5\ndepth=4\n" % D.A1A)
    train = os.path.join(root, "thundergbm_amd", "bin", "thundergbm-train")
    predict = os.path.join(root, "thundergbm_amd", "bin", "thundergbm-predict")
    out = subprocess.run([train, str(conf)], capture_output=True, text=True, cwd=tmp_path, timeout=300)
    assert out.returncode == 0, out.stderr
    assert "#groups = 5" in out.stdout
    assert "[5/5] MAP = 1" in out.stdout
    out = subprocess.run([predict, str(conf)], capture_output=True, text=True, cwd=tmp_path, timeout=300)
    assert out.returncode == 0, out.stderr
    assert "MAP = 1" in out.stdout
    # the same trees as the oracle: the process-wide rand() of a fresh process starts from srand(1)
    val, rp, col, y = D.read_libsvm(D.A1A)
    groups = [100, 300, 400, 200, 605]
    o = O.Oracle(val, rp, col, y, depth=4, n_trees=5, objective="rank:pairwise", groups=groups).prepare()
    LIBC.srand(1)
    o.boost(5)
    assert o.metric_log()[-1] == 1.0
