"""GPU parity on edge shapes: tiny and ragged inputs, empty rows, one feature, extreme depths and bin
counts, every objective. Each case boosts a few rounds with the oracle restarted from the GPU's
predictions (teacher forcing) and compares every tree."""
import os
import zlib

import numpy as np
import pytest

import datasets as D
import oracle_lib as O
import parity as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import thundergbm_amd
    L = thundergbm_amd.load()
    # the first GPU call of a process initialises the runtime (which may draw from rand() itself): do it here,
    # so that no test's random stream depends on which test runs first
    D.warm_up(thundergbm_amd)
    return thundergbm_amd


@pytest.fixture(autouse=True)
def _default_layout():
    for k in ("TGBM_LAYOUT", "TGBM_CSR_HEAD", "TGBM_BATCH_CLASSES", "TGBM_CSC_ROOT", "TGBM_SPARSE_PASS",
              "TGBM_SPARSE_SORTED", "TGBM_SPARSE_COLS", "TGBM_HIST_ARENA_NODES", "TGBM_WIDE_EVAL",
              "TGBM_DENSE_BIN_BYTES", "TGBM_DENSE_W", "TGBM_BUNDLE"):
        os.environ.pop(k, None)
    yield
    for k in ("TGBM_LAYOUT", "TGBM_CSR_HEAD", "TGBM_BATCH_CLASSES", "TGBM_CSC_ROOT", "TGBM_SPARSE_PASS",
              "TGBM_SPARSE_SORTED", "TGBM_SPARSE_COLS", "TGBM_HIST_ARENA_NODES", "TGBM_WIDE_EVAL",
              "TGBM_DENSE_BIN_BYTES", "TGBM_DENSE_W", "TGBM_BUNDLE"):
        os.environ.pop(k, None)


def _ragged(n, F, seed, max_len):
    rng = np.random.default_rng(seed)
    lens = rng.integers(0, max_len + 1, n)
    lens[: max(1, n // 50)] = 0  # some completely empty rows
    rp = np.zeros(n + 1, np.int32)
    np.cumsum(lens, out=rp[1:])
    col = np.concatenate([np.sort(rng.choice(F, size=l, replace=False)) for l in lens] + [np.zeros(0, np.int64)])
    col = col.astype(np.int32)
    val = np.round(rng.standard_normal(len(col)) * 3, 1).astype(np.float32)
    val[val == 0] = 1.5
    if len(col) and col.max() != F - 1:  # make sure the feature count is what the case says
        col[-1] = F - 1
    return val, rp, col


def _target(val, rp, col, n, F, seed, kind):
    rng = np.random.default_rng(seed + 100)
    w = rng.standard_normal(F)
    s = np.zeros(n)
    rows = np.repeat(np.arange(n), np.diff(rp))
    np.add.at(s, rows, w[col] * val)
    s += 0.3 * rng.standard_normal(n)
    if kind == "reg":
        return s.astype(np.float32)
    if kind == "bin":
        return np.where(s > np.median(s), 5.0, 2.0).astype(np.float32)  # arbitrary label values
    if kind == "prob":
        return (1 / (1 + np.exp(-s))).astype(np.float32)
    q = np.quantile(s, [0.2, 0.5, 0.8])
    return (np.digitize(s, q) * 10 - 7).astype(np.float32)  # labels -7, 3, 13, 23


CASES = {
    # name: (n, F, max row length, objective, target kind, kwargs, layout)
    "tiny": (37, 5, 5, "reg:linear", "reg", dict(depth=3, max_num_bin=8), None),
    "one_feature": (500, 1, 1, "reg:linear", "reg", dict(depth=4, max_num_bin=16), None),
    "depth1": (800, 6, 6, "binary:logistic", "bin", dict(depth=1, max_num_bin=32), None),
    "depth10": (3000, 7, 7, "reg:linear", "reg", dict(depth=10, max_num_bin=64, gamma=0.0), None),
    "two_bins": (1000, 9, 9, "binary:logistic", "bin", dict(depth=4, max_num_bin=2), None),
    "reg_logistic": (1200, 8, 8, "reg:logistic", "prob", dict(depth=4, max_num_bin=32), None),
    "softprob": (1500, 10, 8, "multi:softprob", "multi", dict(depth=3, max_num_bin=32), None),
    "wide_dense_blocks": (700, 150, 90, "reg:linear", "reg", dict(depth=4, max_num_bin=16), "dense"),
    "wide_dense_blocks_16_bit_bins": (700, 150, 90, "reg:linear", "reg", dict(depth=4, max_num_bin=16), "dense-16"),
    # blocks of 32 features (what small data with many bins per feature gets), and blocks of 64 features whose
    # histogram fills the LDS of a CU (what large wide data gets)
    "wide_dense_blocks_of_32": (700, 150, 90, "reg:linear", "reg", dict(depth=4, max_num_bin=16), "dense-w32"),
    "wide_dense_blocks_of_64_255_bins": (3000, 150, 90, "reg:linear", "reg", dict(depth=5, max_num_bin=255), "dense-w64"),
    "wide_sparse": (2500, 700, 12, "binary:logistic", "bin", dict(depth=5, max_num_bin=63), "sparse"),
    # the same through the kernel without an LDS head (every value goes to HBM atomics)
    "wide_sparse_no_head": (2500, 700, 12, "binary:logistic", "bin", dict(depth=5, max_num_bin=63), "sparse-nohead"),
    "lambda0_mcw5": (900, 6, 6, "reg:linear", "reg", dict(depth=4, max_num_bin=32, lambda_=0.0, min_child_weight=5.0),
                     None),
    "gamma_prunes_all": (600, 5, 5, "reg:linear", "reg", dict(depth=4, max_num_bin=16, gamma=1e9), None),
    # depth 12: the sparse layout leaves its level pass (12-bit node ids) for per-node histograms in HBM
    "sparse_depth12_per_node_path": (6000, 60, 8, "binary:logistic", "bin",
                                     dict(depth=12, max_num_bin=16, gamma=0.0, min_child_weight=0.05), "sparse"),
    "sparse_depth11_level_pass": (6000, 60, 8, "binary:logistic", "bin",
                                  dict(depth=11, max_num_bin=16, gamma=0.0, min_child_weight=0.05), "sparse"),
    # A node whose chosen candidate gains 0.8363545 with the missing rows sent left and 0.8363642 with them sent right
    # (86 missing rows, fourth round, class 3, node 12): the direction is a near tie between two gains of one
    # candidate and may fall either way within the 1e-5 tolerance; found by random-shape testing.
    "softmax_direction_near_tie_16_bit_bins": (4097, 8, 2, "multi:softmax", "multi", dict(depth=6, max_num_bin=8), "dense-16"),
    "softmax_direction_near_tie": (4097, 8, 2, "multi:softmax", "multi", dict(depth=6, max_num_bin=8), "dense"),
    # five labels of both signs whose mean is a hundredth of their size: the base score's 1e-5 is relative to the
    # labels, not to the mean (two float sums in different orders differ by 4e-7 here)
    "labels_cancel_in_the_base_score": (5, 60, 47, "reg:linear", "reg", dict(depth=4, max_num_bin=255), "sparse-nohead"),
    # a candidate whose right child's hessians add up to min_child_weight or one ulp less: with the three rows that
    # lack the feature it passes the gate on either side, without them on one side only, so the two sides take
    # different default directions with gains of 1.33 and 2.00
    "default_direction_on_the_min_child_weight_gate": (700, 5, 5, "binary:logistic", "bin", dict(depth=11, max_num_bin=8), "sparse-nohead"),
    # a node of gain 1.0000001 against 0.99999994 with gamma = 1: pruned on one side only
    "gain_on_the_pruning_threshold": (4097, 7, 6, "binary:logistic", "bin", dict(depth=9, max_num_bin=33), "sparse-nohead"),
}
CASE_SEEDS = {"softmax_direction_near_tie_16_bit_bins": 31479, "softmax_direction_near_tie": 31479,
              "labels_cancel_in_the_base_score": 80436, "default_direction_on_the_min_child_weight_gate": 73303,
              "gain_on_the_pruning_threshold": 71740}


@pytest.mark.parametrize("name", sorted(CASES))
def test_edge_case_matches_oracle(T, name):
    margins = P.Margins("edge/" + name)
    run_case(T, name, CASE_SEEDS.get(name, zlib.crc32(name.encode()) % 1000), margins)
    margins.report()


def test_random_small_cases(T):
    """150 seeded random shapes (rows 2..20000, 1..12 features, depth 1..6, 2..255 bins, every objective and
    layout) through the same teacher-forced comparison."""
    objs = [("reg:linear", "reg"), ("binary:logistic", "bin"), ("reg:logistic", "prob"), ("multi:softmax", "multi")]
    ran = 0
    margins = P.Margins("random_small_cases")
    for seed in range(1000, 1150):
        rng = np.random.default_rng(seed)
        n = int(rng.choice([2, 5, 17, 64, 65, 257, 700, 1500, 4097, 9000, 20000]))
        F = int(rng.integers(1, 13))
        depth = int(rng.integers(1, 7))
        bins = int(rng.choice([2, 3, 8, 33, 255]))
        objective, kind = objs[int(rng.integers(0, 4))]
        layout = [None, "dense", "sparse", "sparse-nohead"][int(rng.integers(0, 4))]
        if kind in ("bin", "multi") and n < 8:
            objective, kind = "reg:linear", "reg"
        case = (n, F, int(rng.integers(1, F + 1)), objective, kind, dict(depth=depth, max_num_bin=bins), layout)
        if len(_ragged(n, F, seed, case[2])[0]) == 0:
            continue  # a dataset without stored values aborts by design
        for k in ("TGBM_LAYOUT", "TGBM_CSR_HEAD"):
            os.environ.pop(k, None)
        try:
            run_case(T, case, seed, margins)
        except AssertionError as e:
            raise AssertionError("seed %d case %r: %s" % (seed, case, e))
        ran += 1
    margins.report()
    assert ran > 120


def test_random_small_cases_16_bit_bins(T):
    """40 more seeded random shapes through the dense layout with 16-bit bins (forced: the data has at most 255 bins
    per feature, so the oracle can follow), same teacher-forced comparison."""
    objs = [("reg:linear", "reg"), ("binary:logistic", "bin"), ("reg:logistic", "prob"), ("multi:softmax", "multi")]
    ran = 0
    margins = P.Margins("random_small_cases_16_bit_bins")
    for seed in range(3000, 3040):
        rng = np.random.default_rng(seed)
        n = int(rng.choice([5, 64, 65, 700, 4097, 9000, 20000]))
        F = int(rng.choice([1, 2, 3, 5, 9, 17, 40]))
        depth = int(rng.integers(1, 7))
        bins = int(rng.choice([2, 8, 33, 255]))
        objective, kind = objs[int(rng.integers(0, 4))]
        if kind in ("bin", "multi") and n < 8:
            objective, kind = "reg:linear", "reg"
        case = (n, F, int(rng.integers(1, F + 1)), objective, kind, dict(depth=depth, max_num_bin=bins), "dense-16")
        if len(_ragged(n, F, seed, case[2])[0]) == 0:
            continue
        try:
            run_case(T, case, seed, margins)
        except AssertionError as e:
            raise AssertionError("seed %d case %r: %s" % (seed, case, e))
        ran += 1
    margins.report()
    assert ran > 30


def run_case(T, name, seed, margins=None):
    n, F, max_len, objective, kind, kw, layout = CASES[name] if isinstance(name, str) else name
    if layout:
        os.environ["TGBM_LAYOUT"] = layout.split("-")[0]
        if layout.endswith("-nohead"):
            os.environ["TGBM_CSR_HEAD"] = "0"
        if layout.endswith("-16"):
            os.environ["TGBM_DENSE_BIN_BYTES"] = "2"
        if layout.endswith("-w32") or layout.endswith("-w64"):
            os.environ["TGBM_DENSE_W"] = layout[-2:]
    val, rp, col = _ragged(n, F, seed, max_len)
    y = _target(val, rp, col, n, F, seed, kind)
    rounds = 4
    kw = dict(kw, objective=objective, n_trees=rounds, learning_rate=0.5)
    lam = kw.get("lambda_", 1.0)
    s = T.Session(val, rp, col, y, **kw)
    if layout and layout.endswith("-16"):
        assert s.info("dense_bin_bytes") == 2
    if isinstance(name, str) and name.startswith("sparse_depth"):
        assert s.info("sparse") == 1 and s.info("sparse_pass") == (1 if kw["depth"] <= 11 else 0)
    if layout and layout[-4:] in ("-w32", "-w64"):
        assert s.info("dense_W") == int(layout[-2:])
    o = O.Oracle(val, rp, col, y, debug=True, **kw).prepare()
    # data preparation: exact
    cv, crp, cf = s.cuts()
    ocv, ocrp, ocf = o.cuts()
    assert np.array_equal(cv, ocv) and np.array_equal(crp, ocrp) and np.array_equal(cf, ocf)
    gb, _ = s.global_bin_ids(rp, col)
    assert np.array_equal(gb, o.bin_ids())
    assert np.array_equal(s.y(), o.y()) and np.array_equal(s.labels(), o.labels())
    # (a mean of labels of both signs: like every other sum, 1e-5 of the terms' absolute values, not of the result)
    np.testing.assert_allclose(s.base_score, o.base_score, rtol=1e-5, atol=1e-7 + 1e-5 * float(np.abs(y).mean()))
    present = np.zeros((n, s.F), bool)
    present[np.repeat(np.arange(n), np.diff(rp)), col] = True
    for r in range(rounds):
        o.set_y_pred(s.y_pred())
        s.gradient()
        gh = s.gh()  # the gradients this round is built from (boost recomputes the same values)
        s.boost(1)
        o.compute_gradient()
        np.testing.assert_allclose(gh, o.gh(), rtol=1e-5, atol=2e-7)
        o.set_gh(gh)
        model = s.model()
        tol = np.zeros(len(o.y_pred()))
        clean = True
        for k in range(s.tree_per_rounds):
            o.build_tree(k)
            final_nid = o.nid()
            ghk = np.abs(gh[k * n:(k + 1) * n].astype(np.float64)).sum(axis=0)
            d = P.compare_trees(model[r, k], o.nodes(), lam, crp=crp, orc_scores=o.tree_scores(), orc_dir_gaps=o.tree_dir_gaps(),
                                missing_rows=lambda x, f: int((~present[P.rows_in_node(final_nid, x), f]).sum()),
                                abs_scale=(ghk[0], ghk[1]), mcw=kw.get("min_child_weight", 1.0), gamma=kw.get("gamma", 1.0))
            clean &= not d.near_ties
            if margins is not None:
                margins.add(d)
                margins.ties += len(P.significant_ties(d.near_ties))
            sl = slice(k * n, (k + 1) * n)
            tol[sl] = P.pred_tolerance(o.nodes(), final_nid, 0.5, lam, (ghk[0], ghk[1]), o.y_pred()[sl])
        if clean:
            perr = np.abs(s.y_pred().astype(np.float64) - o.y_pred())
            assert np.all(perr <= tol)
            if margins is not None:
                margins.note("pred", perr, tol)
            assert np.array_equal(s.nid(), o.nid())
            # classification metrics count decisions: a row whose decision margin is inside the prediction
            # tolerance may fall on either side
            yp = o.y_pred().reshape(-1, n)
            if objective.startswith("multi:"):
                top = np.sort(yp, axis=0)
                flips = int((top[-1] - top[-2] <= 2 * tol.reshape(-1, n).max(axis=0)).sum())
            elif objective == "binary:logistic":
                flips = int((np.abs(yp[0]) <= 2 * tol).sum())
            else:
                flips = 0
            np.testing.assert_allclose(s.metric_log()[-1], o.metric(), rtol=1e-4, atol=1e-5 + flips / n)
    if name == "gamma_prunes_all":
        assert all(t[0]["is_leaf"] for rnd in s.model() for t in rnd)  # every tree collapsed into its root
    s.close()


@pytest.mark.parametrize("objective,kind", [("reg:linear", "reg"), ("binary:logistic", "bin"),
                                            ("reg:logistic", "prob")])
def test_one_boost_call_equals_round_by_round(T, objective, kind):
    """boost(6) ends every round with one fused pass (prediction update, metric, next gradients and their
    block statistics); the stage-wise calls run the separate kernels.
    Both must give the same bits."""
    n, F = 6000, 9
    val, rp, col = _ragged(n, F, 7, F)
    y = _target(val, rp, col, n, F, 7, kind)
    kw = dict(objective=objective, n_trees=6, depth=5, max_num_bin=32, learning_rate=0.3)
    a = T.Session(val, rp, col, y, **kw)
    a.boost(6)
    b = T.Session(val, rp, col, y, **kw)
    metrics = []
    for _ in range(6):
        b.gradient()
        b.tree_init(0)
        for level in range(5):
            b.find_split(level)
            b.partition(level)
        b.finish_tree(0)
        metrics.append(b.metric())
    assert a.model().tobytes() == b.model().tobytes()
    assert np.array_equal(a.y_pred(), b.y_pred())
    assert np.array_equal(a.metric_log(), np.array(metrics, np.float32))
    # the gradients left behind by the fused pass are those of the next round
    g_next = a.gh()
    b.gradient()
    assert np.array_equal(g_next, b.gh())
    a.close()
    b.close()


@pytest.mark.parametrize("layout", ["dense", "sparse"])
def test_class_trees_built_together_equal_one_by_one(T, layout):
    """The class trees of a softmax round are built by common launches (one buffer set per class); with
    TGBM_BATCH_CLASSES=0 they are built one after the other. Same bits either way, also through the
    stage-wise calls."""
    os.environ["TGBM_LAYOUT"] = layout
    n, F = 5000, 12
    val, rp, col = _ragged(n, F, 11, F)
    y = _target(val, rp, col, n, F, 11, "multi")
    kw = dict(objective="multi:softprob", n_trees=3, depth=5, max_num_bin=32, learning_rate=0.4)
    a = T.Session(val, rp, col, y, **kw)
    assert a.info("n_sets") == 4
    a.boost(3)
    os.environ["TGBM_BATCH_CLASSES"] = "0"
    b = T.Session(val, rp, col, y, **kw)
    assert b.info("n_sets") == 1
    b.boost(3)
    os.environ.pop("TGBM_BATCH_CLASSES")
    c = T.Session(val, rp, col, y, **kw)
    for _ in range(3):
        c.gradient()
        for k in range(4):
            c.tree_init(k)
            for level in range(5):
                c.find_split(level)
                c.partition(level)
            c.finish_tree(k)
    ma = a.model().tobytes()
    assert ma == b.model().tobytes() and ma == c.model().tobytes()
    assert np.array_equal(a.y_pred(), b.y_pred()) and np.array_equal(a.y_pred(), c.y_pred())
    assert np.array_equal(a.metric_log(), b.metric_log())
    for s in (a, b, c):
        s.close()


@pytest.mark.parametrize("objective,kind,rate", [("reg:linear", "reg", 0.5), ("binary:logistic", "bin", 0.3),
                                                 ("multi:softmax", "multi", 0.7), ("reg:linear", "reg", 0.05)])
def test_column_sampling_matches_oracle(T, objective, kind, rate):
    """column_sampling_rate < 1: every round ignores max(1, int(F * rate)) shuffled columns. The library
    restates libstdc++'s std::random_shuffle over the process-wide rand(); the oracle calls
    std::random_shuffle itself. Both are started from the same srand() seed; whole boosting runs (no
    teacher forcing) must then pick the same columns and build the same trees."""
    import ctypes
    libc = ctypes.CDLL(None)
    n, F = 3000, 11
    val, rp, col = _ragged(n, F, 21, F)
    y = _target(val, rp, col, n, F, 21, kind)
    kw = dict(objective=objective, n_trees=5, depth=4, max_num_bin=32, learning_rate=0.5)
    s = T.Session(val, rp, col, y, **kw)
    s.set_option("column_sampling_rate", rate)
    o = O.Oracle(val, rp, col, y, debug=True, **kw).prepare()
    o.set_column_sampling_rate(rate)
    n_ignored = max(1, int(F * rate))
    for r in range(5):
        o.set_y_pred(s.y_pred())
        s.gradient()
        gh = s.gh()
        libc.srand(1234 + r)
        s.boost(1)
        libc.srand(1234 + r)
        o.sample_columns()
        o.compute_gradient()
        o.set_gh(gh)
        model = s.model()
        used = set()
        for k in range(s.tree_per_rounds):
            o.build_tree(k)
            ghk = np.abs(gh[k * n:(k + 1) * n].astype(np.float64)).sum(axis=0)
            d = P.compare_trees(model[r, k], o.nodes(), 1.0, crp=s.cuts()[1], orc_scores=o.tree_scores(), orc_dir_gaps=o.tree_dir_gaps(),
                                abs_scale=(ghk[0], ghk[1]))
            assert not P.significant_ties(d.near_ties)
            nodes = model[r, k]
            used |= set(int(f) for f in nodes["split_fid"][(nodes["is_valid"] == 1) & (nodes["split_fid"] >= 0)])
        assert len(used) <= F - n_ignored  # the round's trees only split on columns that were not ignored
    s.close()


@pytest.mark.parametrize("objective,kind,reorder", [("reg:linear", "reg", False), ("binary:logistic", "bin", False),
                                                    ("multi:softmax", "multi", False), ("reg:linear", "reg", True),
                                                    ("binary:logistic", "bin", True), ("multi:softmax", "multi", True)])
def test_bagging_matches_oracle(T, objective, kind, reorder):
    """bagging = 1 (RowSampler::do_bagging, row_sampler.cu:9-38; booster.h:84): every round multiplies the
    gradient pairs by bootstrap draw counts from thrust's minstd engine seeded with one rand(). The draw
    counts must be the oracle's exactly (integer work), and boosting on the bagged gradients must build the
    oracle's trees."""
    import ctypes
    libc = ctypes.CDLL(None)
    libc.rand.restype = ctypes.c_int
    n, F = 3000, 9
    val, rp, col = _ragged(n, F, 33, F)
    y = _target(val, rp, col, n, F, 33, kind)
    # min_child_weight 0.5: the bagged hessians of squared loss are whole numbers, so child sums would sit
    # exactly on a gate of 1 and candidates that isolate the same rows through different features would tie
    kw = dict(objective=objective, n_trees=4, depth=4, max_num_bin=32, learning_rate=0.5, min_child_weight=0.5)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, debug=True, **kw).prepare()
    if reorder:  # the draw counts belong to the caller's row indices, also after the rows were re-ordered
        for key, v in (("reorder_min_rows", 0), ("reorder_first", 1), ("reorder_every", 1)):
            s.set_option(key, v)
    s.gradient()
    plain = s.gh().copy()
    s.set_option("bagging", 1)
    o.set_bagging(True)
    N = plain.shape[0]
    assert N == s.num_class * n  # the whole gradient array is resampled, as in the reference
    for seed in (7, 8):
        libc.srand(seed)
        draw_seed = libc.rand()
        libc.srand(seed)
        s.gradient()
        counts = np.bincount(O.bagging_draws(draw_seed, N), minlength=N).astype(np.float32)
        assert np.array_equal(s.gh(), plain * counts[:, None])
    ties = 0
    for r in range(4):
        o.set_y_pred(s.y_pred())
        libc.srand(100 + r)
        s.gradient()
        gh = s.gh()
        libc.srand(100 + r)
        o.compute_gradient()
        np.testing.assert_allclose(gh, o.gh(), rtol=1e-5, atol=2e-6)
        o.set_gh(gh)
        libc.srand(100 + r)
        s.boost(1)
        model = s.model()
        for k in range(s.tree_per_rounds):
            o.build_tree(k)
            ghk = np.abs(gh[k * n:(k + 1) * n].astype(np.float64)).sum(axis=0)
            d = P.compare_trees(model[r, k], o.nodes(), 1.0, crp=s.cuts()[1], orc_scores=o.tree_scores(), orc_dir_gaps=o.tree_dir_gaps(),
                                abs_scale=(ghk[0], ghk[1]), mcw=0.5)
            ties += len(P.significant_ties(d.near_ties))
    # rows drawn zero times carry no weight, so neighbouring candidates can describe the same partition;
    # compare_trees has checked that every differing choice is such a tie in the oracle's own gains
    assert ties <= 3
    assert s.info("reorders_done") == (4 if reorder else 0)
    if reorder:  # counts after re-orderings: still per original row
        s.gradient()  # plain gradients are not available any more; check through the oracle instead
        libc.srand(55)
        o.set_y_pred(s.y_pred())
        o.compute_gradient()
        libc.srand(55)
        s.gradient()
        np.testing.assert_allclose(s.gh(), o.gh(), rtol=1e-5, atol=2e-6)
    s.close()


def test_bagging_through_the_c_abi(T):
    """The bagging argument of sparse_train_scikit: same srand() seed, same model; without bagging another."""
    import ctypes
    libc = ctypes.CDLL(None)
    rng = np.random.default_rng(4)
    X = rng.standard_normal((2000, 6)).astype(np.float32)
    y = (X[:, 0] - X[:, 1] + 0.3 * rng.standard_normal(2000)).astype(np.float32)
    preds = []
    # the first GPU call of a process initialises the runtime, which may draw from rand() itself
    T.TGBMRegressor(depth=2, n_trees=1, verbose=0).fit(X, y)
    for bagging, seed in ((1, 5), (1, 5), (1, 6), (0, 5)):
        libc.srand(seed)
        m = T.TGBMRegressor(depth=4, n_trees=6, learning_rate=0.5, bagging=bagging, verbose=0).fit(X, y)
        preds.append(np.asarray(m.predict(X), np.float32).copy())
    assert np.array_equal(preds[0], preds[1])
    assert not np.array_equal(preds[0], preds[2])
    assert not np.array_equal(preds[0], preds[3])
    assert np.sqrt(np.mean((preds[0] - y) ** 2)) < 0.8 * np.std(y)  # still learns


def test_sessions_release_their_device_memory(T):
    """Every layout's session (dense with row re-ordering, sparse, ranking, class trees built together) gives
    its device memory back when it is closed: free memory after ten open/boost/close cycles is what it was."""
    rng = np.random.default_rng(12)
    n = 1_200_000  # above the row count from which rows are re-ordered
    X = rng.standard_normal((n, 6)).astype(np.float32)
    y = (X[:, 0] - X[:, 1] > 0).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    ym = rng.integers(0, 3, n).astype(np.float32)
    yr = rng.integers(0, 4, n).astype(np.float32)
    groups = np.full(n // 100, 100, np.int32)

    def cycle():
        s = T.Session(val, rp, col, y, depth=4, n_trees=4, objective="binary:logistic")
        s.boost(4)
        assert s.info("reorders_done") >= 1
        free = s.info("device_free_mb")
        s.close()
        os.environ["TGBM_LAYOUT"] = "sparse"
        s = T.Session(val, rp, col, y, depth=4, n_trees=2, objective="binary:logistic")
        s.boost(2)
        s.close()
        os.environ.pop("TGBM_LAYOUT")
        s = T.Session(val, rp, col, ym, depth=4, n_trees=2, objective="multi:softmax", num_class=3)
        s.boost(2)
        s.close()
        s = T.Session(val, rp, col, yr, depth=4, n_trees=2, objective="rank:ndcg", groups=groups)
        s.boost(2)
        s.close()
        return free

    first = cycle()
    for _ in range(9):
        last = cycle()
    assert abs(first - last) <= 64, (first, last)


def test_fits_from_two_threads_are_serialised(T):
    """sparse_train_scikit / sparse_predict_scikit hold a process-wide lock (the reference serialises
    Booster::boost with a global mutex, booster.h:17,78): four threads fitting and predicting at once get the
    models and predictions of the same calls made one after the other."""
    import threading
    rng = np.random.default_rng(8)
    sets = []
    for i in range(4):
        X = rng.standard_normal((3000 + 500 * i, 5 + i)).astype(np.float32)
        y = (X[:, 0] * (i + 1) - X[:, 1] + 0.2 * rng.standard_normal(len(X))).astype(np.float32)
        sets.append((X, y))
    fit = lambda X, y: np.asarray(T.TGBMRegressor(depth=5, n_trees=8, learning_rate=0.4, verbose=0).fit(X, y).predict(X),
                                  np.float32).copy()
    serial = [fit(X, y) for X, y in sets]
    out = [None] * 4

    def work(i):
        out[i] = fit(*sets[i])

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for a, b in zip(serial, out):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("objective,kind", [("reg:linear", "reg"), ("binary:logistic", "bin"),
                                            ("multi:softmax", "multi")])
def test_row_reordering_is_invisible(T, objective, kind):
    """boost() physically re-orders the rows by the leaves of a tree every few rounds (here: after every
    round) so that the rows of a node lie together. Histograms and root sums are exact integer sums, so the
    trees must not change in any bit, and everything handed out per row must stay in the caller's row order."""
    n, F = 30000, 40  # 40 features: two feature blocks
    val, rp, col = _ragged(n, F, 9, F)
    y = _target(val, rp, col, n, F, 9, kind)
    kw = dict(objective=objective, n_trees=7, depth=6, max_num_bin=64, learning_rate=0.3)
    runs = []
    for first, every in ((0, 0), (1, 1), (2, 3)):
        s = T.Session(val, rp, col, y, **kw)
        s.set_option("reorder_min_rows", 0)
        s.set_option("reorder_first", first)
        s.set_option("reorder_burst", 1)
        s.set_option("reorder_every", every)
        before = s.binmat().copy()
        s.boost(7)
        assert s.info("reorders_done") == {0: 0, 1: 7, 2: 2}[first]
        runs.append(dict(model=s.model().copy(), yp=s.y_pred().copy(), nid=s.nid().copy(), y=s.y().copy(),
                         binmat=s.binmat().copy(), metric=s.metric_log().copy(), before=before))
        s.close()
    base = runs[0]
    for r in runs[1:]:
        assert np.array_equal(r["y"], base["y"]) and np.array_equal(r["binmat"], base["binmat"])
        assert np.array_equal(r["before"], r["binmat"])
        # Every sum a tree is made of is an exact integer sum (the root's included, which replaces the float
        # reduction over the rows): the whole model - sums, weights, gains, default directions - and the
        # predictions are the same bits in any row order. Only the metric is a float reduction over the rows.
        assert r["model"].tobytes() == base["model"].tobytes()
        assert np.array_equal(r["nid"], base["nid"])
        assert np.array_equal(r["yp"], base["yp"])
        np.testing.assert_allclose(r["metric"], base["metric"], rtol=1e-5)


def test_row_reordering_then_stagewise_and_setters(T):
    """After a re-ordering, the stage-wise calls, set("y_pred") / set("gh") and the row lists still speak the
    caller's row order: a lock-step tree against the oracle on top of re-ordered rows."""
    n, F = 20000, 6
    val, rp, col = _ragged(n, F, 12, F)
    y = _target(val, rp, col, n, F, 12, "reg")
    kw = dict(objective="reg:linear", n_trees=5, depth=5, max_num_bin=32, learning_rate=0.5)
    s = T.Session(val, rp, col, y, **kw)
    for key, v in (("reorder_min_rows", 0), ("reorder_first", 1), ("reorder_every", 1)):
        s.set_option(key, v)
    s.boost(2)
    assert s.info("reorders_done") == 2
    o = O.Oracle(val, rp, col, y, debug=True, **kw).prepare()
    o.set_y_pred(s.y_pred())
    o.compute_gradient()
    s.gradient()
    gh = s.gh()
    np.testing.assert_allclose(gh, o.gh(), rtol=1e-5, atol=2e-7)
    s.set("gh", gh)  # round trip through the permutation
    assert np.array_equal(s.gh(), gh)
    o.set_gh(gh)
    s.tree_init(0)
    o.tree_init(0)
    for level in range(5):
        s.find_split(level)
        o.find_split(level)
        o.update_tree()
        o.set_nodes(s.nodes())  # both sides apply the same splits (near ties are the other tests' subject)
        s.partition(level)
        o.update_ins2node()
        assert np.array_equal(s.nid(), o.nid()), level
        if level < 4:  # the row lists name rows by the caller's ids
            seg = s.get("seg", np.int32, (-1, 2))
            lists = s.get("ridx%d" % ((level + 1) & 1), np.int32)
            nid = s.nid()
            for x in range((1 << (level + 1)) - 1, (1 << (level + 2)) - 1):
                a, b = seg[x]
                if b > a:
                    assert np.array_equal(np.sort(lists[a:b]), np.flatnonzero(nid == x))
    s.finish_tree(0)
    s.close()


@pytest.mark.parametrize("layout", ["dense", "sparse"])
def test_training_is_bit_reproducible(T, layout):
    """Histograms are exact integer sums (LDS and HBM atomics alike) and every float reduction has a fixed
    order, so two runs on the same input give the same bytes - which the reference's float atomics do not."""
    os.environ["TGBM_LAYOUT"] = layout
    n, F = 40000, 20
    val, rp, col = _ragged(n, F, 5, F)
    y = _target(val, rp, col, n, F, 5, "bin")
    kw = dict(objective="binary:logistic", n_trees=8, depth=6, max_num_bin=64, learning_rate=0.3)
    runs = []
    for _ in range(3):
        s = T.Session(val, rp, col, y, **kw)
        s.boost(8)
        runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.metric_log().tobytes()))
        s.close()
    assert runs[0] == runs[1] == runs[2]


@pytest.mark.parametrize("head", ["1", "0"])
@pytest.mark.parametrize("objective,kind", [("binary:logistic", "bin"), ("multi:softmax", "multi")])
def test_sparse_root_histogram_from_either_copy(T, objective, kind, head):
    """Sparse layout: the level pass over the bin-major copy (tables in LDS, no per-node histogram in HBM) and the
    row-list kernels with per-node histograms (TGBM_SPARSE_PASS=0; root from the bin-major copy or row by row with
    atomics, TGBM_CSC_ROOT; with and without the LDS head) sum the same integers: same root histogram, same model,
    same predictions, byte for byte."""
    os.environ["TGBM_LAYOUT"] = "sparse"
    os.environ["TGBM_CSR_HEAD"] = head
    n, F = 30000, 300
    val, rp, col = _ragged(n, F, 9, 12)
    y = _target(val, rp, col, n, F, 9, kind)
    kw = dict(objective=objective, n_trees=4, depth=5, max_num_bin=16, learning_rate=0.3)
    if kind == "multi":
        kw["num_class"] = int(y.max()) + 1
    runs = []
    try:
        for level_pass, csc, srt in (("1", "1", "1"), ("1", "1", "0"), ("0", "1", "1"), ("0", "0", "1")):
            os.environ["TGBM_SPARSE_PASS"] = level_pass
            os.environ["TGBM_CSC_ROOT"] = csc
            os.environ["TGBM_SPARSE_SORTED"] = srt  # "0": every feature through the (bin, node) tables
            s = T.Session(val, rp, col, y, **kw)
            assert s.info("sparse_pass") == int(level_pass)
            s.gradient()
            s.tree_init(0)
            s.find_split(0)
            root_hist = s.level_hist(0).tobytes()
            s.close()
            s = T.Session(val, rp, col, y, **kw)
            s.boost(4)
            runs.append((root_hist, s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        os.environ.pop("TGBM_CSC_ROOT", None)
        os.environ.pop("TGBM_SPARSE_PASS", None)
        os.environ.pop("TGBM_SPARSE_SORTED", None)
    assert runs[0] == runs[1] == runs[2] == runs[3]


@pytest.mark.parametrize("mcw,gamma", [(1.0, 0.0), (40.0, 0.0), (1.0, 30.0)])
def test_sparse_sorted_pass_equals_table_pass_on_deep_uneven_trees(T, mcw, gamma):
    """Sparse level pass: features of a few thousand values are searched through their values kept sorted by
    (feature, node, bin) from level to level, the frequent ones through (bin, node) tables; TGBM_SPARSE_SORTED=0
    sends every feature through the tables. Same integers either way: identical models, predictions and row -> node
    maps, on trees whose nodes stop at different levels (min_child_weight) and with frequent and rare features
    mixed (a few columns in nearly every row, many in a handful of rows)."""
    os.environ["TGBM_LAYOUT"] = "sparse"
    rng = np.random.default_rng(21)
    n, F = 40000, 900
    # Zipf-like column usage: columns 0..5 in most rows (more than one tile of values), the rest rare
    cols = []
    rp = np.zeros(n + 1, np.int32)
    for i in range(n):
        c = set(np.flatnonzero(rng.random(6) < 0.7).tolist())
        c.update((6 + rng.integers(0, F - 6, rng.integers(0, 7))).tolist())
        cols.append(np.sort(np.fromiter(c, np.int32, len(c))))
        rp[i + 1] = rp[i] + len(c)
    col = np.concatenate(cols).astype(np.int32)
    val = rng.lognormal(0, 1, len(col)).astype(np.float32)
    y = _target(val, rp, col, n, F, 21, "bin")
    kw = dict(objective="binary:logistic", n_trees=5, depth=8, max_num_bin=32, learning_rate=0.4,
              min_child_weight=mcw, gamma=gamma)
    runs = []
    try:
        # (TGBM_SPARSE_COLS=0: the row -> node update searches every row's bin ids instead of reading the frequent
        # features' byte columns)
        for srt, cols in (("1", "1"), ("0", "1"), ("1", "0")):
            os.environ["TGBM_SPARSE_SORTED"] = srt
            os.environ["TGBM_SPARSE_COLS"] = cols
            s = T.Session(val, rp, col, y, **kw)
            assert s.info("sparse_pass") == 1
            s.boost(5)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        os.environ.pop("TGBM_SPARSE_SORTED", None)
        os.environ.pop("TGBM_SPARSE_COLS", None)
    assert runs[0] == runs[1] == runs[2]


def test_predict_transforms_through_the_c_abi(T):
    """sparse_predict_scikit for every objective against the oracle's predictor + transform on unseen rows."""
    n, F = 1500, 7
    val, rp, col = _ragged(n, F, 5, 7)
    tv, trp, tc = _ragged(400, F, 6, 7)
    for objective, kind, cls in (("reg:linear", "reg", "r"), ("reg:logistic", "prob", "r"),
                                 ("binary:logistic", "bin", "c"), ("multi:softmax", "multi", "c"),
                                 ("multi:softprob", "multi", "c")):
        y = _target(val, rp, col, n, F, 5, kind)
        import scipy.sparse as sp
        X = sp.csr_matrix((val, col, rp), shape=(n, F))
        Xt = sp.csr_matrix((tv, tc, trp), shape=(400, F))
        Est = T.TGBMRegressor if cls == "r" else T.TGBMClassifier
        m = Est(depth=4, n_trees=6, learning_rate=0.4, objective=objective, verbose=0, max_num_bin=32).fit(X, y)
        got = np.asarray(m.predict(Xt)).ravel()
        o = O.Oracle(val, rp, col, y, depth=4, n_trees=6, learning_rate=0.4, objective=objective, max_num_bin=32,
                     num_class=2).prepare()
        o.boost(6)
        raw = O.predict_raw(tv, trp, tc, F, o.model(), 0.4, 0.0)  # the C-API path has no base score
        labels = o.labels() if cls == "c" else np.zeros(1, np.float32)
        exp = O.predict_transform(objective, raw, 400, o.num_class, labels)
        if objective in ("binary:logistic", "multi:softmax"):
            assert np.mean(got == exp) > 0.99
        else:
            np.testing.assert_allclose(got, exp, rtol=1e-4, atol=1e-5)


def test_negative_column_index_is_rejected_before_any_kernel_uses_it(T):
    """The C ABI takes the caller's column indices as they are; the largest and smallest are taken on the device
    right after the upload, and a negative one (e.g. a 0-based file read as 1-based) stops the call with a
    message instead of indexing device memory with it. Runs in a child process: the library aborts like the
    reference's CHECK."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import ctypes as C, sys\nimport numpy as np\nsys.path.insert(0, %r)\nimport thundergbm_amd\n"
        "L = thundergbm_amd.load()\n"
        "val = np.ones(6, np.float32); col = np.array([0, 1, -1, 1, 0, 2], np.int32)\n"
        "rp = np.array([0, 2, 4, 6], np.int32); y = np.zeros(3, np.float32)\n"
        "p = lambda a: a.ctypes.data_as(C.c_void_p)\n"
        "L.tgbm_trainer_create_grouped(3, p(val), p(rp), p(col), p(y), 3, 1, 1.0, 1.0, 1.0, 16, 1.0, b'reg:linear',"
        " 1, 0, None, 0)\n" % root)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode != 0 and "negative column index -1" in out.stderr, out.stderr


@pytest.mark.parametrize("layout,objective,kind", [("dense", "reg:linear", "reg"), ("dense", "multi:softmax", "multi"),
                                                    ("sparse", "binary:logistic", "bin")])
def test_capped_histogram_arena_gives_the_same_trees(T, layout, objective, kind):
    """The per-node histogram paths keep the node histograms of two levels; when the deepest level does not fit the
    free memory the arena is capped and deeper levels are built in batches of nodes (the first such level still by
    subtraction from its parents, the ones below with both siblings from rows), as the reference does beyond its
    max_trick_depth (hist_tree_builder_single.cu:811-832, :544-570). TGBM_HIST_ARENA_NODES forces a small arena:
    histograms are exact integer sums, so the trees, predictions and row -> node maps are the same bytes wherever a
    row counts the same in every node (integer hessians with wide gradient fields, the sparse layout)."""
    os.environ["TGBM_LAYOUT"] = layout
    os.environ["TGBM_SPARSE_PASS"] = "0"  # the sparse layout's per-node path (the level pass has no arena)
    n, F = 20000, 12
    val, rp, col = _ragged(n, F, 31, 9)
    y = _target(val, rp, col, n, F, 31, kind)
    kw = dict(objective=objective, n_trees=3, depth=7, max_num_bin=32, learning_rate=0.5, min_child_weight=1.0, gamma=0.0)
    if kind == "multi":
        kw["num_class"] = int(y.max()) + 1
    runs = []
    try:
        for cap in (None, "4", "16"):
            if cap is None:
                os.environ.pop("TGBM_HIST_ARENA_NODES", None)
            else:
                os.environ["TGBM_HIST_ARENA_NODES"] = cap
            s = T.Session(val, rp, col, y, **kw)
            s.boost(3)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        os.environ.pop("TGBM_HIST_ARENA_NODES", None)
        os.environ.pop("TGBM_SPARSE_PASS", None)
    if kind == "multi":
        # float hessians in packed 32 + 32-bit LDS bins: a dense work item counts at a scale that depends on its
        # node's row count, so a sibling built from its own rows and one derived as parent - built differ by
        # roundings far below the 1e-5 tolerance - not bit for bit. Same structure, predictions within 1e-4.
        ref = np.frombuffer(runs[0][1], np.float32)
        for r in runs[1:]:
            np.testing.assert_allclose(np.frombuffer(r[1], np.float32), ref, rtol=1e-4, atol=1e-4)
            assert np.mean(np.frombuffer(r[2], np.int32) == np.frombuffer(runs[0][2], np.int32)) > 0.999
        return
    same = [[a == b for a, b in zip(runs[0], r)] for r in runs[1:]]  # (model, predictions, row -> node map)
    assert same == [[True] * 3] * 2, same


@pytest.mark.parametrize("layout", ["sparse", "dense"])
def test_split_search_per_feature_and_node_equals_the_packed_one(T, layout):
    """The split search for features of any number of bins (one workgroup per (feature, node), chunks of 256 bins
    with a carried prefix) against the packed one (a wavefront per run of whole features of at most 256 bins) on
    data both can serve: same candidates, gains and tie rule, so the same bytes. TGBM_WIDE_EVAL=1 switches it on
    for the dense layout and the CSR layout's per-node path."""
    os.environ["TGBM_LAYOUT"] = layout
    os.environ["TGBM_SPARSE_PASS"] = "0"
    n, F = 6000, 9
    val, rp, col = _ragged(n, F, 41, 8)
    runs = []
    try:
        for objective, kind in (("reg:linear", "reg"), ("binary:logistic", "bin")):
            y = _target(val, rp, col, n, F, 41, kind)
            for wide in ("0", "1"):
                os.environ["TGBM_WIDE_EVAL"] = wide
                s = T.Session(val, rp, col, y, objective=objective, n_trees=4, depth=6, max_num_bin=200, learning_rate=0.4,
                              gamma=0.0)
                assert s.info("wide_eval") == int(wide)
                s.boost(4)
                runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
                s.close()
    finally:
        os.environ.pop("TGBM_WIDE_EVAL", None)
        os.environ.pop("TGBM_SPARSE_PASS", None)
    assert [a == b for a, b in zip(runs[0], runs[1])] == [True] * 3
    assert [a == b for a, b in zip(runs[2], runs[3])] == [True] * 3


@pytest.mark.parametrize("layout,max_bins", [("dense", 1024), ("dense", 3000), ("dense", 6000), ("sparse", 1024)])
def test_more_than_255_bins_per_feature(T, layout, max_bins):
    """max_num_bin above 255 (the reference cannot go there: its split bin is a byte, include/thundergbm/tree.h:23,
    so there is nothing to compare a tree with): the dense layout keeps 16-bit bins, the CSR layout's global bin ids
    carry any number of bins per feature anyway (1024 bins: eight features per block of the dense layout; 3000: two,
    with two histogram workgroups per CU; 6000: two, with one). Checked for both: cut points and bin ids against the oracle's
    restatement of the cut rule (bit-exact, it has no such limit), every row's final node against a walk down the tree
    by the raw feature values and the stored thresholds, the training prediction against the sum of the leaf values
    along those walks, the hessian sums of the final nodes against a count of the rows that arrived, and a loss that
    goes down."""
    os.environ["TGBM_LAYOUT"] = layout
    rng = np.random.default_rng(7)
    n, F = 8000, 5
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.1] = 0.0  # zeros are not stored: missing values
    val, rp, col = D.dense_to_csr(X)
    y = (np.sin(2 * X[:, 0]) + X[:, 1] * X[:, 2] + 0.1 * rng.standard_normal(n)).astype(np.float32)
    lr, depth, rounds = 0.3, 6, 6
    s = T.Session(val, rp, col, y, objective="reg:linear", n_trees=rounds, depth=depth, max_num_bin=max_bins,
                  learning_rate=lr, gamma=0.0)
    assert s.info("wide_bins") == 1 and s.info("wide_eval") == 1
    if layout == "dense":
        assert s.info("sparse") == 0 and s.info("dense_bin_bytes") == 2
    else:
        assert s.info("sparse") == 1
    cut_val, crp, cut_fid = s.cuts()
    assert np.diff(crp).max() > max_bins // 2 and np.diff(crp).max() <= max_bins
    o_val, o_crp, o_fid = O.cut_points(val, col, F, max_bins)
    assert np.array_equal(crp, o_crp) and np.array_equal(cut_val, o_val) and np.array_equal(cut_fid, o_fid)
    gb, local = s.global_bin_ids(rp, col)
    assert np.array_equal(gb, O.bin_ids(val, col, o_val, o_crp))
    assert local.max() > 255
    if layout == "dense":  # a feature without a stored value in a row holds the 16-bit sentinel
        m = s.binmat()
        W = s.info("dense_W")
        dense = np.concatenate([m[b] for b in range(m.shape[0])], axis=1)[:, :F]
        assert m.dtype == np.uint16 and np.array_equal(dense == 65535, X == 0)
    base = float(s.base_score)
    s.boost(rounds)
    log = s.metric_log()
    assert np.all(np.diff(log) < 0)
    model = s.model()[:, 0, :]
    nid = s.nid()
    Xm = np.where(X == 0, np.nan, X)
    pred = np.full(n, base, np.float64)
    for t in range(rounds):
        nodes = model[t]
        cur = np.zeros(n, np.int64)
        for _ in range(depth):
            nd = nodes[cur]
            stop = (nd["is_leaf"] == 1) | (nd["split_fid"] < 0)
            v = Xm[np.arange(n), np.maximum(nd["split_fid"], 0)]
            right = np.where(np.isnan(v), nd["default_right"] == 1, v >= nd["split_value"])
            cur = np.where(stop, cur, np.where(right, nd["rch"], nd["lch"]))
        assert not nodes["is_pruned"].any()  # gamma = 0: nothing is pruned, a row's weight is its final node's
        if t == rounds - 1:
            np.testing.assert_array_equal(nid, cur)
            # node sums of the nodes that hold rows against an fp64 recount of unit hessians (squared loss)
            cnt = np.bincount(cur, minlength=len(nodes))
            held = cnt > 0
            np.testing.assert_allclose(nodes["sum_h"][held], cnt[held], rtol=1e-6)
        pred += lr * nodes["base_weight"].astype(np.float64)[cur]
    np.testing.assert_allclose(s.y_pred(), pred, rtol=1e-4, atol=1e-4)
    s.close()


def test_dense_layout_keeps_the_later_of_two_entries_with_the_same_column(T):
    """Rows that store a column twice (not something the wrappers produce: they sort and merge columns) - the dense
    bin matrix has one cell per (row, feature) and keeps the bin of the later entry, in both bin widths."""
    rng = np.random.default_rng(3)
    n, F = 500, 6
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[X == 0] = 0.5
    val, rp, col = D.dense_to_csr(X)
    # every third row gets a second entry for column 2 right after the first, with another value
    vals, cols, ptr = [], [], [0]
    for r in range(n):
        v, c = list(val[rp[r]:rp[r + 1]]), list(col[rp[r]:rp[r + 1]])
        if r % 3 == 0:
            k = c.index(2)
            v.insert(k + 1, np.float32(-v[k]))
            c.insert(k + 1, 2)
        vals += v
        cols += c
        ptr.append(len(vals))
    val2, col2, rp2 = np.array(vals, np.float32), np.array(cols, np.int32), np.array(ptr, np.int32)
    y = X[:, 0].copy()
    os.environ["TGBM_LAYOUT"] = "dense"
    for nbytes in ("1", "2"):
        os.environ["TGBM_DENSE_BIN_BYTES"] = nbytes
        s = T.Session(val2, rp2, col2, y, objective="reg:linear", n_trees=1, depth=3, max_num_bin=32)
        cut_val, crp, _ = s.cuts()
        m = s.binmat()
        dense = np.concatenate([m[b] for b in range(m.shape[0])], axis=1)[:, :F].astype(np.int64)
        later = np.where(np.arange(n) % 3 == 0, -X[:, 2], X[:, 2])
        cuts2 = cut_val[crp[2]:crp[3]]
        # the bin rule (hist_tree_builder_single.cu:81-119): number of cut points <= value, at most k - 1
        expect = np.minimum((cuts2[None, :] <= later[:, None]).sum(axis=1), len(cuts2) - 1)
        assert np.array_equal(dense[:, 2], expect)
        s.close()
    os.environ.pop("TGBM_DENSE_BIN_BYTES", None)


def test_dense_layout_with_unsorted_rows_that_repeat_a_column(T):
    """Rows whose columns do not ascend and that store a column twice with other entries in between: the later entry
    counts, the same bins on every run (sixteen lanes share a row of sorted data; such rows are filled by one thread
    each, front to back)."""
    rng = np.random.default_rng(8)
    n, F = 3000, 9
    vals, cols, ptr, later = [], [], [0], np.zeros((n, F), np.float32)
    for r in range(n):
        c = list(rng.permutation(F)[: int(rng.integers(3, F + 1))])
        c += [c[0]] * int(rng.integers(0, 2))  # sometimes the first column once more at the end
        v = list(np.round(rng.standard_normal(len(c)) * 2, 1).astype(np.float32) + np.float32(0.05))
        for cc, vv in zip(c, v):
            later[r, cc] = vv
        cols += c
        vals += v
        ptr.append(len(cols))
    val, col, rp = np.array(vals, np.float32), np.array(cols, np.int32), np.array(ptr, np.int32)
    y = later[:, 0].copy()
    os.environ["TGBM_LAYOUT"] = "dense"
    mats = []
    for nbytes in ("1", "2", "1"):
        os.environ["TGBM_DENSE_BIN_BYTES"] = nbytes
        s = T.Session(val, rp, col, y, objective="reg:linear", n_trees=1, depth=3, max_num_bin=32)
        cut_val, crp, _ = s.cuts()
        m = s.binmat()
        dense = np.concatenate([m[b] for b in range(m.shape[0])], axis=1)[:, :F].astype(np.int64)
        for f in range(F):
            cf = cut_val[crp[f]:crp[f + 1]]
            expect = np.minimum((cf[None, :] <= later[:, f][:, None]).sum(axis=1), len(cf) - 1)
            stored = later[:, f] != 0
            assert np.array_equal(dense[stored, f], expect[stored]), f
            assert np.all(dense[~stored, f] == (255 if nbytes == "1" else 65535))
        s.boost(1)
        mats.append((dense, s.model().tobytes()))
        s.close()
    os.environ.pop("TGBM_DENSE_BIN_BYTES", None)
    assert np.array_equal(mats[0][0], mats[2][0]) and mats[0][1] == mats[2][1]


def test_dense_16_bit_bins_with_sampling_and_a_capped_arena(T):
    """The 16-bit layout under the options that change which rows and columns a tree sees (bagging, column sampling;
    same srand() seed for every run) and with a capped histogram arena (nodes in batches): same models, predictions
    and row -> node maps as the byte layout, byte for byte."""
    import ctypes
    libc = ctypes.CDLL(None)
    os.environ["TGBM_LAYOUT"] = "dense"
    rng = np.random.default_rng(21)
    n, F = 20000, 9
    X = np.round(rng.standard_normal((n, F)) * 2, 1).astype(np.float32)
    X[rng.random((n, F)) < 0.2] = 0.0
    val, rp, col = D.dense_to_csr(X)
    y = (X[:, 0] + X[:, 3] * X[:, 4] + 0.5 * rng.standard_normal(n)).astype(np.float32)  # squared loss: integer hessians
    runs = []
    try:
        for nbytes, cap in (("1", None), ("2", None), ("2", "4")):
            os.environ["TGBM_DENSE_BIN_BYTES"] = nbytes
            os.environ.pop("TGBM_HIST_ARENA_NODES", None)
            if cap:
                os.environ["TGBM_HIST_ARENA_NODES"] = cap
            s = T.Session(val, rp, col, y, objective="reg:linear", n_trees=4, depth=7, max_num_bin=64,
                          learning_rate=0.4, gamma=0.0, min_child_weight=0.5)
            assert s.info("dense_bin_bytes") == int(nbytes)
            s.set_option("bagging", 1)
            s.set_option("column_sampling_rate", 0.4)
            libc.srand(99)
            s.boost(4)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        os.environ.pop("TGBM_DENSE_BIN_BYTES", None)
        os.environ.pop("TGBM_HIST_ARENA_NODES", None)
    assert [a == b for a, b in zip(runs[0], runs[1])] == [True] * 3
    assert [a == b for a, b in zip(runs[0], runs[2])] == [True] * 3


def test_more_than_255_bins_through_the_c_abi(T, tmp_path):
    """fit / predict / save / load of the estimator (sparse_train_scikit, sparse_predict_scikit, save / load through
    the model file) with 2000 bins per feature: the predictor follows split_value, so the prediction of the training
    rows is the session's training prediction without the base score (the C-API predict path carries none), also
    after a round trip through the model file, whose split_bid keeps only the split bin's low byte."""
    rng = np.random.default_rng(11)
    n, F = 20000, 7
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.05] = 0.0
    y = (np.cos(3 * X[:, 0]) * X[:, 1] + 0.5 * X[:, 2] + 0.05 * rng.standard_normal(n)).astype(np.float32)
    kw = dict(depth=6, n_trees=8, learning_rate=0.3, max_num_bin=2000)
    m = T.TGBMRegressor(objective="reg:linear", verbose=0, **kw)
    m.fit(X, y)
    pred = np.asarray(m.predict(X)).ravel()
    val, rp, col = D.dense_to_csr(X)
    s = T.Session(val, rp, col, y, objective="reg:linear", **kw)
    assert s.info("wide_bins") == 1 and s.info("dense_bin_bytes") == 2
    s.boost(8)
    np.testing.assert_allclose(pred, s.y_pred() - s.base_score, rtol=1e-5, atol=1e-5)
    assert np.sqrt(np.mean((pred + s.base_score - y) ** 2)) < 0.6 * np.std(y)
    s.close()
    path = str(tmp_path / "wide.model")
    m.save_model(path)
    m2 = T.TGBMRegressor(objective="reg:linear", verbose=0)
    m2.load_model(path)
    assert np.array_equal(np.asarray(m2.predict(X)).ravel(), pred)


@pytest.mark.parametrize("objective,F,reorder", [("reg:linear", 5, "0"), ("binary:logistic", 40, "always"),
                                                 ("multi:softmax", 11, "0"), ("binary:logistic", 3, "0")])
def test_dense_16_bit_bins_equal_byte_bins(T, objective, F, reorder):
    """The dense layout with 16-bit bins (TGBM_DENSE_BIN_BYTES=2 forces it for data that byte bins can hold) against
    the byte layout: other feature blocks, the same exact integer sums per bin, so the same models, predictions and
    row -> node maps byte for byte (every feature has rows without a value, so neither run takes the root's sums from
    a complete feature's bins). With a re-ordering of the rows after every tree, with class trees built together, and
    with the split search of wide features (TGBM_WIDE_EVAL=1) on top."""
    os.environ["TGBM_LAYOUT"] = "dense"
    os.environ["TGBM_REORDER"] = reorder
    rng = np.random.default_rng(F)
    n = 30000
    X = np.round(rng.standard_normal((n, F)) * 2, 1).astype(np.float32)
    X[rng.random((n, F)) < 0.15] = 0.0
    val, rp, col = D.dense_to_csr(X)
    score = X[:, 0] - 0.5 * X[:, 1] * X[:, 2] + 0.3 * rng.standard_normal(n)
    if objective == "reg:linear":
        y = score.astype(np.float32)
    elif objective == "binary:logistic":
        y = (score > 0).astype(np.float32)
    else:
        y = np.digitize(score, [-1.0, 0.0, 1.0]).astype(np.float32)
    kw = dict(objective=objective, n_trees=4, depth=6, max_num_bin=100, learning_rate=0.4, gamma=0.0)
    runs, mats = [], []
    try:
        for nbytes, wide in (("1", "0"), ("2", "0"), ("2", "1")):
            os.environ["TGBM_DENSE_BIN_BYTES"] = nbytes
            os.environ["TGBM_WIDE_EVAL"] = wide
            s = T.Session(val, rp, col, y, **kw)
            assert s.info("sparse") == 0 and s.info("dense_bin_bytes") == int(nbytes) and s.info("wide_eval") == int(wide)
            m = s.binmat()
            mats.append(np.concatenate([m[b] for b in range(m.shape[0])], axis=1)[:, :F].astype(np.int32))
            s.boost(4)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        for k in ("TGBM_DENSE_BIN_BYTES", "TGBM_WIDE_EVAL", "TGBM_REORDER"):
            os.environ.pop(k, None)
    assert np.array_equal(np.where(mats[0] == 255, 65535, mats[0]), mats[1])
    assert [a == b for a, b in zip(runs[0], runs[1])] == [True] * 3
    assert [a == b for a, b in zip(runs[0], runs[2])] == [True] * 3


def _one_hot_data(n, seed, groups, n_dense, empty_rate=0.0):
    """n_dense quantised columns followed by one-hot groups of the given sizes (zeros are missing values); with
    empty_rate some rows store nothing of a group."""
    rng = np.random.default_rng(seed)
    F = n_dense + sum(groups)
    X = np.zeros((n, F), np.float32)
    X[:, :n_dense] = np.floor(rng.random((n, n_dense)) * 40) + 1
    c0 = n_dense
    code = []
    for g in groups:
        k = rng.integers(0, g, size=n)
        keep = rng.random(n) >= empty_rate
        X[np.arange(n)[keep], c0 + k[keep]] = 1 + (rng.integers(0, 3, size=n)[keep] if g < 6 else 0)  # small groups: 3 values
        code.append(np.where(keep, k, -1))
        c0 += g
    score = X[:, 0] / 20 - X[:, 1] / 30 + 0.7 * (code[0] % 3) - 0.4 * (code[-1] % 5) + 0.3 * rng.standard_normal(n)
    return X, score


@pytest.mark.parametrize("objective,reorder", [("reg:linear", "0"), ("binary:logistic", "always"), ("multi:softmax", "0")])
@pytest.mark.parametrize("shape", ["two_groups", "group_wider_than_a_byte", "only_groups"])
def test_bundled_columns_equal_one_column_per_feature(T, objective, reorder, shape):
    """Runs of consecutive features that never meet in a row (one-hot groups) share a column of the dense matrix
    (TGBM_BUNDLE=0: a column per feature). Same bins once taken apart, same exact integer sums, so the same models,
    predictions and row -> node maps byte for byte - also when a group has more bins than a byte holds (it is split),
    when rows store nothing of a group, with re-ordered rows and with class trees built together."""
    os.environ["TGBM_LAYOUT"] = "dense"
    os.environ["TGBM_REORDER"] = reorder
    groups, n_dense = {"two_groups": ([4, 40], 6), "group_wider_than_a_byte": ([5, 300, 3], 3),
                       "only_groups": ([3, 7, 9], 0)}[shape]
    n = 20000
    X, score = _one_hot_data(n, len(shape), groups, n_dense, empty_rate=0.1)
    F = X.shape[1]
    val, rp, col = D.dense_to_csr(X)
    if objective == "reg:linear":
        y = score.astype(np.float32)
    elif objective == "binary:logistic":
        y = (score > np.median(score)).astype(np.float32)
    else:
        y = np.digitize(score, np.quantile(score, [0.3, 0.6, 0.85])).astype(np.float32)
    kw = dict(objective=objective, n_trees=4, depth=6, max_num_bin=64, learning_rate=0.4, gamma=0.0)
    runs, mats, cols = [], [], []
    try:
        # third run: 16-bit bins, which keep a column per feature whatever TGBM_BUNDLE says
        for bundle, bin_bytes in (("1", None), ("0", None), ("1", "2")):
            os.environ["TGBM_BUNDLE"] = bundle
            if bin_bytes:
                os.environ["TGBM_DENSE_BIN_BYTES"] = bin_bytes
            s = T.Session(val, rp, col, y, **kw)
            assert s.info("sparse") == 0 and s.info("dense_bin_bytes") == int(bin_bytes or 1)
            cols.append(s.info("dense_cols"))
            m = s.binmat()
            m = np.concatenate([m[b] for b in range(m.shape[0])], axis=1)[:, :F].astype(np.int32)
            mats.append(np.where(m == 65535, 255, m) if bin_bytes else m)
            s.boost(4)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        for k in ("TGBM_BUNDLE", "TGBM_REORDER", "TGBM_DENSE_BIN_BYTES"):
            os.environ.pop(k, None)
    assert cols[1] == F and cols[0] < F and cols[2] == F
    assert np.array_equal(mats[2], mats[1])
    assert [a == b for a, b in zip(runs[2], runs[1])] == [True] * 3


def test_bundle_of_a_complete_feature_and_an_empty_one(T):
    """A feature stored in every row can only share its column with features that no row stores. The root's sums are
    then still taken from that feature's bins, as without bundles (they are taken from the gradients otherwise, which
    rounds differently): same bits with a re-ordering after every tree."""
    os.environ["TGBM_LAYOUT"] = "dense"
    os.environ["TGBM_REORDER"] = "always"
    rng = np.random.default_rng(144)
    n, g = 3000, 30
    X = np.zeros((n, 6 + g), np.float32)
    X[:, :3] = np.floor(rng.random((n, 3)) * 30)        # some zeros: not complete
    X[:, 3] = 1 + rng.integers(0, 3, size=n)            # complete
    # column 4 stays empty, column 5 is rare
    X[rng.random(n) < 0.01, 5] = 2
    X[np.arange(n), 6 + rng.integers(0, g, size=n)] = 1
    y = ((X[:, 0] - X[:, 1]) / 10 + X[:, 3] + 0.5 * rng.standard_normal(n) > 2).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    runs = []
    try:
        for bundle in ("1", "0"):
            os.environ["TGBM_BUNDLE"] = bundle
            s = T.Session(val, rp, col, y, objective="binary:logistic", n_trees=4, depth=5, max_num_bin=8, learning_rate=0.5)
            if bundle == "1":
                fc = s.get("feat_col", np.int32)
                assert fc[3] == fc[4] and s.info("dense_cols") < s.F
            s.boost(4)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        for k in ("TGBM_BUNDLE", "TGBM_REORDER"):
            os.environ.pop(k, None)
    assert [a == b for a, b in zip(runs[0], runs[1])] == [True] * 3


def test_sparse_level_pass_at_its_deepest_level(T):
    """Depth 11 (1024 nodes on the last level: the sparse level pass's limit, 12-bit node field of the sorted keys,
    20 KB of per-node LDS state): sorted pass against tables, byte for byte."""
    os.environ["TGBM_LAYOUT"] = "sparse"
    n, F = 60000, 400
    val, rp, col = _ragged(n, F, 51, 10)
    y = _target(val, rp, col, n, F, 51, "bin")
    runs = []
    try:
        for srt in ("1", "0"):
            os.environ["TGBM_SPARSE_SORTED"] = srt
            s = T.Session(val, rp, col, y, objective="binary:logistic", n_trees=2, depth=11, max_num_bin=48,
                          learning_rate=0.5, gamma=0.0, min_child_weight=0.05)
            assert s.info("sparse_pass") == 1
            s.boost(2)
            runs.append((s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()))
            s.close()
    finally:
        os.environ.pop("TGBM_SPARSE_SORTED", None)
    assert [a == b for a, b in zip(runs[0], runs[1])] == [True] * 3


@pytest.mark.parametrize("objective", ["reg:linear", "binary:logistic"])
@pytest.mark.parametrize("F,reorder", [(28, "0"), (28, "always"), (12, "0"), (20, "always"), (40, "0"), (60, "always")])
def test_gradient_words_in_the_bin_matrix_give_the_same_bits(T, objective, F, reorder):
    """With a spare dword at the end of a row's bin-matrix record (features <= row bytes - 4), one tree per round and a
    squared or 0/1-label logistic loss, the histogram kernels take a row's gradient pair from a 32-bit word stored in
    that dword instead of gathering it from the gradient array (TGBM_GH_WORD=0: always gather). The word decodes to
    the very floats of the gradient kernel, the sums are exact integers: models, predictions, row -> node maps and
    the histograms of a level are the same byte for byte - also with missing values, with re-ordered rows, and when a
    level is driven stage by stage after gradients were uploaded by hand (which the words do not know: the kernels
    must fall back to the array)."""
    os.environ["TGBM_LAYOUT"] = "dense"
    os.environ["TGBM_REORDER"] = reorder
    rng = np.random.default_rng(F)
    n = 30000
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.05] = 0
    score = X[:, 0] - X[:, 1] * X[:, 2] + 0.3 * rng.standard_normal(n)
    y = score.astype(np.float32) if objective == "reg:linear" else (score > 0).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    kw = dict(objective=objective, n_trees=5, depth=6, max_num_bin=64, learning_rate=0.3)
    runs = []
    try:
        for word in ("1", "0"):
            os.environ["TGBM_GH_WORD"] = word
            s = T.Session(val, rp, col, y, **kw)
            assert s.info("sparse") == 0 and s.info("dense_blocks") == 1
            assert s.info("gh_word_lane") == (s.info("dense_W") // 4 - 1 if word == "1" else -1)
            s.boost(4)
            out = [s.model().tobytes(), s.y_pred().tobytes(), s.nid().tobytes()]
            # the next round's pairs (inside boost() they may exist as words only: the getter has them recomputed)
            # and its root level by hand, started from what the fused end of the last round left
            s.tree_init()
            s.find_split(0)
            out.append(s.gh().tobytes())
            out.append(s.level_hist(0).tobytes())
            # a level by hand with freshly computed gradients, then with uploaded ones
            s.gradient()
            s.tree_init()
            s.find_split(0)
            out.append(s.level_hist(0).tobytes())
            gh = s.gh().copy()
            gh[:, 0] *= np.float32(0.5)
            s.set("gh", gh)
            s.tree_init()
            s.find_split(0)
            out.append(s.level_hist(0).tobytes())
            runs.append(out)
            s.close()
    finally:
        for k in ("TGBM_GH_WORD", "TGBM_REORDER", "TGBM_LAYOUT"):
            os.environ.pop(k, None)
    assert [a == b for a, b in zip(*runs)] == [True] * 7
    assert runs[0][4] == runs[0][5] and runs[0][5] != runs[0][6]  # the uploaded gradients were used
