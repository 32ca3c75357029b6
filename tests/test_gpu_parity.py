"""GPU parity tests: the HIP library (through its C ABI) against the CPU oracle on the same seeded
inputs. Run on the MI355X box with `pytest -m gpu`."""
import ctypes as C
import os

import numpy as np
import pytest

import datasets as D
import oracle_lib as O
import parity as P

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _default_layout():
    os.environ.pop("TGBM_LAYOUT", None)  # the library picks the layout itself unless a case forces one
    yield
    os.environ.pop("TGBM_LAYOUT", None)


@pytest.fixture(scope="module")
def T():
    import thundergbm_amd
    L = thundergbm_amd.load()
    # the first GPU call of a process initialises the runtime (which may draw from rand() itself): do it here,
    # so that no test's random stream depends on which test runs first
    D.warm_up(thundergbm_amd)
    return thundergbm_amd


def _missing_dataset(n, F, seed, frac=0.3, round_to=1):
    rng = np.random.default_rng(seed)
    X = np.round(rng.standard_normal((n, F)) * 2, round_to).astype(np.float32)
    X[X == 0] = 0.5
    miss = rng.random((n, F)) < frac
    miss[:, 0] = False
    X[miss] = 0
    y = (X[:, 0] * 1.5 - X[:, 1] + rng.standard_normal(n) * 0.3).astype(np.float32)
    return X, y


def _outlier_dataset(n, F, seed):
    """Gaussian regression target with five labels 1e4 times larger than the rest: the gradients of reg:linear
    inherit the outliers, so max|g| is ~1e4 times a typical |g|."""
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[X == 0] = 0.25
    y = (X[:, 0] - 0.5 * X[:, 3] + 0.3 * rng.standard_normal(n)).astype(np.float32)
    y[rng.choice(n, size=5, replace=False)] *= 1e4
    return X, y


def _cases():
    X1, y1 = D.config1(10000, 8, seed=0)
    X2, y2 = _missing_dataset(6000, 11, 3)
    X3, y3 = D.config2(20000, seed=1)
    X5, y5 = D.config5(8000, seed=4)
    v4, rp4, c4, y4 = D.config4(n=20000, F=3000, nnz_per_row=20, seed=3)
    Xw, yw = D.config3(n=20000, F=200, seed=2)
    Xo, yo = _outlier_dataset(20000, 12, 6)
    return {
        "c3_wide_heavy_tails": (D.dense_to_csr(Xw), yw, dict(objective="reg:linear", depth=6, max_num_bin=255)),
        "outlier_regression": (D.dense_to_csr(Xo), yo, dict(objective="reg:linear", depth=6, max_num_bin=255)),
        "c4_sparse": ((v4, rp4, c4), y4, dict(objective="binary:logistic", depth=6, max_num_bin=63)),
        "c1_regression": (D.dense_to_csr(X1), y1, dict(objective="reg:linear", depth=6, max_num_bin=255)),
        "missing_regression": (D.dense_to_csr(X2), y2, dict(objective="reg:linear", depth=5, max_num_bin=16)),
        "c2_binary": (D.dense_to_csr(X3), y3, dict(objective="binary:logistic", depth=6, max_num_bin=255)),
        "c5_softmax": (D.dense_to_csr(X5), y5, dict(objective="multi:softmax", depth=4, max_num_bin=255)),
    }


CASES = None


def case(name):
    """Returns (csr, y, kwargs). Names ending in @sparse run the same data through the CSR layout."""
    global CASES
    if CASES is None:
        CASES = _cases()
    os.environ["TGBM_LAYOUT"] = "sparse" if name.endswith("@sparse") or name.startswith("c4") else "dense"
    return CASES[name.split("@")[0]]


CASE_NAMES = ["c1_regression", "missing_regression", "c2_binary", "c3_wide_heavy_tails", "outlier_regression",
              "c5_softmax", "c4_sparse", "missing_regression@sparse", "c5_softmax@sparse"]


# ----------------------------------------------------------------------- cuts and bin ids (exact)
def _cut_points_gpu(T, val, rp, col, F, max_bin):
    L = T.load()
    val = np.ascontiguousarray(val, np.float32)
    rp = np.ascontiguousarray(rp, np.int32)
    col = np.ascontiguousarray(col, np.int32)
    cap = max(len(val), 1)
    cv = np.zeros(cap, np.float32)
    cf = np.zeros(cap, np.int32)
    crp = np.zeros(F + 1, np.int32)
    bins = np.zeros(cap, np.int32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    nb = L.tgbm_cut_points(len(rp) - 1, F, p(val), p(rp), p(col), max_bin, p(cv), p(crp), p(cf), p(bins))
    return cv[:nb], crp, cf[:nb], bins[: len(val)]


@pytest.mark.parametrize("max_bin", [2, 16, 63, 255])
def test_cut_points_and_bins_exact(T, max_bin):
    rng = np.random.default_rng(max_bin)
    n, F = 30000, 13
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[:, 1] = np.round(X[:, 1], 1)            # few uniques (< 255)
    X[:, 2] = rng.integers(0, 255, n)          # exactly around max_bin uniques, zeros become missing
    X[:, 3] = rng.integers(0, 2, n)            # one unique stored value
    X[:, 4] = 0                                # feature without any stored value
    X[:, 5] = -np.abs(X[:, 5])                 # all negative
    X[:, 6] = rng.integers(-300, 300, n) * 0.5
    X[rng.random((n, F)) < 0.2] = 0
    val, rp, col = D.dense_to_csr(X)
    ocv, ocrp, ocf = O.cut_points(val, col, F, max_bin)
    obins = O.bin_ids(val, col, ocv, ocrp)
    cv, crp, cf, bins = _cut_points_gpu(T, val, rp, col, F, max_bin)
    assert np.array_equal(crp, ocrp)
    assert np.array_equal(cv.view(np.uint32), ocv.view(np.uint32))
    assert np.array_equal(cf, ocf)
    assert np.array_equal(bins, obins)


def test_cut_points_ragged_and_empty_rows(T):
    rng = np.random.default_rng(9)
    n, F = 5000, 300
    lens = rng.integers(0, 12, n)
    lens[:10] = 0
    rp = np.zeros(n + 1, np.int32)
    np.cumsum(lens, out=rp[1:])
    col = np.concatenate([np.sort(rng.choice(F, size=l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.lognormal(0, 1, len(col)).astype(np.float32)
    ocv, ocrp, ocf = O.cut_points(val, col, F, 63)
    cv, crp, cf, bins = _cut_points_gpu(T, val, rp, col, F, 63)
    assert np.array_equal(crp, ocrp) and np.array_equal(cv, ocv) and np.array_equal(cf, ocf)
    assert np.array_equal(bins, O.bin_ids(val, col, ocv, ocrp))


def test_cut_points_a1a_fixture(T):
    val, rp, col, y = D.read_libsvm(D.A1A)
    cv, crp, cf, bins = _cut_points_gpu(T, val, rp, col, 119, 255)
    assert np.all(cv == 1.0) and np.array_equal(cf, np.unique(col))
    assert np.array_equal(bins, crp[col])  # single cut per feature -> local bin 0


@pytest.mark.parametrize("name", CASE_NAMES)
def test_session_cuts_bins_base_score(T, name):
    (val, rp, col), y, kw = case(name)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    cv, crp, cf = s.cuts()
    ocv, ocrp, ocf = o.cuts()
    assert np.array_equal(cv, ocv) and np.array_equal(crp, ocrp) and np.array_equal(cf, ocf)
    gb, local = s.global_bin_ids(rp, col)
    assert np.array_equal(gb, o.bin_ids())
    assert s.info("sparse") == (1 if os.environ["TGBM_LAYOUT"] == "sparse" else 0)
    if not s.info("sparse"):
        # every (row, feature) without a stored value is the missing sentinel
        m = s.binmat()
        W = s.info("dense_W")
        stored = np.zeros((s.n, m.shape[0] * W), bool)
        stored[np.repeat(np.arange(s.n), np.diff(rp)), col] = True
        flat = m.transpose(1, 0, 2).reshape(s.n, -1)
        assert np.all(flat[~stored] == 255)
    assert s.num_class == o.num_class and s.tree_per_rounds == o.tree_per_rounds
    assert np.array_equal(s.labels(), o.labels())
    assert np.array_equal(s.y(), o.y())
    # (a mean of labels of both signs: like every other sum, 1e-5 of the terms' absolute values, not of the result)
    np.testing.assert_allclose(s.base_score, o.base_score, rtol=1e-5, atol=1e-7 + 1e-5 * float(np.abs(y).mean()))
    np.testing.assert_allclose(s.y_pred(), o.y_pred(), rtol=1e-5, atol=1e-7)
    s.close()


# ------------------------------------------------------------------------------------- gradients
@pytest.mark.parametrize("name", CASE_NAMES)
def test_gradients(T, name):
    (val, rp, col), y, kw = case(name)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    rng = np.random.default_rng(5)
    yp = (rng.standard_normal(len(o.y_pred())) * 2).astype(np.float32)
    s.set("y_pred", yp)
    o.set_y_pred(yp)
    s.gradient()
    o.compute_gradient()
    g, og = s.gh(), o.gh()
    if kw["objective"] == "reg:linear":
        assert np.array_equal(g, og)
    else:
        np.testing.assert_allclose(g[:, 0], og[:, 0], rtol=1e-5, atol=2e-7)
        np.testing.assert_allclose(g[:, 1], og[:, 1], rtol=1e-5, atol=2e-7)
    s.close()


# ------------------------------------------------------------ one tree in lock step, level by level
@pytest.mark.parametrize("name", CASE_NAMES)
def test_tree_lockstep(T, name):
    (val, rp, col), y, kw = case(name)
    kw = dict(kw, gamma=0.5)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, debug=True, shadow64=True, **kw).prepare()
    n, nb, depth = s.n, s.n_bins, kw["depth"]
    _, crp, cf = s.cuts()
    rows = np.repeat(np.arange(n), np.diff(rp))
    gbins = o.bin_ids()
    s.gradient()
    gh_all = s.gh()
    o.set_gh(gh_all)  # both sides build from bit-identical gradients
    lam = 1.0
    sparse = bool(s.info("sparse"))
    margins = P.Margins("lockstep/" + name)
    for k in range(s.tree_per_rounds):
        gh = gh_all[k * n:(k + 1) * n]
        ghk = np.abs(gh.astype(np.float64)).sum(axis=0)
        dG, dH = P.sum_bounds(ghk)
        s.tree_init(k)
        o.tree_init(k)
        quant = s.quant()
        # resolution of the fixed-point plan: the coarsest step against the largest |g| of the tree: 47-bit gradient
        # fields and 32768 rows between two drains when every hessian is an integer (squared loss), else 32 bits
        # and 8192 rows
        if not sparse:
            gmax = float(np.abs(gh[:, 0]).max())
            assert bool(quant["h_integer"]) == (kw["objective"] == "reg:linear")
            assert P.node_quantum(quant, n, False)[0] <= gmax * 2.0 ** (-31 if quant["h_integer"] else -17)
        node_of_row = np.zeros(n, np.int64)
        tol_prev = None  # tolerance arrays of the previous level's nodes
        diverged = False
        for level in range(depth):
            s.find_split(level)
            o.find_split(level)
            o.update_tree()
            gh_level = s.level_hist(level)
            onodes = o.nodes()
            gnodes = s.nodes()
            off = (1 << level) - 1
            sp_g, sp_o = s.splits(level), o.splits()
            # Tolerance of a node built from rows: 1e-5 of its own per-bin sum of |g|, |h| plus half a fixed-point
            # step per stored entry; of a node derived as parent - sibling: the sum of the two operands' tolerances.
            S_own, cnt = P.node_hist_refs(gbins, rows, gh, nb, node_of_row, off, 1 << level)
            loc = node_of_row - off
            n_rows = np.bincount(loc[(loc >= 0) & (loc < (1 << level))], minlength=1 << level)
            # built from rows: the root, then of every sibling pair the child with fewer rows, ties the left one
            # (hist_tree_builder_single.cu:466-467)
            built = [level == 0 or n_rows[x] < n_rows[x ^ 1] or (n_rows[x] == n_rows[x ^ 1] and x % 2 == 0)
                     for x in range(1 << level)]
            if s.info("sparse_pass"):  # the sparse level pass sums every node from its own rows
                built = [True] * (1 << level)
            tol_level = [None] * (1 << level)
            for x in range(1 << level):
                if built[x]:
                    tol_level[x] = P.hist_tolerance(S_own[x], cnt[x], P.node_quantum(quant, n_rows[x], sparse))
            for x in range(1 << level):
                if tol_level[x] is None:
                    tol_level[x] = tol_prev[x >> 1] + tol_level[x ^ 1]
            for x in range(1 << level):
                if not onodes[off + x]["is_valid"]:
                    assert sp_g[x]["nid"] == -1 and sp_o[x]["nid"] == -1
                    continue
                _, h64 = o.level_hist(x)
                what = "tree %d level %d node %d" % (k, level, x)
                err = P.assert_hist_close(gh_level[x], h64, tol_level[x], what)
                nz = tol_level[x] > 0
                margins.note("hist", err[nz], tol_level[x][nz])
                if built[x] and (sparse or quant["h_integer"]):
                    # wide fixed-point fields (64-bit sums in the sparse layout, 50-bit gradient fields for squared
                    # loss): also without the half-step allowance, every bin whose entries are not far below the
                    # node's typical |g| is within 1e-5 of its own sum
                    typical = S_own[x][:, 0].sum() / max(1, cnt[x].sum())
                    judged = S_own[x][:, 0] >= 1e-3 * typical * cnt[x]
                    assert np.all(err[judged, 0] <= 1e-5 * S_own[x][judged, 0] + 1e-30), what
                a, b = sp_g[x], sp_o[x]
                ws = [float(onodes[off + x]["base_weight"])]
                if onodes[off + x]["lch"] >= 0:
                    ws += [float(onodes[2 * (off + x) + 1]["base_weight"]), float(onodes[2 * (off + x) + 2]["base_weight"])]
                if a["best_index"] != b["best_index"]:
                    sc = o.tree_scores()[off + x]
                    best = abs(sc).max()
                    assert best - abs(sc[a["best_index"]]) <= 2 * P.gain_tolerance(ws, best, dG, dH), \
                        "level %d node %d picks %d vs %d" % (level, x, a["best_index"], b["best_index"])
                    diverged = True
                    continue
                assert a["fid"] == b["fid"] and a["bid"] == b["bid"] and a["fval"] == b["fval"]
                assert abs(a["gain"] - b["gain"]) <= P.gain_tolerance(ws, b["gain"], dG, dH), what
                margins.note("split_gain", abs(float(a["gain"]) - float(b["gain"])), P.gain_tolerance(ws, b["gain"], dG, dH))
                for key, d in (("lch_g", dG), ("lch_h", dH), ("miss_g", dG), ("miss_h", dH)):
                    assert abs(a[key] - b[key]) <= d, (key, a[key], b[key])
                    margins.note("split_sums", abs(float(a[key]) - float(b[key])), d)
            tol_prev = tol_level
            if diverged:
                break
            # same splits -> node arrays agree and the partition must be bit-identical
            for key in ("is_valid", "is_leaf", "split_fid", "split_bid"):
                assert np.array_equal(gnodes[key], onodes[key]), key
            assert np.array_equal(gnodes["split_value"], onodes["split_value"])
            # default direction matters only where values are missing; force agreement for the rest
            # by copying the GPU's nodes into the oracle (sums differ in the last ulps only)
            np.testing.assert_allclose(gnodes["sum_g"], onodes["sum_g"], rtol=0, atol=dG)
            np.testing.assert_allclose(gnodes["sum_h"], onodes["sum_h"], rtol=0, atol=dH)
            o.set_nodes(gnodes)
            s.partition(level)
            has = o.update_ins2node()
            assert np.array_equal(s.nid(), o.nid()), "node assignment differs at level %d" % level
            node_of_row = s.nid().astype(np.int64)
            if not s.info("row_lists"):  # the sparse level pass keeps the row -> node map only
                if not has:
                    break
                continue
            # row lists: every node's segment holds exactly its rows in ascending order
            seg = s.get("seg", np.int32, (-1, 2))
            ridx = s.get("ridx%d" % ((level + 1) & 1), np.int32)
            nid = s.nid()
            last = level == s.info("depth") - 1  # the last level's children only exist in the row -> node map
            for x in range((2 << level) - 1, (4 << level) - 1):
                b, e = seg[x]
                mine = np.flatnonzero(nid == x)
                if not last and gnodes[(x - 1) // 2]["split_fid"] >= 0 and not gnodes[(x - 1) // 2]["is_leaf"]:
                    assert np.array_equal(ridx[b:e], mine), "row list of node %d" % x
                else:
                    assert e - b == 0
            if not has:
                break
        if diverged:
            continue
        s.finish_tree(k)
        o.prune()
        o.predict_in_training(k)
        d = P.compare_trees(s.nodes(), o.nodes(), lam, crp=crp, orc_scores=o.tree_scores(), abs_scale=(ghk[0], ghk[1]),
                            gamma=kw["gamma"])
        assert not d.near_ties
        margins.add(d)
        sl = slice(k * n, (k + 1) * n)
        tol = P.pred_tolerance(o.nodes(), o.nid(), 1.0, lam, (ghk[0], ghk[1]), o.y_pred()[sl])
        perr = np.abs(s.y_pred()[sl].astype(np.float64) - o.y_pred()[sl])
        assert np.all(perr <= tol)
        margins.note("pred", perr, tol)
    margins.report()
    s.close()


# -------------------------------------------------------------------- boosting, tree by tree
# (case, rounds, significant near ties allowed = the count observed on the MI355X + 1; the two of outlier_regression
# are nodes of a few rows next to the 1e4x outliers)
@pytest.mark.parametrize("name,rounds,tie_budget", [
    ("c1_regression", 40, 1), ("missing_regression", 10, 1), ("c2_binary", 10, 1), ("c3_wide_heavy_tails", 6, 1),
    ("outlier_regression", 8, 3), ("c5_softmax", 3, 1), ("c4_sparse", 10, 1), ("missing_regression@sparse", 10, 1),
    ("c1_regression@sparse", 5, 1)])
def test_boosting_teacher_forced(T, name, rounds, tie_budget):
    """Each round both sides start from the GPU's predictions, so every tree is compared on its own."""
    (val, rp, col), y, kw = case(name)
    kw = dict(kw, n_trees=rounds, learning_rate=0.1 if name == "c1_regression" else 0.3)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, debug=True, **kw).prepare()
    _, crp, _ = s.cuts()
    n = s.n
    present = np.zeros((n, s.F), bool)
    present[np.repeat(np.arange(n), np.diff(rp)), col] = True
    total_ties = 0
    margins = P.Margins("teacher_forced/" + name)
    for r in range(rounds):
        yp = s.y_pred()
        o.set_y_pred(yp)
        s.gradient()
        gh = s.gh()  # the gradients this round is built from (boost recomputes the same values)
        s.boost(1)
        model = s.model()
        o.compute_gradient()
        ogh = o.gh()
        np.testing.assert_allclose(gh, ogh, rtol=1e-5, atol=2e-7)
        o.set_gh(gh)
        ok_round = True
        tol = np.zeros(len(yp))
        for k in range(s.tree_per_rounds):
            o.build_tree(k)
            final_nid = o.nid()
            ghk = np.abs(gh[k * n:(k + 1) * n].astype(np.float64)).sum(axis=0)
            d = P.compare_trees(model[r, k], o.nodes(), 1.0, crp=crp, orc_scores=o.tree_scores(), orc_dir_gaps=o.tree_dir_gaps(),
                                missing_rows=lambda x, f: int((~present[P.rows_in_node(final_nid, x), f]).sum()),
                                abs_scale=(ghk[0], ghk[1]))
            # candidates that cut a node's rows into the same two sets have equal gains in exact arithmetic and
            # differ by float round-off only (wide data, nodes of a few rows): those are not counted
            total_ties += len(P.significant_ties(d.near_ties))
            ok_round &= not d.near_ties
            margins.add(d)
            sl = slice(k * n, (k + 1) * n)
            tol[sl] = P.pred_tolerance(o.nodes(), final_nid, kw["learning_rate"], 1.0, (ghk[0], ghk[1]), o.y_pred()[sl])
        if ok_round:
            perr = np.abs(s.y_pred().astype(np.float64) - o.y_pred())
            assert np.all(perr <= tol)
            margins.note("pred", perr, tol)
            np.testing.assert_allclose(s.metric_log()[-1], o.metric(), rtol=1e-4, atol=1e-5)
    margins.ties = total_ties
    margins.report()
    assert total_ties <= tie_budget, "too many near ties: %d" % total_ties
    # how much of the 1e-5 bounds the two implementations use (the GPU's sums are exact integers; what is left is the
    # float32 prefix scan and subtraction chain of the reference's algorithm): at most 0.4 observed
    assert max(margins.worst.values()) <= 0.8, margins.worst
    s.close()


def test_free_running_c1_matches_oracle(T):
    """Benchmark configuration 1 end to end (10 000 x 8, 40 trees, depth 6, lr 0.1) without teacher forcing."""
    X, y = D.config1(10000, 8, seed=0)
    val, rp, col = D.dense_to_csr(X)
    kw = dict(depth=6, n_trees=40, learning_rate=0.1, max_num_bin=255)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    s.boost(40)
    o.boost(40)
    ml, oml = s.metric_log(), o.metric_log()
    assert np.all(np.diff(ml) < 0)
    np.testing.assert_allclose(ml, oml, rtol=2e-3)
    np.testing.assert_allclose(ml[:5], oml[:5], rtol=1e-5)
    s.close()


# -------------------------------------------------------------------------- prediction and C ABI
@pytest.mark.parametrize("objective", ["reg:linear", "binary:logistic", "multi:softmax", "multi:softprob"])
def test_estimator_fit_predict_save_load(T, objective, tmp_path):
    n, F = 3000, 9
    X, y = _missing_dataset(n, F, 17)
    if objective == "binary:logistic":
        y = np.where(y > 0, 1.0, -1.0).astype(np.float32)
    elif objective.startswith("multi:"):
        y = (np.digitize(y, np.quantile(y, [0.25, 0.5, 0.75])) * 2 + 1).astype(np.float32)
    cls = T.TGBMRegressor if objective == "reg:linear" else T.TGBMClassifier
    m = cls(depth=4, n_trees=5, learning_rate=0.5, objective=objective, verbose=0, max_num_bin=32)
    m.fit(X, y)
    pred = m.predict(X)
    # the oracle on the same CSR input
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=4, n_trees=5, learning_rate=0.5, objective=objective, max_num_bin=32,
                 num_class=2).prepare()
    o.boost(5)
    # the C-API predict path carries no base score (reference quirk): raw = sum of trees only
    raw = O.predict_raw(val, rp, col, F, o.model(), 0.5, 0.0)
    labels = o.labels() if objective != "reg:linear" else np.zeros(1, np.float32)
    exp = O.predict_transform(objective, raw, n, o.num_class, labels)
    assert m.num_class == o.num_class and m.tree_per_iter == o.tree_per_rounds
    if objective == "reg:linear" or objective == "multi:softprob":
        np.testing.assert_allclose(pred.ravel(), exp, rtol=1e-4, atol=1e-5)
    else:
        assert np.mean(pred == exp) > 0.995
    # tree export
    trees = m.get_trees()
    assert len(trees) == 5 * m.tree_per_iter and len(trees[0]["feature"]) == 31
    om = o.model().reshape(-1, 31)
    leaf = om[0]["is_leaf"] == 1
    assert np.array_equal(trees[0]["children_left"][leaf], -np.ones(leaf.sum(), np.int32))
    # save / load round trip gives identical predictions
    path = str(tmp_path / "m.model")
    m.save_model(path)
    m2 = cls(objective=objective, verbose=0)
    m2.load_model(path)
    pred2 = m2.predict(X)
    assert np.array_equal(np.asarray(pred), np.asarray(pred2))
    assert m2.group_label == m.group_label or objective == "reg:linear"


def test_predict_raw_equals_training_prediction(T):
    (val, rp, col), y, kw = case("c2_binary")
    s = T.Session(val, rp, col, y, n_trees=8, learning_rate=0.3, **kw)
    s.boost(8)
    L = T.load()
    model = C.c_void_p(s.export_model())
    out = np.zeros(s.n, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    L.tgbm_predict_raw(s.n, p(val), p(rp), p(col), model, 8, 1, 0.3, s.base_score, p(out))
    np.testing.assert_allclose(out, s.y_pred(), rtol=1e-5, atol=1e-6)
    # and against the oracle's predictor on the GPU's model
    ref = O.predict_raw(val, rp, col, s.F, s.model(), 0.3, s.base_score)
    np.testing.assert_allclose(out, ref, rtol=1e-6, atol=1e-6)
    L.model_free(C.byref(model))
    s.close()


def test_predict_wide_float_path_and_unseen_rows(T):
    # F > 96 takes the reference's float accumulation path; unseen rows exercise default directions
    rng = np.random.default_rng(3)
    n, F = 4000, 130
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.5] = 0
    y = (X[:, 0] - X[:, 5] + 0.1 * rng.standard_normal(n)).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    s = T.Session(val, rp, col, y, depth=5, n_trees=6, learning_rate=0.4, max_num_bin=64)
    s.boost(6)
    Xt = rng.standard_normal((1000, F)).astype(np.float32)
    Xt[rng.random((1000, F)) < 0.5] = 0
    tv, trp, tc = D.dense_to_csr(Xt)
    L = T.load()
    model = C.c_void_p(s.export_model())
    out = np.zeros(1000, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    L.tgbm_predict_raw(1000, p(tv), p(trp), p(tc), model, 6, 1, 0.4, s.base_score, p(out))
    ref = O.predict_raw(tv, trp, tc, F, s.model(), 0.4, s.base_score)
    np.testing.assert_allclose(out, ref, rtol=1e-6, atol=1e-6)
    L.model_free(C.byref(model))
    s.close()


@pytest.mark.parametrize("F,depth,num_class", [(20, 6, 1), (60, 3, 1), (96, 5, 3), (30, 12, 1), (12, 8, 4)])
def test_predict_paths_of_the_dense_vector_kernels(T, F, depth, num_class):
    """The predictor's kernels that spread a row into a dense vector in LDS (F <= 96): trees staged in LDS for 256 rows
    per workgroup (F <= 48) or 128 (F <= 96), several trees per stage when they are small, and the walk through the
    48-byte nodes in global memory when one tree does not fit the LDS (depth 12) - each against the oracle's
    predictor on the same model and unseen rows."""
    rng = np.random.default_rng(F + depth)
    n = 3000
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.3] = 0
    score = X[:, 0] - X[:, 1] * X[:, 2] + 0.1 * rng.standard_normal(n)
    kw = dict(depth=depth, n_trees=5, learning_rate=0.4, max_num_bin=32, min_child_weight=0.1)
    if num_class > 1:
        y = np.digitize(score, np.quantile(score, np.linspace(0, 1, num_class + 1)[1:-1])).astype(np.float32)
        kw["objective"] = "multi:softprob"
    else:
        y = score.astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    s = T.Session(val, rp, col, y, **kw)
    s.boost(5)
    Xt = rng.standard_normal((777, F)).astype(np.float32)
    Xt[rng.random((777, F)) < 0.3] = 0
    tv, trp, tc = D.dense_to_csr(Xt)
    if len(tc) and tc.max() != F - 1:
        tc[-1] = F - 1
    L = T.load()
    model = C.c_void_p(s.export_model())
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    k = s.tree_per_rounds
    base = s.base_score if k == 1 else 0.0
    ref = O.predict_raw(tv, trp, tc, F, s.model(), 0.4, base)
    out = np.zeros(777 * k, np.float32)
    L.tgbm_predict_raw(777, p(tv), p(trp), p(tc), model, 5, k, 0.4, base, p(out))
    np.testing.assert_allclose(out, ref, rtol=1e-6, atol=1e-6)
    L.model_free(C.byref(model))
    s.close()


def _model_file(path, objective, lr, base_score, labels, model):
    """The reference's model file (parser.cpp:102-171) for trees given as NODE arrays [n_iter, trees per round, nodes]."""
    import struct
    n_iter, k, n_nodes = model.shape
    out = struct.pack("<i", len(objective)) + objective
    out += struct.pack("<fiif", lr, max(k, 1) if k > 1 else 1, n_iter, base_score)
    out += struct.pack("<i", len(labels)) + struct.pack("<%df" % len(labels), *labels)
    out += struct.pack("<i", n_iter)
    for it in range(n_iter):
        out += struct.pack("<i", k)
        for t in range(k):
            out += struct.pack("<Q", n_nodes) + np.ascontiguousarray(model[it, t]).tobytes()
    with open(path, "wb") as f:
        f.write(out)


def _predict_variants(L, n, tv, trp, tc, model, n_iter, k, lr, base, settings):
    """tgbm_predict_raw under each (TGBM_PREDICT_COMPACT, TGBM_PREDICT_TPS) setting; the switches are read per call."""
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    outs = {}
    try:
        for compact, tps in settings:
            os.environ["TGBM_PREDICT_COMPACT"], os.environ["TGBM_PREDICT_TPS"] = str(compact), str(tps)
            out = np.zeros(n * k, np.float32)
            L.tgbm_predict_raw(n, p(tv), p(trp), p(tc), model, n_iter, k, lr, base, p(out))
            outs[(compact, tps)] = out
    finally:
        os.environ.pop("TGBM_PREDICT_COMPACT", None)
        os.environ.pop("TGBM_PREDICT_TPS", None)
    return outs


@pytest.mark.parametrize("num_class,depth", [(1, 6), (3, 4)])
def test_predict_kernels_agree_bit_for_bit(T, num_class, depth, tmp_path):
    """The predictor's LDS kernels - 48-byte nodes in global memory, 16-byte records, 8-byte records with one or two
    trees walked at a time, with and without the coalesced spreading of equal-length rows - give the same bits,
    and the oracle's predictor agrees, on: dense rows (equal length, some stored +inf / NaN / -inf), the same rows with
    one row's columns descending and one column repeated (the later entry counts), ragged rows, and rows that lack
    the model's last features. The same trees with their nodes stored in another order (children not side by side:
    the 8-byte records do not apply) predict the same bits too."""
    rng = np.random.default_rng(7 + num_class)
    n, F, n_iter, lr = 3000, 20, 7, 0.4
    X = rng.standard_normal((n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.1] = 0
    score = X[:, 0] - X[:, 1] * X[:, 2] + X[:, F - 1] + 0.1 * rng.standard_normal(n)
    kw = dict(depth=depth, n_trees=n_iter, learning_rate=lr, max_num_bin=32, min_child_weight=0.1)
    if num_class > 1:
        y = np.digitize(score, np.quantile(score, np.linspace(0, 1, num_class + 1)[1:-1])).astype(np.float32)
        kw["objective"] = "multi:softprob"
    else:
        y = score.astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    s = T.Session(val, rp, col, y, **kw)
    s.boost(n_iter)
    k = s.tree_per_rounds
    base = s.base_score if k == 1 else 0.0
    nodes = s.model().copy()
    assert (nodes["split_fid"] == F - 1).any()
    L = T.load()
    model = C.c_void_p(s.export_model())
    m = 1001  # not a multiple of the workgroup's rows
    Xt = rng.standard_normal((m, F)).astype(np.float32)
    Xt[5, 3], Xt[6, 0], Xt[7, 1] = np.inf, np.nan, -np.inf
    full_rp = (np.arange(m + 1) * F).astype(np.int32)
    full_col = np.tile(np.arange(F, dtype=np.int32), m)
    full_val = Xt.reshape(-1).copy()
    cases = {"dense": (full_val, full_rp, full_col, F)}
    c2, v2 = full_col.copy(), full_val.copy()
    c2[300 * F + 4], c2[300 * F + 5] = 5, 4        # row 300: columns 4 and 5 swapped (descending)
    c2[700 * F + 9] = 8                              # row 700: column 8 stored twice, the later entry counts
    cases["unsorted"] = (v2, full_rp, c2, F)
    Xr = Xt.copy()
    Xr[rng.random((m, F)) < 0.4] = 0
    cases["ragged"] = D.dense_to_csr(Xr)[0], D.dense_to_csr(Xr)[1], D.dense_to_csr(Xr)[2], F
    short = F - 3                                     # the data's last column is 16: the model's features 17..19 are missing
    keep = np.tile(np.arange(F) < short, m)
    cases["short"] = (full_val[keep], (np.arange(m + 1) * short).astype(np.int32), full_col[keep], short)
    settings = [(0, 0), (0, 1), (0, 4), (1, 1), (1, 2), (2, 1), (2, 2)]
    results = {}
    for name, (tv, trp, tc, Fd) in cases.items():
        tv, trp, tc = np.ascontiguousarray(tv), np.ascontiguousarray(trp), np.ascontiguousarray(tc)
        outs = _predict_variants(L, m, tv, trp, tc, model, n_iter, k, lr, base, settings)
        first = outs[settings[0]]
        for key, out in outs.items():
            assert np.array_equal(out, first, equal_nan=True), (name, key)
        if name == "unsorted":
            # what the row-per-thread loop defines: the later entry of a repeated column; order does not matter
            srt = full_val.copy()
            srt[300 * F + 4], srt[300 * F + 5] = full_val[300 * F + 5], full_val[300 * F + 4]
            srt[700 * F + 8] = full_val[700 * F + 9]
            gone = 700 * F + 9  # row 700 has no column 9 any more
            rp_ref = full_rp.copy()
            rp_ref[701:] -= 1
            ref = O.predict_raw(np.delete(srt, gone), rp_ref, np.delete(full_col, gone), F, nodes, lr, base)
        else:
            ref = O.predict_raw(tv, trp, tc, Fd, nodes, lr, base)
        np.testing.assert_allclose(first, ref, rtol=1e-6, atol=1e-6, err_msg=name)
        results[name] = first
    L.model_free(C.byref(model))
    # the same trees with the nodes of every tree in another order
    perm_nodes = nodes.copy()
    n_nodes = nodes.shape[2]
    for it in range(n_iter):
        for t in range(k):
            order = np.concatenate([[0], 1 + rng.permutation(n_nodes - 1)])  # new position -> old index; the root stays
            where = np.empty(n_nodes, np.int64)
            where[order] = np.arange(n_nodes)
            tree = nodes[it, t][order].copy()
            for name in ("lch", "rch", "parent"):
                old = tree[name]
                tree[name] = np.where(old >= 0, where[np.clip(old, 0, n_nodes - 1)], old)
            perm_nodes[it, t] = tree
    path = str(tmp_path / "perm.model")
    labels = [float(v) for v in range(max(k, 2))]
    _model_file(path, b"multi:softprob" if k > 1 else b"reg:linear", lr, base, labels, perm_nodes)
    model2 = C.c_void_p(None)
    f1, i1, i2, i3 = (C.c_float * 1)(), (C.c_int * 1)(), (C.c_int * 1)(), (C.c_int * 1)()
    vp = lambda a: C.cast(a, C.c_void_p)
    L.load_model(path.encode(), vp(f1), vp(i1), vp(i2), vp(i3), vp(C.byref(model2)))
    assert i2[0] == n_iter * k or i2[0] == n_iter
    tv, trp, tc, _ = cases["dense"]
    outs = _predict_variants(L, m, tv, trp, tc, model2, n_iter, k, lr, base, [(1, 2), (0, 0)])
    assert np.array_equal(outs[(1, 2)], results["dense"], equal_nan=True)
    assert np.array_equal(outs[(0, 0)], results["dense"], equal_nan=True)
    L.model_free(C.byref(model2))
    s.close()


@pytest.mark.parametrize("layout", ["dense", "sparse"])
def test_a1a_quickstart_known_answer(T, layout):
    # README.md:76-80 of the reference: RMSE = 0.489562 (zero initial prediction, see the oracle test)
    os.environ["TGBM_LAYOUT"] = layout
    val, rp, col, y = D.read_libsvm(D.A1A)
    s = T.Session(val, rp, col, y, depth=6, n_trees=40, learning_rate=1.0)
    s.set("y_pred", np.zeros(len(y), np.float32))
    s.boost(40)
    assert abs(float(s.metric_log()[-1]) - 0.489562) < 5e-5
    s.close()


# ------------------------------------- the benchmark configurations at full size: properties, then the oracle
_FULL = {}


def _full_data(name):
    """CSR arrays and labels of a full-size configuration; the tests of one configuration follow each other, and only
    the last one asked for is kept."""
    if name not in _FULL:
        _FULL.clear()
        if name == "c2":
            X, y = D.config2(10_000_000, seed=1)
        elif name == "c3":
            X, y = D.config3()
        elif name == "c5":
            X, y = D.config5()
        if name == "c4":
            val, rp, col, y = D.config4()
        else:
            val, rp, col = D.dense_to_csr(X)
            del X
        _FULL[name] = (val, rp, col, y)
    return _FULL[name]


class _Stored:
    """Which rows store which feature: lacking(f) = mask of the rows without feature f. Rows that store every
    feature are skipped outright (continuous data has a handful of rows with an exact zero); data with many
    incomplete rows gets a column-major copy when first asked (a direction that differs is rare)."""

    def __init__(self, rp, col, F):
        self.rp, self.col, self.F, self.n = rp, col, F, len(rp) - 1
        self.incomplete = np.flatnonzero(np.diff(rp) < F)
        self.csc = None

    def lacking(self, f):
        m = np.zeros(self.n, bool)
        if len(self.incomplete) <= 10000:
            for r in self.incomplete:
                m[r] = f not in self.col[self.rp[r]:self.rp[r + 1]]
            return m
        if self.csc is None:
            import scipy.sparse as sp
            self.csc = sp.csr_matrix((np.ones(len(self.col), np.int8), self.col, self.rp), shape=(self.n, self.F)).tocsc()
        m[:] = True
        m[self.csc.indices[self.csc.indptr[f]:self.csc.indptr[f + 1]]] = False
        return m


def _oracle_tree_at_full_size(T, s, o, round_index, crp, lr, margins, stored):
    """One boosting round of the library against the oracle started from the library's predictions and gradients:
    every class tree through compare_trees (candidate gains from probes: the oracle records, per node, its best gain
    and the gain of the candidate the GPU chose), the row -> node map bit for bit, predictions within the bound.
    Returns the number of near ties."""
    n, K = s.n, s.tree_per_rounds
    o.set_y_pred(s.y_pred())
    s.gradient()
    gh = s.gh()
    s.boost(1)
    model = s.model()
    o.compute_gradient()
    np.testing.assert_allclose(gh, o.gh(), rtol=1e-5, atol=2e-7)
    o.set_gh(gh)
    ties = 0
    for k in range(K):
        gpu = model[round_index, k]
        o.set_probes(P.probes_for(gpu, crp))
        o.build_tree(k)
        final_nid = o.nid()
        ghk = np.abs(gh[k * n:(k + 1) * n].astype(np.float64)).sum(axis=0)

        def rows_without(x, f):
            m = stored.lacking(f)
            return m & P.rows_in_node(final_nid, x) if m.any() else m

        d = P.compare_trees(gpu, o.nodes(), 1.0, crp=crp, orc_scores=P.ProbeScores(*o.probes()),
                            missing_rows=lambda x, f: int(rows_without(x, f).sum()), abs_scale=(ghk[0], ghk[1]),
                            few_missing_rows=4)
        margins.add(d)
        ties += len(P.significant_ties(d.near_ties))
        for t in d.near_ties:  # how close the candidates are that the two sides chose between
            margins.worst["near_tie_rel_gap"] = max(margins.worst.get("near_tie_rel_gap", 0.0), (t[1] - t[2]) / max(t[1], 1e-30))
        margins.worst["near_ties_all"] = margins.worst.get("near_ties_all", 0) + len(d.near_ties)
        if d.near_ties:
            continue
        # rows that may sit elsewhere: the few without the split feature of a node where sending them left or right
        # gains the same within the tolerance (continuous data holds a handful of exact zeros, which are not stored)
        excused = np.zeros(n, bool)
        for x, f in d.direction_ties:
            excused |= rows_without(x, f)
        assert excused.sum() <= 4 * len(d.direction_ties)
        if k == K - 1:
            assert np.array_equal(s.nid()[~excused], final_nid[~excused]), "row -> node map differs"
        sl = slice(k * n, (k + 1) * n)
        tol = P.pred_tolerance(o.nodes(), final_nid, lr, 1.0, (ghk[0], ghk[1]), o.y_pred()[sl])
        perr = np.abs(s.y_pred()[sl].astype(np.float64) - o.y_pred()[sl])
        assert np.all(perr[~excused] <= tol[~excused])
        margins.note("pred", perr[~excused], tol[~excused])
    o.set_probes(None)
    return ties


def test_full_size_properties_config2(T):
    n = int(os.environ.get("TGBM_TEST_FULL_ROWS", "10000000"))
    X, y = D.config2(n, seed=1)
    val, rp, col = D.dense_to_csr(X)
    # the cut rule in closed form on three full-size columns (hist_cut.cu:259-265): sorted distinct stored values,
    # all of them when fewer than max_num_bin, else every (n_unique / max_num_bin)-th, max_num_bin of them
    expected_cuts, columns = {}, {}
    for f in (0, 13, 27):
        columns[f] = X[:, f].copy()
        u = np.unique(X[:, f][X[:, f] != 0])
        expected_cuts[f] = u if len(u) < 255 else u[np.arange(255) * (len(u) // 255)]
    del X
    s = T.Session(val, rp, col, y, depth=8, n_trees=2, objective="binary:logistic", learning_rate=0.3)
    _, crp, cf = s.cuts()
    # cut invariants
    cv = s.cuts()[0]
    for f in range(s.F):
        seg = cv[crp[f]:crp[f + 1]]
        assert len(seg) <= 255 and np.all(np.diff(seg) > 0)
    binmat = s.binmat()  # [blocks, n, W] bytes, in the caller's row order
    W = s.info("dense_W")
    for f, exp in expected_cuts.items():
        assert np.array_equal(cv[crp[f]:crp[f + 1]].view(np.uint32), exp.astype(np.float32).view(np.uint32))
        # bin id of every row of the column: min(#{cuts <= v}, k - 1), 255 where nothing is stored
        # (hist_tree_builder_single.cu:81-92, :113-119)
        x = columns[f]
        want = np.minimum(np.searchsorted(exp, x, side="right"), len(exp) - 1).astype(np.uint8)
        want[x == 0] = 255
        assert np.array_equal(binmat[f // W, :, f % W], want)
    del binmat, columns
    s.gradient()
    s.tree_init(0)
    gh = s.gh()[:n].astype(np.float64)
    Ag, Ah = np.abs(gh[:, 0]).sum(), np.abs(gh[:, 1]).sum()
    for level in range(8):
        s.find_split(level)
        hist = s.level_hist(level).astype(np.float64)
        nodes = s.nodes()
        off = (1 << level) - 1
        for x in range(1 << level):
            nd = nodes[off + x]
            if not nd["is_valid"]:
                continue
            for f in (0, 13, 27):  # dense features: every row lands in exactly one bin of the feature
                tot = hist[x, crp[f]:crp[f + 1]].sum(axis=0)
                # node sums come from float32 prefix sums of ancestors' histograms, so their error
                # is relative to the root-level magnitude, not to the node's own
                assert abs(tot[0] - nd["sum_g"]) <= 1e-5 * Ag and abs(tot[1] - nd["sum_h"]) <= 1e-5 * Ah
        s.partition(level)
    nid = s.nid()
    nodes = s.nodes()
    cnt = np.bincount(nid, minlength=len(nodes))
    # rows only sit in valid nodes; child hessian sums match the rows that arrived (fp64 recount)
    assert np.all(nodes["is_valid"][cnt > 0] == 1)
    hs = np.bincount(nid, weights=gh[:, 1], minlength=len(nodes))
    gs = np.bincount(nid, weights=gh[:, 0], minlength=len(nodes))
    occupied = np.flatnonzero(cnt > 0)
    np.testing.assert_allclose(nodes["sum_h"][occupied], hs[occupied], rtol=0, atol=1e-5 * Ah)
    np.testing.assert_allclose(nodes["sum_g"][occupied], gs[occupied], rtol=0, atol=1e-5 * Ag)
    s.finish_tree(0)
    # training-time prediction == predictor on a sample of the training rows
    yp = s.y_pred()
    sub = slice(0, 200000)
    L = T.load()
    model = C.c_void_p(s.export_model())
    out = np.zeros(200000, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    srp = rp[: 200001].copy()
    L.tgbm_predict_raw(200000, p(val), p(srp), p(col), model, 1, 1, 0.3, s.base_score, p(out))
    np.testing.assert_allclose(out, yp[sub], rtol=1e-5, atol=1e-6)
    L.model_free(C.byref(model))
    s.close()


def _check_boosted_round(T, val, rp, col, y, n_sample, pre_rounds=0, **kw):
    """One production boost() round at full size, checked through properties that need no oracle run:
    every tree's root sum is the fp64 sum of its class's gradients; the rows that ended in a node (last
    class tree) reproduce that node's sums in an fp64 recount; children add up to their parent; the
    predictor on a sample of training rows reproduces the training-time predictions."""
    n = len(rp) - 1
    s = T.Session(val, rp, col, y, n_trees=2 + pre_rounds, learning_rate=0.3, **kw)
    K = s.tree_per_rounds
    if pre_rounds:
        s.boost(pre_rounds)
    s.gradient()
    gh = s.gh().astype(np.float64)
    s.boost(1)
    model = s.model()
    for k in range(K):
        ghk = gh[k * n:(k + 1) * n]
        Ag, Ah = np.abs(ghk[:, 0]).sum(), np.abs(ghk[:, 1]).sum()
        nodes = model[pre_rounds, k]
        assert nodes[0]["is_valid"]
        assert abs(nodes[0]["sum_g"] - ghk[:, 0].sum()) <= 1e-5 * Ag and abs(nodes[0]["sum_h"] - ghk[:, 1].sum()) <= 1e-5 * Ah
        inner = np.flatnonzero((nodes["is_valid"] == 1) & (nodes["split_fid"] >= 0))
        l, r = nodes["lch"][inner], nodes["rch"][inner]
        assert np.all(np.abs(nodes["sum_g"][l].astype(np.float64) + nodes["sum_g"][r] - nodes["sum_g"][inner]) <= 1e-5 * Ag)
        assert np.all(np.abs(nodes["sum_h"][l].astype(np.float64) + nodes["sum_h"][r] - nodes["sum_h"][inner]) <= 1e-5 * Ah)
    nid = s.nid()  # of the last class tree
    cnt = np.bincount(nid, minlength=len(nodes))
    occupied = np.flatnonzero(cnt > 0)
    assert np.all(nodes["is_valid"][occupied] == 1) and np.all(nodes["split_fid"][occupied] < 0)
    np.testing.assert_allclose(nodes["sum_h"][occupied], np.bincount(nid, weights=ghk[:, 1], minlength=len(nodes))[occupied],
                               rtol=0, atol=1e-5 * Ah)
    np.testing.assert_allclose(nodes["sum_g"][occupied], np.bincount(nid, weights=ghk[:, 0], minlength=len(nodes))[occupied],
                               rtol=0, atol=1e-5 * Ag)
    yp = s.y_pred().reshape(-1, n)
    L = T.load()
    handle = C.c_void_p(s.export_model())
    m = n_sample
    out = np.zeros(K * m, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    srp = rp[: m + 1].copy()
    L.tgbm_predict_raw(m, p(val), p(srp), p(col), handle, 1 + pre_rounds, K, 0.3, s.base_score if K == 1 else 0.0,
                       p(out))
    np.testing.assert_allclose(out.reshape(K, m), yp[:, :m], rtol=1e-5, atol=1e-6)
    L.model_free(C.byref(handle))
    s.close()


def test_full_size_properties_config2_reordered_rows(T):
    """10 M x 28 after the rows were physically re-ordered (boost() does that after the second tree): the
    fourth tree's sums against an fp64 recount through the row -> node map, which like the gradients and the
    predictions comes back in the caller's row order, and the predictor against the training predictions."""
    val, rp, col, y = _full_data("c2")
    _check_boosted_round(T, val, rp, col, y, 100000, pre_rounds=3, objective="binary:logistic", depth=8,
                         max_num_bin=255)


def test_full_size_oracle_config2(T):
    """10 M x 28, depth 8, 255 bins against the oracle at the full shape: the first tree (rows in the caller's order,
    512-item plans, work items drained every 8192 rows) and the fifth (after three physical re-orderings of the
    rows)."""
    val, rp, col, y = _full_data("c2")
    kw = dict(objective="binary:logistic", depth=8, max_num_bin=255, learning_rate=0.3, n_trees=5)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    cv, crp, cf = s.cuts()
    ocv, ocrp, ocf = o.cuts()
    assert np.array_equal(cv.view(np.uint32), ocv.view(np.uint32)) and np.array_equal(crp, ocrp)
    gb, _ = s.global_bin_ids(rp, col)
    assert np.array_equal(gb, o.bin_ids())
    del gb
    stored = _Stored(rp, col, s.F)
    margins = P.Margins("full_size/config2")
    ties = _oracle_tree_at_full_size(T, s, o, 0, crp, 0.3, margins, stored)
    s.boost(3)
    assert s.info("reorders_done") >= 3
    ties += _oracle_tree_at_full_size(T, s, o, 4, crp, 0.3, margins, stored)
    margins.ties = ties
    margins.report()
    assert ties <= 1
    s.close()


def test_full_size_properties_16_bit_bins_reordered_rows(T):
    """4 M x 28 with up to 1024 bins per feature (the dense layout's 16-bit bins, four blocks of eight features),
    rows re-ordered after the trees before: same properties."""
    X, y = D.config2(4_000_000, seed=1)
    val, rp, col = D.dense_to_csr(X)
    del X
    _check_boosted_round(T, val, rp, col, y, 100000, pre_rounds=3, objective="binary:logistic", depth=8,
                         max_num_bin=1024)


def test_full_size_properties_config5_softmax(T):
    """1 M x 54, 8 classes: the class trees of the round are built by common launches."""
    val, rp, col, y = _full_data("c5")
    _check_boosted_round(T, val, rp, col, y, 100000, objective="multi:softmax", depth=8, max_num_bin=255)


def test_full_size_oracle_config5_softmax(T):
    """1 M x 54, 8 classes, depth 8 against the oracle at the full shape: the eight class trees of the first and of
    the second round (bundled one-hot columns, class trees built by common launches)."""
    val, rp, col, y = _full_data("c5")
    kw = dict(objective="multi:softmax", depth=8, max_num_bin=255, learning_rate=0.3, n_trees=2)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    _, crp, _ = s.cuts()
    assert np.array_equal(s.cuts()[0].view(np.uint32), o.cuts()[0].view(np.uint32)) and np.array_equal(crp, o.cuts()[1])
    assert np.array_equal(s.global_bin_ids(rp, col)[0], o.bin_ids())
    stored = _Stored(rp, col, s.F)
    margins = P.Margins("full_size/config5")
    ties = _oracle_tree_at_full_size(T, s, o, 0, crp, 0.3, margins, stored)
    ties += _oracle_tree_at_full_size(T, s, o, 1, crp, 0.3, margins, stored)
    margins.ties = ties
    margins.report()
    assert ties <= 2
    s.close()


def test_full_size_properties_config3_wide(T):
    """500k x 2000, depth 6: 63 feature blocks per work item, 4 MB of histogram per node."""
    val, rp, col, y = _full_data("c3")
    _check_boosted_round(T, val, rp, col, y, 20000, objective="reg:linear", depth=6, max_num_bin=255)


def test_full_size_oracle_config3_wide(T):
    """500k x 2000, depth 6 against the oracle at the full shape (blocks of 64 features, 510 000 bins): two trees."""
    val, rp, col, y = _full_data("c3")
    kw = dict(objective="reg:linear", depth=6, max_num_bin=255, learning_rate=0.3, n_trees=2)
    s = T.Session(val, rp, col, y, **kw)
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    _, crp, _ = s.cuts()
    assert np.array_equal(s.cuts()[0].view(np.uint32), o.cuts()[0].view(np.uint32)) and np.array_equal(crp, o.cuts()[1])
    stored = _Stored(rp, col, s.F)
    margins = P.Margins("full_size/config3")
    ties = _oracle_tree_at_full_size(T, s, o, 0, crp, 0.3, margins, stored)
    ties += _oracle_tree_at_full_size(T, s, o, 1, crp, 0.3, margins, stored)
    margins.ties = ties
    margins.report()
    assert ties <= 1
    s.close()
    _FULL.clear()


def test_full_size_properties_config4_sparse(T):
    """2 M x 100k CSR with Zipf-distributed feature ids: sparse layout with the LDS head."""
    val, rp, col, y = _full_data("c4")
    _check_boosted_round(T, val, rp, col, y, 100000, objective="binary:logistic", depth=8, max_num_bin=63)


def test_full_size_oracle_config4_sparse(T):
    """2 M x 100k CSR, depth 8, 63 bins against the oracle at the full shape (6.3 M cut points: the oracle keeps the
    reference's histogram of all of them per node): the first tree of the level pass - 981 frequent features through
    tables and byte columns, 99 k rare ones through the sorted pass."""
    val, rp, col, y = _full_data("c4")
    kw = dict(objective="binary:logistic", depth=8, max_num_bin=63, learning_rate=0.3, n_trees=1)
    s = T.Session(val, rp, col, y, **kw)
    assert s.info("sparse_pass") == 1
    o = O.Oracle(val, rp, col, y, **kw).prepare()
    _, crp, _ = s.cuts()
    assert np.array_equal(s.cuts()[0].view(np.uint32), o.cuts()[0].view(np.uint32)) and np.array_equal(crp, o.cuts()[1])
    assert np.array_equal(s.global_bin_ids(rp, col)[0], o.bin_ids())
    stored = _Stored(rp, col, s.F)
    margins = P.Margins("full_size/config4")
    ties = _oracle_tree_at_full_size(T, s, o, 0, crp, 0.3, margins, stored)
    margins.ties = ties
    margins.report()
    assert ties <= 1
    s.close()
    _FULL.clear()


def test_estimator_cross_validation(T):
    """TGBMModel.cv (python/thundergbm/thundergbm.py:223-282): five folds from a seeded permutation; the
    test accuracy of a separable problem is high and below the train accuracy's ceiling of 1."""
    rng = np.random.default_rng(3)
    X = rng.standard_normal((3000, 6)).astype(np.float32)
    y = (X[:, 0] + 0.5 * X[:, 1] > 0).astype(np.float32)
    clf = T.TGBMClassifier(depth=4, n_trees=10, objective="binary:logistic", learning_rate=0.5, verbose=0)
    res = clf.cv(X, y, nfold=5, seed=1)
    assert set(res) == {"train-accuracy-mean", "train-accuracy-std", "test-accuracy-mean", "test-accuracy-std"}
    assert 0.9 < res["test-accuracy-mean"] <= res["train-accuracy-mean"] <= 1.0
    reg = T.TGBMRegressor(depth=4, n_trees=10, objective="reg:linear", learning_rate=0.5, verbose=0)
    yr = (X @ rng.standard_normal(6)).astype(np.float32)
    res = reg.cv(X, yr, nfold=4, shuffle=False)
    assert res["train-RMSE-mean"] < res["test-RMSE-mean"] < float(np.var(yr))


def test_cli_train_and_predict_on_a1a(T, tmp_path):
    """thundergbm-train <conf> + thundergbm-predict <conf> (reference: docs/how-to.md:20-31): LIBSVM
    loader, key=value parser, model file with base score, predictor and metric."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    conf = tmp_path / "machine.conf"
    conf.write_text("data=%s\n" % D.A1A)
    train = os.path.join(root, "thundergbm_amd", "bin", "thundergbm-train")
    predict = os.path.join(root, "thundergbm_amd", "bin", "thundergbm-predict")
    out = subprocess.run([train, str(conf)], capture_output=True, text=True, cwd=tmp_path, timeout=300)
    assert out.returncode == 0, out.stderr
    assert "#instances = 1605, #features = 119" in out.stdout
    assert "[40/40] RMSE = " in out.stdout and "training time = " in out.stdout
    assert os.path.exists(tmp_path / "tgbm.model")
    last = float(out.stdout.split("[40/40] RMSE = ")[1].split()[0])
    # the oracle's value for the current algorithm (with base score) on the same file
    val, rp, col, y = D.read_libsvm(D.A1A)
    o = O.Oracle(val, rp, col, y, depth=6, n_trees=40, learning_rate=1.0).prepare()
    o.boost(40)
    assert abs(last - float(o.metric_log()[-1])) < 2e-4
    out = subprocess.run([predict, str(conf)], capture_output=True, text=True, cwd=tmp_path, timeout=300)
    assert out.returncode == 0, out.stderr
    rmse = float(out.stdout.split("RMSE = ")[-1].split()[0])
    assert abs(rmse - last) < 1e-4  # the predictor on the training file reproduces the training metric
    # command-line overrides and XGBoost aliases (parser.cpp:40-73)
    out = subprocess.run([train, str(conf), "max_depth=3", "num_round=4", "eta=0.5", "objective=binary:logistic",
                          "verbosity=1"], capture_output=True, text=True, cwd=tmp_path, timeout=300)
    assert out.returncode == 0, out.stderr
    assert "[4/4] test error = " in out.stdout


def test_r_entry_points(T, tmp_path):
    """train_R / predict_R (gbm_R_interface.cpp:10-86) the way R's .C() calls them: every argument a pointer,
    strings as char**. The model file they write equals what the estimator saves for the same parameters."""
    L = T.load()
    ci = lambda v: C.byref(C.c_int(v))
    cd = lambda v: C.byref(C.c_double(v))

    def cs(v):
        arr = (C.c_char_p * 1)(str(v).encode())
        return arr

    model_path = tmp_path / "r.model"
    data, obj, method, out = cs(D.A1A), cs("binary:logistic"), cs("hist"), cs(model_path)
    L.train_R(ci(4), ci(6), ci(1), ci(0), ci(0), data, ci(63), cd(1.0), ci(0), ci(1), cd(0.5), obj, ci(2), ci(1),
              cd(1.0), cd(0.5), method, out)
    assert os.path.getsize(model_path) > 0
    m = T.TGBMClassifier(verbose=0)
    m.load_model(str(model_path))
    assert (m.n_trees, m.num_class, m.tree_per_iter) == (6, 2, 1) and abs(m.learning_rate - 0.5) < 1e-7
    val, rp, col, y = D.read_libsvm(D.A1A)
    import scipy.sparse as sp
    X = sp.csr_matrix((val, col, rp), shape=(len(y), 119))
    ref = T.TGBMClassifier(depth=4, n_trees=6, max_num_bin=63, learning_rate=0.5, objective="binary:logistic",
                           gamma=0.5, verbose=0, tree_method="hist").fit(X, y)
    for t in range(6):
        a, b = m.get_trees()[t], ref.get_trees()[t]
        assert np.array_equal(a["feature"], b["feature"]) and np.array_equal(a["threshold"], b["threshold"])
        assert np.array_equal(a["value"], b["value"])
    import subprocess, sys
    code = ("import ctypes as C, thundergbm_amd as T; L = T.load();"
            "L.predict_R((C.c_char_p * 1)(%r.encode()), (C.c_char_p * 1)(%r.encode()), C.byref(C.c_int(1)))")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", code % (D.A1A, str(model_path))], capture_output=True, text=True,
                         cwd=root, timeout=300)
    assert res.returncode == 0, res.stderr
    assert "test error = " in res.stdout
