"""Pins the CPU oracle (oracle/tgbm_oracle.cpp) without running the reference: closed forms,
brute force on small inputs, invariants, and the reference's own fixture / known answers."""
import os

import numpy as np
import pytest

import datasets as D
import oracle_lib as O


# ------------------------------------------------------------------------------------------ a1 cuts
def _cuts_closed_form(values, max_bin):
    u = np.unique(np.asarray(values, dtype=np.float32))
    step = len(u) // max_bin
    if step == 0:
        return u
    return u[np.arange(max_bin) * step]


@pytest.mark.parametrize("m,max_bin", [(5, 255), (254, 255), (255, 255), (256, 255), (509, 255), (510, 255),
                                       (1000, 255), (1000, 63), (7, 2), (1, 255)])
def test_cut_rule_single_feature(m, max_bin):
    rng = np.random.default_rng(m)
    u = np.sort(rng.choice(100000, size=m, replace=False)).astype(np.float32) / 7
    vals = rng.permutation(np.concatenate([u, u[: m // 2]]))  # duplicates must not matter
    cv, crp, cf = O.cut_points(vals, np.zeros(len(vals), np.int32), 1, max_bin)
    exp = _cuts_closed_form(vals, max_bin)
    assert np.array_equal(cv, exp)
    assert crp.tolist() == [0, len(exp)]
    assert np.all(cf == 0)
    assert cv[0] == vals.min()  # the minimum is always a cut
    assert len(cv) <= max_bin


def test_cut_rule_known_indices():
    # 1000 uniques, 255 bins -> step 3 -> indices 0,3,...,762
    vals = np.arange(1000, dtype=np.float32)
    cv, _, _ = O.cut_points(vals, np.zeros(1000, np.int32), 1, 255)
    assert np.array_equal(cv, np.arange(255, dtype=np.float32) * 3)
    assert cv[-1] == 762


def test_cuts_multi_feature_and_empty_features():
    rng = np.random.default_rng(0)
    F = 6
    col = rng.integers(0, F, size=4000).astype(np.int32)
    col[col == 2] = 3  # feature 2 has no stored value
    val = np.round(rng.standard_normal(4000), 1).astype(np.float32)
    cv, crp, cf = O.cut_points(val, col, F, 16)
    assert crp[2] == crp[3]
    for f in range(F):
        exp = _cuts_closed_form(val[col == f], 16) if np.any(col == f) else np.zeros(0, np.float32)
        assert np.array_equal(cv[crp[f]:crp[f + 1]], exp)
        assert np.all(cf[crp[f]:crp[f + 1]] == f)
        seg = cv[crp[f]:crp[f + 1]]
        assert np.all(np.diff(seg) > 0)
        assert np.all(np.isin(seg, val[col == f]))


def test_cuts_a1a_fixture():
    val, row_ptr, col, y = D.read_libsvm(D.A1A)
    # loader facts asserted by the reference: src/test/test_dataset.cpp:178-181
    assert len(y) == 1605 and col.max() + 1 == 119 and y[0] == -1 and val[1] == 1
    cv, crp, cf = O.cut_points(val, col, 119, 255)
    present = np.unique(col)
    assert len(cv) == len(present)
    assert np.all(cv == 1.0)
    assert np.array_equal(cf, present)


# --------------------------------------------------------------------------------------- a2 bin ids
def test_bin_ids_bruteforce():
    rng = np.random.default_rng(1)
    F = 5
    n = 3000
    col = rng.integers(0, F, size=n).astype(np.int32)
    val = np.round(rng.standard_normal(n) * 3, 1).astype(np.float32)
    col[:50] = 4
    val[:50] = 2.5  # a feature region with one unique value among others
    for max_bin in (4, 16, 255):
        cv, crp, cf = O.cut_points(val, col, F, max_bin)
        got = O.bin_ids(val, col, cv, crp)
        for i in range(n):
            f = col[i]
            cuts = cv[crp[f]:crp[f + 1]]
            k = len(cuts)
            local = min(int(np.sum(cuts <= val[i])), k - 1)
            assert got[i] == crp[f] + local
        # searchsorted formulation
        for f in range(F):
            cuts = cv[crp[f]:crp[f + 1]]
            m = col == f
            exp = np.minimum(np.searchsorted(cuts, val[m], side="right"), len(cuts) - 1) + crp[f]
            assert np.array_equal(got[m], exp)


def test_bin_ids_single_cut_and_never_bin0():
    # k == 1 -> everything in bin 0; k >= 2 -> local bin 0 is never produced (values >= min cut)
    val = np.array([1, 1, 1, 5, 6, 7, 8, 9], np.float32)
    col = np.array([0, 0, 0, 1, 1, 1, 1, 1], np.int32)
    cv, crp, cf = O.cut_points(val, col, 2, 255)
    b = O.bin_ids(val, col, cv, crp)
    assert b[:3].tolist() == [0, 0, 0]
    assert b[3:].tolist() == [1 + 1, 1 + 2, 1 + 3, 1 + 4, 1 + 4]  # top two ranges share the last bin


def test_bin_ids_monotone():
    rng = np.random.default_rng(2)
    val = np.sort(rng.standard_normal(5000).astype(np.float32))
    col = np.zeros(5000, np.int32)
    cv, crp, _ = O.cut_points(val, col, 1, 63)
    b = O.bin_ids(val, col, cv, crp)
    assert np.all(np.diff(b) >= 0)
    assert b.max() == len(cv) - 1


# ------------------------------------------------------------------------------------- a3 gradients
def test_gradient_squared_exact():
    rng = np.random.default_rng(3)
    y = rng.standard_normal(1000).astype(np.float32)
    yp = rng.standard_normal(1000).astype(np.float32)
    gh = O.gradient("reg:linear", y, yp)
    assert np.array_equal(gh[:, 0], yp - y)
    assert np.all(gh[:, 1] == 1)


def test_gradient_logistic_closed_form():
    rng = np.random.default_rng(4)
    y = (rng.random(2000) < 0.5).astype(np.float32)
    yp = (rng.standard_normal(2000) * 4).astype(np.float32)
    yp[:3] = [-60, 60, 0]
    gh = O.gradient("binary:logistic", y, yp)
    p = 1 / (1 + np.exp(-yp.astype(np.float64)))
    np.testing.assert_allclose(gh[:, 0], p - y, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gh[:, 1], np.maximum(p * (1 - p), 1e-16), rtol=1e-4, atol=2e-7)  # 1-p cancels in fp32
    assert gh[:, 1].min() >= np.float32(1e-16)


def test_gradient_softmax_closed_form():
    rng = np.random.default_rng(5)
    n, K = 500, 8
    y = rng.integers(0, K, size=n).astype(np.float32)
    yp = (rng.standard_normal((K, n)) * 3).astype(np.float32)
    gh = O.gradient("multi:softmax", y, yp.ravel(), num_class=K).reshape(K, n, 2)
    z = yp.astype(np.float64)
    p = np.exp(z - z.max(axis=0))
    p /= p.sum(axis=0)
    onehot = (np.arange(K)[:, None] == y[None, :]).astype(np.float64)
    np.testing.assert_allclose(gh[:, :, 0], p - onehot, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gh[:, :, 1], np.maximum(2 * p * (1 - p), 1e-16), rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(gh[:, :, 0].sum(axis=0), 0, atol=1e-5)  # gradients of a softmax sum to zero


def test_group_label():
    y = np.array([3, -1, 3, 7, -1, 7, 7], np.float32)
    ym, lab = O.group_label(y)
    assert lab.tolist() == [-1, 3, 7]
    assert ym.tolist() == [1, 0, 1, 2, 0, 2, 2]


# ------------------------------------------------------------------------------ a12 metrics (KATs)
def test_metric_known_answers():
    # src/test/test_metrics.cpp:58-97: the first four a1a labels are all -1
    _, _, _, y = D.read_libsvm(D.A1A)
    y4 = y[:4]
    assert np.all(y4 == -1)
    yp = np.zeros(8, np.float32)
    yp[0] = 1
    assert O.metric_score("multi:softmax", y4, yp, num_class=2) == 0  # :70
    yp = np.zeros(4, np.float32)
    yp[0] = 1
    assert O.metric_score("binary:logistic", y4, yp, num_class=2) == 1  # :84
    assert O.metric_score("reg:linear", y4, np.zeros(4, np.float32)) == 1  # :96


def test_metric_values():
    rng = np.random.default_rng(6)
    y = rng.standard_normal(100).astype(np.float32)
    yp = rng.standard_normal(100).astype(np.float32)
    np.testing.assert_allclose(O.metric_score("reg:linear", y, yp),
                               np.sqrt(np.mean((yp.astype(np.float64) - y) ** 2)), rtol=1e-5)
    yb = (rng.random(100) < 0.5).astype(np.float32)
    np.testing.assert_allclose(O.metric_score("binary:logistic", yb, yp, 2), 1 - np.mean((yp > 0) == yb), rtol=1e-6)
    K = 4
    ypk = rng.standard_normal((K, 100)).astype(np.float32)
    yk = rng.integers(0, K, 100).astype(np.float32)
    np.testing.assert_allclose(O.metric_score("multi:softmax", yk, ypk.ravel(), K),
                               np.mean(ypk.argmax(axis=0) == yk), rtol=1e-6)


# -------------------------------------------------------------------------------------- tree init
def test_tree_init_layout():
    X, y = D.config1(200, 3)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=6).prepare()
    o.compute_gradient()
    o.tree_init(0)
    nodes = o.nodes()
    assert len(nodes) == 127  # src/test/test_tree.cpp:68
    assert nodes[5]["final_id"] == 5 and nodes[1]["split_fid"] == -1  # :72-73
    assert nodes[0]["is_valid"] == 1 and not nodes[1:]["is_valid"].any()
    assert np.all(nodes[:63]["is_leaf"] == 0) and np.all(nodes[63:]["is_leaf"] == 1)
    assert np.array_equal(nodes[:63]["lch"], 2 * np.arange(63) + 1)
    assert np.all(nodes[63:]["lch"] == -1)
    assert nodes[0]["parent"] == -1 and np.array_equal(nodes[1:]["parent"], (np.arange(1, 127) - 1) // 2)
    gh = o.gh().astype(np.float64)
    np.testing.assert_allclose(nodes[0]["sum_g"], gh[:, 0].sum(), rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(nodes[0]["sum_h"], 200)
    np.testing.assert_allclose(nodes[0]["base_weight"], -gh[:, 0].sum() / (200 + 1), rtol=1e-4, atol=1e-6)


# ------------------------------------------------------------------- a5 histogram + split (brute)
def _brute_best_split(X_present, Xv, gh, cut_val, crp, mcw, lam):
    """Enumerate (feature, candidate bin, default direction) from ROWS in float64.
    X_present[i,f]: value stored; Xv: values. Candidate j of feature f sends present rows whose
    clamped-upper-bound bin is < j to the left. Returns per-candidate signed score (+ = default left)."""
    n, F = Xv.shape
    G, H = gh[:, 0].sum(), gh[:, 1].sum()

    def gain(lg, lh):
        rg, rh = G - lg, H - lh
        if lh >= mcw and rh >= mcw:
            return lg * lg / (lh + lam) + rg * rg / (rh + lam) - G * G / (H + lam)
        return 0.0

    scores = np.zeros(crp[-1])
    for f in range(F):
        cuts = cut_val[crp[f]:crp[f + 1]]
        k = len(cuts)
        if k == 0:
            continue
        pres = X_present[:, f]
        local = np.minimum(np.searchsorted(cuts, Xv[:, f], side="right"), k - 1)
        mg, mh = gh[~pres, 0].sum(), gh[~pres, 1].sum()
        for j in range(k):
            left = pres & (local < j)
            lg, lh = gh[left, 0].sum(), gh[left, 1].sum()
            gr = max(0.0, gain(lg, lh))
            gl = max(0.0, gain(lg + mg, lh + mh))
            scores[crp[f] + j] = gl if gl > gr else -gr
    return scores


def _make_missing_dataset(n, F, seed, frac_missing=0.3, round_to=1):
    rng = np.random.default_rng(seed)
    X = np.round(rng.standard_normal((n, F)) * 2, round_to).astype(np.float32)
    X[X == 0] = 0.5
    miss = rng.random((n, F)) < frac_missing
    miss[:, 0] = False  # one fully dense feature
    X[miss] = 0
    y = (X[:, 0] * 1.5 - X[:, 1] + rng.standard_normal(n) * 0.3).astype(np.float32)
    return X, y


@pytest.mark.parametrize("objective", ["reg:linear", "binary:logistic"])
def test_root_hist_and_split_bruteforce(objective):
    n, F = 400, 4
    X, y = _make_missing_dataset(n, F, 7)
    if objective == "binary:logistic":
        y = (y > 0).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=3, max_num_bin=8, objective=objective, debug=True, shadow64=True,
                 min_child_weight=1.0, lambda_=1.0).prepare()
    cv, crp, cf = o.cuts()
    o.compute_gradient()
    gh = o.gh()[:n]
    o.tree_init(0)
    o.find_split(0)
    h32, h64 = o.level_hist(0)
    # brute-force histogram in float64 straight from the matrix
    bins = o.bin_ids()
    exp = np.zeros((o.n_bins, 2))
    rows = np.repeat(np.arange(n), np.diff(rp))
    np.add.at(exp, bins, gh[rows].astype(np.float64))
    np.testing.assert_allclose(h64, exp, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(h32, exp, rtol=1e-5, atol=1e-4)
    if objective == "reg:linear":
        assert np.array_equal(h32[:, 1], np.bincount(bins, minlength=o.n_bins).astype(np.float32))
    # per feature: sum of bins + missing == node sum
    nodes = o.nodes()
    for f in range(F):
        tot = exp[crp[f]:crp[f + 1]].sum(axis=0)
        missing = gh[X[:, f] == 0].astype(np.float64).sum(axis=0)
        np.testing.assert_allclose(tot + missing, [nodes[0]["sum_g"], nodes[0]["sum_h"]], rtol=1e-4, atol=1e-3)
    # brute-force split enumeration
    scores = _brute_best_split(X != 0, X, gh.astype(np.float64), cv, crp, 1.0, 1.0)
    got = o.tree_scores()[0]
    np.testing.assert_allclose(np.abs(got), np.abs(scores), rtol=2e-4, atol=2e-4)
    sp = o.splits()[0]
    best = int(np.argmax(np.abs(scores)))  # numpy argmax: first max -> smallest index on ties
    assert abs(abs(scores[sp["best_index"]]) - abs(scores[best])) <= 2e-4 * max(1, abs(scores[best]))
    assert sp["fid"] == cf[sp["best_index"]]
    assert sp["bid"] == sp["best_index"] - crp[sp["fid"]]
    # direction sign agrees wherever the two directions differ by more than noise
    f = sp["fid"]
    if np.any(X[:, f] == 0):
        assert sp["default_right"] == int(scores[sp["best_index"]] < 0)
    # threshold: previous cut, or below the minimum for the first bin
    if sp["bid"] == 0:
        c0 = cv[crp[f]]
        assert sp["fval"] == np.float32(np.float64(np.float32(c0 - abs(c0))) - 1e-5)
        assert sp["fval"] < c0
    else:
        assert sp["fval"] == cv[sp["best_index"] - 1]


def test_split_tie_break_and_first_bin_equivalence():
    # local bin 0 is never populated when a feature has >= 2 cuts, so candidates 0 and 1 of every
    # feature have identical gain and the smaller index wins
    X, y = D.config1(300, 2, seed=11)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=2, max_num_bin=6, debug=True).prepare()
    o.compute_gradient()
    o.tree_init(0)
    o.find_split(0)
    sc = o.tree_scores()[0]
    cv, crp, cf = o.cuts()
    for f in range(2):
        assert sc[crp[f]] == sc[crp[f] + 1]
    sp = o.splits()[0]
    best = np.flatnonzero(np.abs(sc) == np.abs(sc).max())[0]
    assert sp["best_index"] == best


def test_min_child_weight_gate():
    X, y = D.config1(50, 2, seed=12)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=2, max_num_bin=8, min_child_weight=30.0, debug=True).prepare()
    o.compute_gradient()
    o.tree_init(0)
    o.find_split(0)
    sc = o.tree_scores()[0]
    h32, _ = o.level_hist(0)
    cv, crp, cf = o.cuts()
    for f in range(2):
        left_h = np.concatenate([[0], np.cumsum(h32[crp[f]:crp[f + 1], 1])[:-1]])
        bad = (left_h < 30) | (50 - left_h < 30)
        assert np.all(sc[crp[f]:crp[f + 1]][bad] == 0)


# ------------------------------------------------- a6..a8 levels: subtraction, partition, counts
def test_levels_sibling_subtraction_and_partition():
    n, F = 600, 5
    X, y = _make_missing_dataset(n, F, 21)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=4, max_num_bin=16, gamma=0.0, debug=True, shadow64=True).prepare()
    cv, crp, cf = o.cuts()
    bins = o.bin_ids()
    o.compute_gradient()
    gh = o.gh().astype(np.float64)
    o.tree_init(0)
    rows = np.repeat(np.arange(n), np.diff(rp))
    for level in range(4):
        nid_before = o.nid()
        o.find_split(level)
        o.update_tree()
        nodes = o.nodes()
        off = (1 << level) - 1
        # every node of the level: histogram == brute force over its rows (built or subtracted)
        for x in range(1 << level):
            h32, h64 = o.level_hist(x)
            m = nid_before[rows] == off + x
            exp = np.zeros((o.n_bins, 2))
            np.add.at(exp, bins[m], gh[rows[m]])
            if nodes[off + x]["is_valid"] and (nid_before == off + x).any():
                np.testing.assert_allclose(h64, exp, atol=1e-9)
                np.testing.assert_allclose(h32, exp, atol=2e-3)
        has = o.update_ins2node()
        nid_after = o.nid()
        for i in range(n):
            x = nid_before[i]
            nd = nodes[x]
            if nd["is_leaf"] or not nd["is_valid"]:
                assert nid_after[i] == x
                continue
            f = nd["split_fid"]
            v = X[i, f]
            if v == 0:  # missing
                assert nid_after[i] == (nd["rch"] if nd["default_right"] else nd["lch"])
            else:  # bins and thresholds are consistent: left iff value < split_value
                assert nid_after[i] == (nd["lch"] if v < nd["split_value"] else nd["rch"])
        # squared loss: hessian sum of a child == its row count
        for x in range(off, off + (1 << level)):
            nd = nodes[x]
            if nd["is_valid"] and not nd["is_leaf"]:
                assert round(float(nodes[nd["lch"]]["sum_h"])) == int((nid_after == nd["lch"]).sum())
                assert round(float(nodes[nd["rch"]]["sum_h"])) == int((nid_after == nd["rch"]).sum())
                # child weights
                for c in (nd["lch"], nd["rch"]):
                    np.testing.assert_allclose(nodes[c]["base_weight"], -nodes[c]["sum_g"] / (nodes[c]["sum_h"] + 1),
                                               rtol=1e-6)
        if not has:
            break
    _, _, built = o.tree_hists()
    nodes = o.nodes()
    # the built sibling is the one with fewer rows (ties: left)
    final_nid = o.nid()
    assert built[0] == 1


def test_smaller_sibling_is_built():
    n, F = 500, 3
    X, y = D.config1(n, F, seed=5)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=3, max_num_bin=32, gamma=0.0, debug=True).prepare()
    o.compute_gradient()
    o.tree_init(0)
    counts = {}
    for level in range(3):
        nid = o.nid()
        for x in np.unique(nid):
            counts[int(x)] = int((nid == x).sum())
        before = o.rows_built()
        o.find_split(level)
        built_rows = o.rows_built() - before
        if level == 0:
            assert built_rows == n
        else:
            off = (1 << level) - 1
            exp = 0
            for p in range(1 << (level - 1)):
                a, b = counts.get(off + 2 * p, 0), counts.get(off + 2 * p + 1, 0)
                exp += min(a, b)
            assert built_rows == exp
        o.update_tree()
        if not o.update_ins2node():
            break
    _, _, built = o.tree_hists()
    for p in range(1, 4):  # pairs of level 1 and 2
        a, b = 2 * p - 1, 2 * p
        if built[a] < 0:
            continue
        if counts.get(a, 0) <= counts.get(b, 0):
            assert built[a] == 1 and built[b] == 0
        else:
            assert built[a] == 0 and built[b] == 1


# ------------------------------------------------------------------------------------- a9 prune
def _blank_tree(depth):
    nn = (1 << (depth + 1)) - 1
    nodes = np.zeros(nn, dtype=O.NODE_DTYPE)
    for i in range(nn):
        nodes[i]["final_id"] = i
        nodes[i]["split_fid"] = -1
        nodes[i]["parent"] = -1 if i == 0 else (i - 1) // 2
        if i < nn // 2:
            nodes[i]["lch"], nodes[i]["rch"] = 2 * i + 1, 2 * i + 2
        else:
            nodes[i]["is_leaf"] = 1
            nodes[i]["lch"] = nodes[i]["rch"] = -1
    return nodes


def test_prune_hand_built():
    # depth-2 tree, 7 nodes. Root split gain 5, node 1 split gain 0.3, node 2 split gain 2.
    nodes = _blank_tree(2)
    nodes["is_valid"] = 1
    nodes[0]["gain"], nodes[1]["gain"], nodes[2]["gain"] = 5.0, 0.3, 2.0
    out, npruned = O.prune_nodes(nodes, 1.0)
    assert npruned == 2
    assert out[3]["is_pruned"] and out[4]["is_pruned"] and out[1]["is_leaf"]
    assert not out[5]["is_pruned"] and not out[2]["is_leaf"]
    assert out["final_id"][[0, 1, 2, 5, 6]].tolist() == [0, 1, 2, 3, 4]
    # cascade: both subtrees weak and the root weak -> everything collapses into the root
    nodes[0]["gain"], nodes[2]["gain"] = 0.5, 0.1
    out, npruned = O.prune_nodes(nodes, 1.0)
    assert npruned == 6 and out[0]["is_leaf"] and out[1:]["is_pruned"].all()
    # gamma 0 prunes nothing (gain < 0 never holds)
    out, npruned = O.prune_nodes(nodes, 0.0)
    assert npruned == 0 and not out["is_pruned"].any()
    # a weak parent with one non-leaf child is kept
    nodes = _blank_tree(2)
    nodes["is_valid"] = 1
    nodes[0]["gain"], nodes[1]["gain"], nodes[2]["gain"] = 0.1, 3.0, 0.1
    out, npruned = O.prune_nodes(nodes, 1.0)
    assert npruned == 2 and not out[0]["is_leaf"] and out[2]["is_leaf"] and not out[1]["is_leaf"]
    # invalid leaves are ignored
    nodes = _blank_tree(2)
    nodes[[0, 1, 2]]["is_valid"] = 1
    nodes["is_valid"][:3] = 1
    nodes[1]["is_leaf"] = nodes[2]["is_leaf"] = 1
    nodes[0]["gain"] = 0.2
    out, npruned = O.prune_nodes(nodes, 1.0)
    assert npruned == 2 and out[0]["is_leaf"]


# --------------------------------------------------------- end to end: closed form and predictor
def test_two_value_feature_cannot_split():
    x = np.array([1.0] * 30 + [2.0] * 50, np.float32)[:, None]
    y = np.array([0.0] * 30 + [4.0] * 50, np.float32)
    val, rp, col = D.dense_to_csr(x)
    o = O.Oracle(val, rp, col, y, depth=1, n_trees=1, gamma=0.0).prepare()
    assert o.bin_ids().tolist() == [1] * 80  # top two ranges merged: both values in the last bin
    o.boost(1)
    assert o.model()[0, 0][0]["is_leaf"] == 1


def test_three_value_feature_closed_form():
    # values 1,2,3 -> cuts [1,2,3]; bins: 1->1, 2->2, 3->2. Best split separates {1} from {2,3}.
    x = np.array([1.0] * 30 + [2.0] * 25 + [3.0] * 25, np.float32)[:, None]
    y = np.array([0.0] * 30 + [4.0] * 50, np.float32)
    val, rp, col = D.dense_to_csr(x)
    lam = 1.0
    o = O.Oracle(val, rp, col, y, depth=1, n_trees=1, learning_rate=0.5, gamma=0.0, lambda_=lam).prepare()
    base = o.base_score
    o.boost(1)
    nodes = o.model()[0, 0]
    assert not nodes[0]["is_leaf"] and nodes[0]["split_fid"] == 0
    assert nodes[0]["split_bid"] == 2 and nodes[0]["split_value"] == 2.0  # left iff v < 2
    gl, hl = (base - 0.0) * 30, 30.0
    gr, hr = (base - 4.0) * 50, 50.0
    np.testing.assert_allclose(nodes[1]["base_weight"], -gl / (hl + lam), rtol=1e-5)
    np.testing.assert_allclose(nodes[2]["base_weight"], -gr / (hr + lam), rtol=1e-5)
    exp_gain = gl * gl / (hl + lam) + gr * gr / (hr + lam) - (gl + gr) ** 2 / (80 + lam)
    np.testing.assert_allclose(nodes[0]["gain"], exp_gain, rtol=1e-4)
    yp = o.y_pred()
    np.testing.assert_allclose(yp[:30], base + 0.5 * (-gl / (hl + lam)), rtol=1e-5)
    np.testing.assert_allclose(yp[30:], base + 0.5 * (-gr / (hr + lam)), rtol=1e-5)


@pytest.mark.parametrize("objective,K", [("reg:linear", 1), ("binary:logistic", 2), ("multi:softmax", 4)])
def test_predictor_equals_training_prediction(objective, K):
    n, F = 1500, 6
    X, y = _make_missing_dataset(n, F, 31)
    if objective == "binary:logistic":
        y = np.where(y > 0, 1.0, -1.0).astype(np.float32)
    elif objective == "multi:softmax":
        y = np.digitize(y, np.quantile(y, [0.25, 0.5, 0.75])).astype(np.float32) * 2 + 1
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=4, n_trees=6, learning_rate=0.3, objective=objective, num_class=K,
                 max_num_bin=32).prepare()
    o.boost(6)
    model = o.model()
    raw = O.predict_raw(val, rp, col, F, model, 0.3, o.base_score)
    np.testing.assert_allclose(raw, o.y_pred(), rtol=1e-5, atol=1e-5)
    # metric log is monotone-ish and consistent with y_pred
    np.testing.assert_allclose(o.metric_log()[-1], O.metric_score(objective, o.y(), o.y_pred(), o.num_class))
    # transform
    out = O.predict_transform(objective, raw, n, o.num_class, o.labels() if K > 1 else np.zeros(1, np.float32))
    assert len(out) == n
    if objective == "binary:logistic":
        assert set(np.unique(out)) <= {-1.0, 1.0}
        assert np.mean(out == y) > 0.8
    if objective == "multi:softmax":
        assert set(np.unique(out)) <= {1.0, 3.0, 5.0, 7.0}
        assert np.mean(out == y) > 0.6


def test_predictor_stored_infinity_by_hand():
    """One split (feature 1 < 0.5 -> leaf 1.0, else leaf 2.0; default left). The reference's shared-memory path
    (F <= 96) marks missing values with +inf and tests `fval < INFINITY` (predictor.cu:96-118), so a stored +inf or
    NaN follows the default direction there; its binary-search path (wider data, :120-189) compares the stored value:
    +inf and NaN are not less than the threshold and go right. -inf is an ordinary small value in both."""
    nodes = np.zeros((1, 1, 3), dtype=O.NODE_DTYPE)
    nodes["lch"], nodes["rch"], nodes["is_leaf"], nodes["is_valid"] = -1, -1, 1, 1
    root = nodes[0, 0, 0:1]
    root["lch"], root["rch"], root["is_leaf"] = 1, 2, 0
    root["split_fid"], root["split_value"], root["default_right"] = 1, 0.5, 0
    nodes[0, 0, 1]["base_weight"], nodes[0, 0, 2]["base_weight"] = 1.0, 2.0
    vals = np.array([0.0, 1.0, np.inf, np.nan, -np.inf], np.float32)  # one row each: feature 1 only
    rp = np.arange(len(vals) + 1, dtype=np.int32)
    col = np.ones(len(vals), np.int32)
    dense = O.predict_raw(vals, rp, col, 3, nodes, 1.0, 0.0)
    assert dense.tolist() == [1.0, 2.0, 1.0, 1.0, 1.0]
    wide = O.predict_raw(vals, rp, col, 200, nodes, 1.0, 0.0)
    assert wide.tolist() == [1.0, 2.0, 2.0, 2.0, 1.0]
    no_row = O.predict_raw(np.zeros(0, np.float32), np.zeros(2, np.int32), np.zeros(0, np.int32), 3, nodes, 1.0, 0.0)
    assert no_row.tolist() == [1.0]  # not stored: default left


def test_base_score_binary_closed_form():
    rng = np.random.default_rng(8)
    X = rng.standard_normal((500, 3)).astype(np.float32)
    y = (rng.random(500) < 0.3).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, objective="binary:logistic", num_class=2).prepare()
    # gradient at 0: p = .5 -> G = sum(.5 - y), H = n/4 ; w = -G/H ; base = logit(sigmoid(w)) = w
    w = -(0.5 * 500 - y.sum()) / (500 / 4)
    np.testing.assert_allclose(o.base_score, w, rtol=1e-4)
    assert np.all(o.y_pred() == np.float32(o.base_score))


def test_base_score_regression_and_softmax_closed_form():
    """init_base_score: reg:linear starts from -G/max(H, 1e-6) at a zero prediction = mean(y)
    (regression_obj.h:35-53); objectives that do not override it start from 0 (objective_function.h:21-24)."""
    rng = np.random.default_rng(12)
    X = rng.standard_normal((700, 4)).astype(np.float32)
    y = (3.0 + 2.0 * rng.standard_normal(700)).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, objective="reg:linear").prepare()
    np.testing.assert_allclose(o.base_score, y.astype(np.float64).mean(), rtol=1e-6)
    assert np.all(o.y_pred() == np.float32(o.base_score))
    yc = rng.integers(0, 4, 700).astype(np.float32)
    o = O.Oracle(val, rp, col, yc, objective="multi:softmax", num_class=4).prepare()
    assert o.base_score == 0.0
    assert np.all(o.y_pred() == 0.0)


def test_softprob_transform_sums_to_one():
    rng = np.random.default_rng(9)
    raw = rng.standard_normal(5 * 40).astype(np.float32)
    out = O.predict_transform("multi:softprob", raw, 40, 5, np.arange(5, dtype=np.float32)).reshape(5, 40)
    np.testing.assert_allclose(out.sum(axis=0), 1, rtol=1e-5)


def test_a1a_quickstart_known_answer():
    # README.md:76-80 / docs/how-to.md:27-31: defaults (depth 6, 40 trees, lr 1, lambda 1, gamma 1,
    # reg:linear) on a1a print "RMSE = 0.489562". The documented number predates the base-score
    # initialisation (include/thundergbm/booster.h:66-73): starting the whole pipeline (cuts, bins,
    # histograms, splits, partition, prune, prediction update, metric) from a zero prediction
    # reproduces it to all six printed digits; with the base score the current code gives 0.5284.
    val, rp, col, y = D.read_libsvm(D.A1A)
    o = O.Oracle(val, rp, col, y, depth=6, n_trees=40, learning_rate=1.0).prepare()
    o.set_y_pred(np.zeros(len(y), np.float32))
    o.boost(40)
    rmse = float(o.metric_log()[-1])
    assert abs(rmse - 0.489562) < 1.5e-6, rmse
    model = o.model()
    raw = O.predict_raw(val, rp, col, 119, model, 1.0, 0.0)
    np.testing.assert_allclose(O.metric_score("reg:linear", y, raw), 0.489562, atol=2e-6)
    o2 = O.Oracle(val, rp, col, y, depth=6, n_trees=40, learning_rate=1.0).prepare()
    o2.boost(40)
    assert abs(float(o2.metric_log()[-1]) - 0.52842) < 1e-3


def test_column_sampling_ignores_the_shuffled_head():
    """Shard::column_sampling (shard.cu:8-22): with F columns and rate r, max(1, int(F * r)) columns are
    ignored per round and no tree of the round splits on them; rate 1 ignores nothing. The shuffle is
    std::random_shuffle over rand(): two runs from the same srand() seed agree, another seed differs."""
    import ctypes
    libc = ctypes.CDLL(None)
    rng = np.random.default_rng(5)
    n, F = 2000, 10
    X = rng.standard_normal((n, F)).astype(np.float32)
    y = (X @ rng.standard_normal(F) + 0.1 * rng.standard_normal(n)).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    kw = dict(objective="reg:linear", n_trees=6, depth=4, max_num_bin=32, learning_rate=0.5)

    def run(rate, seed):
        o = O.Oracle(val, rp, col, y, **kw).prepare()
        o.set_column_sampling_rate(rate)
        libc.srand(seed)
        o.boost(6)
        m = o.model()
        used = [set(int(f) for f in t[0]["split_fid"][(t[0]["is_valid"] == 1) & (t[0]["split_fid"] >= 0)]) for t in m]
        return m, used

    m_a, used_a = run(0.6, 7)
    m_b, _ = run(0.6, 7)
    m_c, used_c = run(0.6, 8)
    assert m_a.tobytes() == m_b.tobytes()
    assert m_a.tobytes() != m_c.tobytes()
    assert all(len(u) <= F - 6 for u in used_a + used_c)  # int(10 * 0.6) = 6 ignored columns per round
    assert len(set().union(*used_a)) > F - 6  # a fresh sample every round: over 6 rounds more columns appear
    m_full, used_full = run(1.0, 7)
    assert max(len(u) for u in used_full) > 4
    _, used_tiny = run(0.01, 7)  # max(1, int(0.1)) = 1 ignored column
    assert all(len(u) <= F - 1 for u in used_tiny)


# ------------------------------------------------------------------------------------------ bagging
def test_bagging_draws_match_thrust_vectors():
    """RowSampler::do_bagging draws with thrust::default_random_engine and thrust::uniform_int_distribution.
    The vectors were produced with the thrust headers of this image (tests/golden/bagging_thrust_vectors.hip);
    the oracle's restatement (std::minstd_rand + thrust's mapping) must give the same indices."""
    import json
    cases = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                        "bagging_thrust_vectors.json")))
    assert len(cases) == 30
    for c in cases:
        draws = O.bagging_draws(c["seed"], c["N"], max(int(p) for p in c["draws"]) + 1)
        for pos, idx in c["draws"].items():
            assert draws[int(pos)] == idx, (c["seed"], c["N"], pos)


def test_bagging_engine_is_minstd_rand():
    # the C++ standard fixes the 10000th output of minstd_rand (default seed 1) at 399268537; with N = m - 1
    # the distribution's mapping is the identity on (output - 1)
    m = 2147483647
    assert O.bagging_draws(1, m - 1, 10000)[9999] == 399268537 - 1


def test_bagging_scales_gradients_by_draw_counts():
    import ctypes as C
    libc = C.CDLL("libc.so.6")
    libc.rand.restype = C.c_int
    X, y = D.config1(500, 4, seed=3)
    val, rp, col = O.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=3, n_trees=2).prepare()
    o.compute_gradient()
    plain = o.gh().copy()
    o.set_bagging(True)
    libc.srand(42)
    seed = libc.rand()
    libc.srand(42)
    o.compute_gradient()
    counts = np.bincount(O.bagging_draws(seed, 500), minlength=500)
    assert counts.sum() == 500 and counts.max() > 1 and (counts == 0).sum() > 100  # a bootstrap sample
    assert np.array_equal(o.gh(), plain * counts[:, None].astype(np.float32))


def test_probes_equal_the_full_debug_arrays():
    """Oracle.set_probes records, per node, the gain of one named candidate, the node's best gain and the direction
    gaps of both: the same numbers as the [n_nodes, n_bins] debug arrays hold, and the tree is the same."""
    import parity as P
    X, y = D.config1(3000, 8, 0)
    X[np.random.default_rng(1).random(X.shape) < 0.2] = 0  # missing values: direction gaps that are not round-off
    val, rp, col = D.dense_to_csr(X)
    o = O.Oracle(val, rp, col, y, depth=5, n_trees=2, debug=True).prepare()
    o.compute_gradient()
    o.build_tree(0)
    nodes, sc, gaps, crp = o.nodes().copy(), o.tree_scores(), o.tree_dir_gaps(), o.cuts()[1]
    rng = np.random.default_rng(0)
    probe = P.probes_for(nodes, crp)
    assert np.all(probe[(nodes["is_valid"] == 1) & (nodes["split_fid"] >= 0)] >= 0)
    for x in range(0, len(probe), 3):  # some probes on other candidates than the chosen one
        if probe[x] >= 0:
            probe[x] = int(rng.integers(0, o.n_bins))
    o2 = O.Oracle(val, rp, col, y, depth=5, n_trees=2).prepare()
    o2.set_probes(probe)
    o2.compute_gradient()
    o2.build_tree(0)
    _, out = o2.probes()
    assert np.array_equal(o2.nodes(), nodes)
    checked = 0
    for x in np.flatnonzero(nodes["is_valid"] == 1):
        if nodes[x]["lch"] < 0:
            continue  # the deepest level is never evaluated
        assert out[x]["best"] == np.abs(sc[x]).max()
        if probe[x] >= 0:
            assert out[x]["score"] == sc[x][probe[x]] and out[x]["dir_gap"] == gaps[x][probe[x]]
            checked += 1
        if nodes[x]["split_fid"] >= 0:
            assert out[x]["best_dir_gap"] == gaps[x][crp[nodes[x]["split_fid"]] + nodes[x]["split_bid"]]
    assert checked > 10
    view = P.ProbeScores(probe, out)
    full = P.FullScores(sc, gaps)
    x = int(np.flatnonzero(probe >= 0)[0])
    assert view.best(x) == full.best(x) and view.of(x, probe[x]) == full.of(x, probe[x])
