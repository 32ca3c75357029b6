"""Comparators shared by the GPU parity tests.

Tolerances (north-star statement): cut points, bin ids and node assignments bit-exact; histogram
sums, gains and predictions within 1e-5 relative in an fp64-accumulated comparison; tree structure
identical wherever the gap between competing split gains exceeds that tolerance.
"""
import numpy as np

REL = 1e-5


def node_hist_refs(bins, rows, gh, n_bins, node_of_row, first, count):
    """For the nodes first .. first + count - 1: per-bin sums of |g|, |h| over the node's own rows
    ([count, n_bins, 2]) and the number of stored entries per bin ([count, n_bins])."""
    x = node_of_row[rows] - first
    m = (x >= 0) & (x < count)
    idx = x[m].astype(np.int64) * n_bins + bins[m]
    a = np.abs(gh[rows[m]].astype(np.float64))
    S = np.zeros((count * n_bins, 2))
    S[:, 0] = np.bincount(idx, weights=a[:, 0], minlength=count * n_bins)
    S[:, 1] = np.bincount(idx, weights=a[:, 1], minlength=count * n_bins)
    cnt = np.bincount(idx, minlength=count * n_bins)
    return S.reshape(count, n_bins, 2), cnt.reshape(count, n_bins)


def item_shift(qmax, rows, bits):
    """The library's rule (k_hist_dense): smallest s >= 0 with rows * (qmax / 2^s + 0.5) < 2^bits."""
    lim = 2.0 ** bits / rows * (1 - 1e-6) - 0.5
    if not qmax >= lim:
        return 0
    return int(np.floor(np.log2(qmax / lim))) + 1


def node_quantum(quant, node_rows, sparse):
    """Coarsest (g, h) step at which a row of a node with node_rows rows is counted. The library sums
    round(g * scale) as exact 64-bit integers; a dense work item coarsens the tree's scale by a power of two
    that depends on the rows it adds between two drains of its packed LDS bins (at most min(node rows, flush_rows): 8192 with float hessians, 32768 with integer ones).
    Every histogram built from rows is therefore exact up to half a step per stored entry."""
    qg, qh = float(quant["inv_g"]), float(quant["inv_h"])
    if sparse:
        return np.array([qg, qh])
    r = max(1, min(int(node_rows), int(quant["flush_rows"])))
    sg = item_shift(float(quant["gq_max"]), r, 63 - int(quant["h_bits"]))
    sh = 0 if quant["h_integer"] else item_shift(float(quant["hq_max"]), r, int(quant["h_bits"]))
    return np.array([qg * 2.0 ** sg, qh * 2.0 ** sh])


def hist_tolerance(S_own, cnt, quantum, rel=REL):
    """rel x (the node's own per-bin sum of |g|, |h|) + half a quantisation step per stored entry of the bin."""
    return rel * S_own + 0.5 * cnt[:, None] * quantum[None, :]


def assert_hist_close(got, ref64, tol, what=""):
    err = np.abs(got.astype(np.float64) - ref64)
    bad = err > tol + 1e-30
    assert not bad.any(), "%s: %d bins off, worst err/tol %.3g" % (
        what, int(bad.sum()), float((err / np.maximum(tol, 1e-300)).max()))
    return err


def sum_bounds(abs_scale, rel=REL):
    """Bounds on a node's gradient / hessian sum: node sums are float32 results of a chain of histogram
    subtractions that starts at the root, so their error is relative to the root-level sums of |g| and |h|."""
    return rel * abs_scale[0] + 1e-7, rel * abs_scale[1] + 1e-7


def gain_tolerance(weights, gain, dG, dH, rel=REL):
    """First-order propagation of |dG|, |dH| into a gain built from the terms G^2 / (H + lambda) of the nodes with
    the given weights w = -G / (H + lambda): d term / dG = -2 w, d term / dH = -w^2."""
    return sum(2 * abs(w) * dG + w * w * dH for w in weights) + rel * max(1.0, abs(float(gain)))


def gain_scale(node_sum, left_sum, lam):
    """Magnitude of the three terms whose difference is the gain."""
    fg, fh = node_sum
    lg, lh = left_sum
    rg, rh = fg - lg, fh - lh
    return lg * lg / (lh + lam) + rg * rg / (rh + lam) + fg * fg / (fh + lam)


class TreeDiff:
    def __init__(self):
        self.compared = 0
        # (node, oracle best |gain|, oracle |gain| of the GPU's choice, magnitude of the oracle gain's terms)
        self.near_ties = []
        # (node, feature) of nodes whose few rows without the split feature took different default directions
        self.direction_ties = []
        # largest observed error / tolerance of the compared node sums, weights and gains (how much of the bound
        # the two implementations actually use)
        self.worst = {"sum": 0.0, "weight": 0.0, "gain": 0.0}

    def __repr__(self):
        return "TreeDiff(compared=%d, near_ties=%r, worst=%r)" % (self.compared, self.near_ties, self.worst)


class Margins:
    """Running maximum of error / tolerance per quantity over the comparisons of a test; report() prints it and,
    when TGBM_MARGIN_LOG names a file, appends a line there."""

    def __init__(self, name):
        self.name = name
        self.worst = {}
        self.ties = 0

    def add(self, diff_or_dict):
        w = diff_or_dict.worst if hasattr(diff_or_dict, "worst") else diff_or_dict
        for k, v in w.items():
            self.worst[k] = max(self.worst.get(k, 0.0), float(v))

    def note(self, key, err, tol):
        r = float(np.max(np.asarray(err, np.float64) / np.maximum(np.asarray(tol, np.float64), 1e-300))) if np.size(err) else 0.0
        self.worst[key] = max(self.worst.get(key, 0.0), r)

    def report(self):
        import json
        import os
        line = json.dumps({"case": self.name, "ties": self.ties,
                           "worst_err_over_tol": {k: float("%.3g" % v) for k, v in sorted(self.worst.items())}})
        print("\nmargins " + line, flush=True)
        path = os.environ.get("TGBM_MARGIN_LOG")
        if path:
            with open(path, "a") as f:
                f.write(line + "\n")


class FullScores:
    """The oracle's candidate gains of one tree as compare_trees reads them, from the complete debug arrays
    (Oracle.tree_scores(), Oracle.tree_dir_gaps(): [n_nodes, n_bins])."""

    def __init__(self, scores, dir_gaps=None):
        self.scores, self.dir_gaps = scores, dir_gaps

    def best(self, x):
        return float(np.abs(self.scores[x]).max())

    def of(self, x, idx):
        return abs(float(self.scores[x][idx]))

    def dir_gap(self, x, idx):
        return None if self.dir_gaps is None else abs(float(self.dir_gaps[x][idx]))


class ProbeScores:
    """The same from probes (Oracle.set_probes / probes()): per node the gain of one named candidate - the GPU's
    choice - and of the oracle's best; for data whose n_nodes x n_bins arrays would take gigabytes."""

    def __init__(self, probe, out):
        self.probe, self.out = probe, out

    def best(self, x):
        return float(self.out[x]["best"])

    def of(self, x, idx):
        assert int(self.probe[x]) == int(idx), "node %d: candidate %d was not probed (%d was)" % (x, idx, self.probe[x])
        return abs(float(self.out[x]["score"]))

    def dir_gap(self, x, idx):
        if int(self.probe[x]) == int(idx):
            return abs(float(self.out[x]["dir_gap"]))
        return abs(float(self.out[x]["best_dir_gap"]))  # (only asked for the oracle's own choice)


def probes_for(gpu, crp):
    """The GPU tree's chosen candidate per node as a global bin index (-1 where it did not split)."""
    fid = gpu["split_fid"].astype(np.int64)
    idx = np.asarray(crp)[np.maximum(fid, 0)].astype(np.int64) + gpu["split_bid"].astype(np.int64)
    return np.where((fid >= 0) & (gpu["is_valid"] == 1), idx, -1).astype(np.int32)


def significant_ties(near_ties):
    """Near ties that are more than float round-off between two candidates: candidates that cut a node's rows into
    the same two sets have equal gains in exact arithmetic, and which of them a float implementation prefers is
    decided by the order of its additions (in the reference: by the order of its atomics)."""
    return [t for t in near_ties if not t[1] - t[2] <= 2e-6 * max(t[1], t[3])]


def rows_in_node(final_nid, x):
    """Mask of the rows whose path from the root passes through heap node x."""
    cur = np.asarray(final_nid).copy()
    while True:
        above = cur > x
        if not above.any():
            break
        cur[above] = (cur[above] - 1) // 2
    return cur == x


def compare_trees(gpu, orc, lam, crp=None, orc_scores=None, missing_rows=None, abs_scale=None, rel=REL, mcw=1.0,
                  orc_dir_gaps=None, few_missing_rows=0, gamma=1.0):
    """Top-down comparison of two heap-ordered trees (NODE_DTYPE arrays).

    Where both trees split on the same candidate everything must agree: threshold and bin exactly,
    gain / child sums / weights to tolerance. Where the choice differs, the oracle's own gain of the
    GPU's candidate must be within tolerance of the oracle's best (a near tie); the subtree below
    such a node is not compared. `default_right` is only compared where
    missing_rows(node, feature) > 0: without missing rows in the node the reference decides it by
    float32 round-off of node_sum - feature_total. Where the node has missing rows the direction is the
    larger of two gains of the same candidate (missing -> left against missing -> right, strict `>`,
    hist_tree_builder_single.cu:300-323); orc_dir_gaps [n_nodes, n_bins] holds the oracle's difference of the
    two, and a direction that differs is a near tie like any other when that difference is within the gain
    tolerance (without orc_dir_gaps a differing direction fails). Such a node's subtree is not compared either -
    unless the node has at most few_missing_rows rows without the feature (a handful of exact zeros in ten million
    rows of continuous data): those few rows cannot move a sum beyond its bound, so the comparison goes on below the
    node and the node is listed in TreeDiff.direction_ties, for the caller to excuse exactly those rows from the
    comparison of the row -> node maps.

    Tolerance: node sums are float32 results of a chain of histogram subtractions that starts at the
    root, so their error is relative to the root-level sums of |g| and |h| (abs_scale = (Ag, Ah)):
    |dG| <= rel * Ag, |dH| <= rel * Ah. Weights and gains get the first-order propagation of those
    two bounds (w = -G/(H+lam); d gain/dG = -2w, d gain/dH = -w^2 per term).
    A choice that differs is also accepted as a near tie when one side's chosen split has a child whose
    hessian sum sits within dH of min_child_weight (mcw): that gate (hist_tree_builder_single.cu
    compute_gain: both children need h >= min_child_weight) flips on the last ulps of a sum, e.g. four
    logistic rows with p = 0.5 give exactly 4 * 0.25 = 1.0 or one ulp less depending on the order. The same gate
    decides between the two default directions of one candidate (the direction whose child falls below it is not
    a candidate), so a direction that differs on the gate is a near tie as well, whatever the two gains.
    Pruning compares a node's gain with gamma (tree.cu:96-128): a node that only one side pruned is a near tie too
    when its gain is within its tolerance of gamma (the flags and final ids of the trees are then not compared).
    orc_scores: [n_nodes, n_bins] signed candidate gains of the oracle, or a FullScores / ProbeScores view of them
    (None forbids any mismatch); crp: cut_row_ptr, to turn (feature, local bin) into a global candidate index.
    """
    diff = TreeDiff()
    stack = [0]
    view = orc_scores
    if orc_scores is not None and not hasattr(orc_scores, "best"):
        view = FullScores(orc_scores, orc_dir_gaps)
    if abs_scale is None:
        abs_scale = (max(1.0, abs(float(orc[0]["sum_g"])) + float(orc[0]["sum_h"])),) * 2
    dG, dH = sum_bounds(abs_scale, rel)

    def gain_tol(x, o):
        ws = [float(orc[x]["base_weight"])]
        if o["lch"] >= 0:
            ws += [float(orc[o["lch"]]["base_weight"]), float(orc[o["rch"]]["base_weight"])]
        return gain_tolerance(ws, o["gain"], dG, dH, rel)

    def on_mcw_gate(x, split_g, split_o):
        on_gate = False
        for t, has in ((gpu, split_g), (orc, split_o)):
            if has:
                hmin = min(float(t[int(t[x]["lch"])]["sum_h"]), float(t[int(t[x]["rch"])]["sum_h"]))
                on_gate |= abs(hmin - mcw) <= dH
        return on_gate

    while stack:
        x = stack.pop()
        g, o = gpu[x], orc[x]
        assert bool(g["is_valid"]) == bool(o["is_valid"]), "node %d validity differs" % x
        if not o["is_valid"]:
            continue
        diff.compared += 1
        S = (float(o["sum_g"]), float(o["sum_h"]))
        assert abs(g["sum_g"] - o["sum_g"]) <= dG and abs(g["sum_h"] - o["sum_h"]) <= dH, \
            "node %d sum differs: gpu (%g,%g) oracle (%g,%g)" % (x, g["sum_g"], g["sum_h"], o["sum_g"], o["sum_h"])
        diff.worst["sum"] = max(diff.worst["sum"], abs(float(g["sum_g"]) - float(o["sum_g"])) / dG,
                                abs(float(g["sum_h"]) - float(o["sum_h"])) / dH)
        w = float(o["base_weight"])
        w_tol = (dG + abs(w) * dH) / (S[1] + lam) + rel * max(1.0, abs(w))
        assert abs(g["base_weight"] - w) <= w_tol, "node %d weight differs: %g vs %g" % (x, g["base_weight"], w)
        diff.worst["weight"] = max(diff.worst["weight"], abs(float(g["base_weight"]) - w) / w_tol)
        split_g, split_o = g["split_fid"] >= 0, o["split_fid"] >= 0
        if not split_g and not split_o:
            continue
        if split_g and split_o and g["split_fid"] == o["split_fid"] and g["split_bid"] == o["split_bid"]:
            assert g["split_value"] == o["split_value"], "node %d threshold differs" % x
            gt = gain_tol(x, o)
            n_missing = 0
            if g["default_right"] != o["default_right"] and missing_rows is not None:
                n_missing = missing_rows(x, int(o["split_fid"]))
            if n_missing > 0 and on_mcw_gate(x, True, True):
                diff.near_ties.append((x, float("nan"), float("nan"), 0.0))
                continue
            assert abs(g["gain"] - o["gain"]) <= gt, "node %d gain %g vs %g" % (x, g["gain"], o["gain"])
            diff.worst["gain"] = max(diff.worst["gain"], abs(float(g["gain"]) - float(o["gain"])) / gt)
            if bool(g["is_leaf"]) != bool(o["is_leaf"]) and abs(float(o["gain"]) - gamma) <= gt:  # pruned on one side
                diff.near_ties.append((x, float(o["gain"]), float(o["gain"]), 0.0))
            if n_missing > 0:
                gap = None
                if view is not None and crp is not None:
                    gap = view.dir_gap(x, int(crp[o["split_fid"]]) + int(o["split_bid"]))
                assert gap is not None and gap <= 2 * gt, \
                    "node %d default direction differs (oracle's gain difference between the directions: %r, tol %g)" % (
                        x, gap, 2 * gt)
                if n_missing <= few_missing_rows:
                    diff.direction_ties.append((x, int(o["split_fid"])))
                    stack.extend([int(o["lch"]), int(o["rch"])])
                    continue
                # the missing rows went to different children: nothing below is comparable
                og = float(o["gain"])
                diff.near_ties.append((x, og, og - gap, gain_scale(
                    S, (float(orc[int(o["lch"])]["sum_g"]), float(orc[int(o["lch"])]["sum_h"])), lam)))
                continue
            stack.extend([int(o["lch"]), int(o["rch"])])
            continue
        assert view is not None and crp is not None, "node %d: split differs (gpu f%d b%d, oracle f%d b%d)" % (
            x, g["split_fid"], g["split_bid"], o["split_fid"], o["split_bid"])
        on_gate = on_mcw_gate(x, split_g, split_o)
        best = view.best(x)
        tol = 2 * gain_tol(x, o)
        if split_g:
            alt = view.of(x, int(crp[g["split_fid"]]) + int(g["split_bid"]))
            ok = best - alt <= tol
            msg = "node %d: gpu chose f%d b%d with oracle gain %g, oracle best %g (f%d b%d), tol %g" % (
                x, g["split_fid"], g["split_bid"], alt, best, o["split_fid"], o["split_bid"], tol)
        else:
            alt = 0.0  # gpu made a leaf where the oracle split: the gain must sit at the rt_eps edge
            ok = best <= 1e-6 + tol
            msg = "node %d: gpu leaf, oracle split gain %g" % (x, best)
        if not ok:
            assert on_gate, msg
            diff.near_ties.append((x, float("nan"), float("nan"), 0.0))
            continue
        # magnitude of the three terms whose difference the gain is (float cancellation noise scales with it)
        terms = gain_scale(S, (float(orc[int(o["lch"])]["sum_g"]), float(orc[int(o["lch"])]["sum_h"])), lam) if split_o else 0.0
        diff.near_ties.append((x, best, alt, terms))
    if not diff.near_ties and not diff.direction_ties:
        for key in ("is_leaf", "is_pruned", "final_id", "lch", "rch", "parent"):
            valid = orc["is_valid"] == 1
            assert np.array_equal(gpu[key][valid], orc[key][valid]), "field %s differs" % key
    return diff


def leaf_of(nodes, nid):
    """Unpruned leaf of every row (climbs pruned nodes, like predict_in_training)."""
    cur = np.asarray(nid).copy()
    while True:
        pr = nodes["is_pruned"][cur] == 1
        if not pr.any():
            return cur
        cur[pr] = nodes["parent"][cur[pr]]


def pred_tolerance(nodes, nid, lr, lam, abs_scale, y_pred, rel=REL):
    """Per-row bound on the prediction update lr * w(leaf) given the node-sum bounds of compare_trees."""
    leaf = leaf_of(nodes, nid)
    w = np.abs(nodes["base_weight"][leaf].astype(np.float64))
    H = nodes["sum_h"][leaf].astype(np.float64)
    dG, dH = sum_bounds(abs_scale, rel)
    return lr * ((dG + w * dH) / (H + lam) + rel * np.maximum(1.0, w)) + rel * np.abs(y_pred) + 1e-6
