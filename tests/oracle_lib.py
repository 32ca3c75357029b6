"""ctypes binding of the CPU oracle (oracle/liboracle.so). Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(ROOT, "oracle", "liboracle.so")

NODE_DTYPE = np.dtype(
    [
        ("final_id", "<i4"), ("lch", "<i4"), ("rch", "<i4"), ("parent", "<i4"),
        ("gain", "<f4"), ("base_weight", "<f4"), ("split_fid", "<i4"), ("split_value", "<f4"),
        ("split_bid", "u1"), ("default_right", "u1"), ("is_leaf", "u1"), ("is_valid", "u1"),
        ("is_pruned", "u1"), ("pad", "u1", (3,)), ("sum_g", "<f4"), ("sum_h", "<f4"),
    ]
)
assert NODE_DTYPE.itemsize == 48

SPLIT_DTYPE = np.dtype(
    [
        ("gain", "<f4"), ("miss_g", "<f4"), ("miss_h", "<f4"), ("lch_g", "<f4"), ("lch_h", "<f4"),
        ("default_right", "<i4"), ("nid", "<i4"), ("fid", "<i4"), ("fval", "<f4"), ("bid", "<i4"),
        ("best_index", "<i4"), ("pad", "<i4"),
    ]
)
assert SPLIT_DTYPE.itemsize == 48

PROBE_DTYPE = np.dtype([("score", "<f4"), ("dir_gap", "<f4"), ("best", "<f4"), ("best_dir_gap", "<f4")])

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
        L = C.CDLL(_SO)
        L.orc_create.restype = C.c_void_p
        L.orc_create.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                 C.c_float, C.c_float, C.c_float, C.c_int, C.c_float, C.c_char_p, C.c_int]
        for name in ("orc_destroy", "orc_prepare", "orc_compute_gradient", "orc_update_tree"):
            getattr(L, name).argtypes = [C.c_void_p]
            getattr(L, name).restype = None
        L.orc_set_debug.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.orc_boost.argtypes = [C.c_void_p, C.c_int]
        L.orc_set_column_sampling_rate.argtypes = [C.c_void_p, C.c_float]
        L.orc_sample_columns.argtypes = [C.c_void_p]
        L.orc_set_bagging.argtypes = [C.c_void_p, C.c_int]
        L.orc_set_bagging.restype = None
        L.orc_bagging_draws.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.orc_bagging_draws.restype = None
        L.orc_set_groups.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.orc_set_groups.restype = None
        L.orc_rank_gradient.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint,
                                        C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_rank_gradient.restype = None
        L.orc_rank_metric.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.orc_rank_metric.restype = C.c_float
        for name in ("orc_tree_init", "orc_find_split", "orc_predict_in_training", "orc_build_tree"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_int]
            getattr(L, name).restype = None
        for name in ("orc_update_ins2node", "orc_prune", "orc_n_features", "orc_n_bins", "orc_num_class",
                     "orc_tree_per_rounds", "orc_n_labels", "orc_n_nodes", "orc_model_size"):
            getattr(L, name).argtypes = [C.c_void_p]
            getattr(L, name).restype = C.c_int
        for name in ("orc_metric", "orc_base_score"):
            getattr(L, name).argtypes = [C.c_void_p]
            getattr(L, name).restype = C.c_float
        for name in ("orc_rows_built", "orc_y_pred_size"):
            getattr(L, name).argtypes = [C.c_void_p]
            getattr(L, name).restype = C.c_long
        for name in ("orc_get_labels", "orc_get_y", "orc_get_bin_ids", "orc_get_y_pred", "orc_set_y_pred",
                     "orc_get_gh", "orc_set_gh", "orc_get_nid", "orc_set_nid", "orc_get_nodes", "orc_set_nodes",
                     "orc_get_tree_scores", "orc_get_tree_dir_gaps", "orc_get_model"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_void_p]
            getattr(L, name).restype = None
        L.orc_set_probes.argtypes = [C.c_void_p, C.c_void_p]
        L.orc_set_probes.restype = None
        L.orc_get_probes.argtypes = [C.c_void_p, C.c_void_p]
        L.orc_get_probes.restype = None
        L.orc_get_cuts.argtypes = [C.c_void_p] * 4
        L.orc_get_splits.argtypes = [C.c_void_p, C.c_void_p]
        L.orc_get_splits.restype = C.c_int
        L.orc_get_level_hist.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        L.orc_get_tree_hists.argtypes = [C.c_void_p] * 4
        L.orc_get_metric_log.argtypes = [C.c_void_p, C.c_void_p]
        L.orc_get_metric_log.restype = C.c_int
        L.orc_get_rows_built_level.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.orc_get_rows_built_level.restype = C.c_int
        L.orc_cut_points.argtypes = [C.c_int, C.c_long, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                     C.c_void_p]
        L.orc_cut_points.restype = C.c_int
        L.orc_bin_ids.argtypes = [C.c_long] + [C.c_void_p] * 5
        L.orc_gradient.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_metric_score.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.orc_metric_score.restype = C.c_float
        L.orc_prune_nodes.argtypes = [C.c_void_p, C.c_int, C.c_float]
        L.orc_prune_nodes.restype = C.c_int
        L.orc_group_label.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_predict_raw.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                      C.c_int, C.c_int, C.c_float, C.c_float, C.c_void_p]
        L.orc_predict_transform.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.orc_predict_transform.restype = C.c_long
        L.orc_num_threads.restype = C.c_int
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def dense_to_csr(X):
    """The reference wrapper's dense -> CSR rule (python/thundergbm/thundergbm.py:91-93,102-103):
    exact zeros are dropped, values float32, column indices ascending."""
    X = np.asarray(X)
    mask = X != 0
    row_ptr = np.zeros(X.shape[0] + 1, dtype=np.int32)
    np.cumsum(mask.sum(axis=1), out=row_ptr[1:])
    col = np.nonzero(mask)[1].astype(np.int32)
    val = X[mask].astype(np.float32)
    return val, row_ptr, col


class Oracle:
    def __init__(self, val, row_ptr, col, y, depth=6, n_trees=40, min_child_weight=1.0, lambda_=1.0, gamma=1.0,
                 max_num_bin=255, learning_rate=1.0, objective="reg:linear", num_class=1, debug=False,
                 shadow64=False, groups=None):
        self.L = lib()
        self.val = np.ascontiguousarray(val, dtype=np.float32)
        self.row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
        self.col = np.ascontiguousarray(col, dtype=np.int32)
        y = np.ascontiguousarray(y, dtype=np.float32)
        self.n = len(self.row_ptr) - 1
        self.nnz = int(self.row_ptr[-1])
        self.objective = objective
        self.depth = depth
        self.h = self.L.orc_create(self.n, _p(self.val), _p(self.row_ptr), _p(self.col), _p(y), depth, n_trees,
                                   min_child_weight, lambda_, gamma, max_num_bin, learning_rate,
                                   objective.encode(), num_class)
        self.L.orc_set_debug(self.h, int(debug), int(shadow64))
        if groups is not None:
            grp = np.ascontiguousarray(groups, dtype=np.int32)
            self.L.orc_set_groups(self.h, _p(grp), len(grp))
        self.shadow64 = shadow64

    def __del__(self):
        if getattr(self, "h", None):
            self.L.orc_destroy(self.h)
            self.h = None

    # driving
    def prepare(self):
        self.L.orc_prepare(self.h)
        self.F = self.L.orc_n_features(self.h)
        self.n_bins = self.L.orc_n_bins(self.h)
        self.num_class = self.L.orc_num_class(self.h)
        self.tree_per_rounds = self.L.orc_tree_per_rounds(self.h)
        self.n_nodes = self.L.orc_n_nodes(self.h)
        return self

    def set_column_sampling_rate(self, rate):
        self.L.orc_set_column_sampling_rate(self.h, rate)

    def sample_columns(self):
        self.L.orc_sample_columns(self.h)

    def set_bagging(self, on):
        self.L.orc_set_bagging(self.h, int(on))

    def boost(self, rounds=1):
        self.L.orc_boost(self.h, rounds)

    def compute_gradient(self):
        self.L.orc_compute_gradient(self.h)

    def tree_init(self, k=0):
        self.L.orc_tree_init(self.h, k)

    def find_split(self, level):
        self.L.orc_find_split(self.h, level)

    def update_tree(self):
        self.L.orc_update_tree(self.h)

    def update_ins2node(self):
        return self.L.orc_update_ins2node(self.h)

    def prune(self):
        return self.L.orc_prune(self.h)

    def predict_in_training(self, k=0):
        self.L.orc_predict_in_training(self.h, k)

    def build_tree(self, k=0):
        self.L.orc_build_tree(self.h, k)

    def metric(self):
        return self.L.orc_metric(self.h)

    # views
    @property
    def base_score(self):
        return self.L.orc_base_score(self.h)

    def labels(self):
        out = np.zeros(self.L.orc_n_labels(self.h), dtype=np.float32)
        self.L.orc_get_labels(self.h, _p(out))
        return out

    def y(self):
        out = np.zeros(self.n, dtype=np.float32)
        self.L.orc_get_y(self.h, _p(out))
        return out

    def cuts(self):
        cv = np.zeros(self.n_bins, dtype=np.float32)
        crp = np.zeros(self.F + 1, dtype=np.int32)
        cf = np.zeros(self.n_bins, dtype=np.int32)
        self.L.orc_get_cuts(self.h, _p(cv), _p(crp), _p(cf))
        return cv, crp, cf

    def bin_ids(self):
        out = np.zeros(self.nnz, dtype=np.int32)
        self.L.orc_get_bin_ids(self.h, _p(out))
        return out

    def y_pred(self):
        out = np.zeros(self.L.orc_y_pred_size(self.h), dtype=np.float32)
        self.L.orc_get_y_pred(self.h, _p(out))
        return out

    def set_y_pred(self, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        assert a.size == self.L.orc_y_pred_size(self.h)
        self.L.orc_set_y_pred(self.h, _p(a))

    def gh(self):
        out = np.zeros((self.num_class * self.n, 2), dtype=np.float32)
        self.L.orc_get_gh(self.h, _p(out))
        return out

    def set_gh(self, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        assert a.size == self.num_class * self.n * 2
        self.L.orc_set_gh(self.h, _p(a))

    def nid(self):
        out = np.zeros(self.n, dtype=np.int32)
        self.L.orc_get_nid(self.h, _p(out))
        return out

    def set_nid(self, a):
        a = np.ascontiguousarray(a, dtype=np.int32)
        assert a.size == self.n
        self.L.orc_set_nid(self.h, _p(a))

    def nodes(self):
        out = np.zeros(self.n_nodes, dtype=NODE_DTYPE)
        self.L.orc_get_nodes(self.h, _p(out))
        return out

    def set_nodes(self, a):
        a = np.ascontiguousarray(a, dtype=NODE_DTYPE)
        assert a.size == self.n_nodes
        self.L.orc_set_nodes(self.h, _p(a))

    def splits(self):
        out = np.zeros(1 << self.depth, dtype=SPLIT_DTYPE)
        m = self.L.orc_get_splits(self.h, _p(out))
        return out[:m]

    def level_hist(self, node_in_level):
        out = np.zeros((self.n_bins, 2), dtype=np.float32)
        out64 = np.zeros((self.n_bins, 2), dtype=np.float64)
        self.L.orc_get_level_hist(self.h, node_in_level, _p(out), _p(out64))
        return out, out64

    def tree_scores(self):
        out = np.zeros((self.n_nodes, self.n_bins), dtype=np.float32)
        self.L.orc_get_tree_scores(self.h, _p(out))
        return out

    def set_probes(self, probe):
        """One candidate (global bin index, -1 = none) per node whose signed gain the next build_tree records next
        to the node's best: what tree_scores / tree_dir_gaps give for all candidates, in O(nodes) memory."""
        if probe is None:
            self.L.orc_set_probes(self.h, None)
            return
        probe = np.ascontiguousarray(probe, dtype=np.int32)
        assert len(probe) == self.n_nodes
        self.L.orc_set_probes(self.h, _p(probe))
        self._probe = probe

    def probes(self):
        out = np.zeros(self.n_nodes, dtype=PROBE_DTYPE)
        self.L.orc_get_probes(self.h, _p(out))
        return self._probe, out

    def tree_dir_gaps(self):
        """gain(missing -> left) - gain(missing -> right) of every candidate of every node of the current tree."""
        out = np.zeros((self.n_nodes, self.n_bins), dtype=np.float32)
        self.L.orc_get_tree_dir_gaps(self.h, _p(out))
        return out

    def tree_hists(self):
        out = np.zeros((self.n_nodes, self.n_bins, 2), dtype=np.float32)
        out64 = np.zeros((self.n_nodes, self.n_bins, 2), dtype=np.float64)
        built = np.zeros(self.n_nodes, dtype=np.int32)
        self.L.orc_get_tree_hists(self.h, _p(out), _p(out64), _p(built))
        return out, out64, built

    def model(self):
        m = self.L.orc_model_size(self.h)
        out = np.zeros((m, self.tree_per_rounds, self.n_nodes), dtype=NODE_DTYPE)
        if m:
            self.L.orc_get_model(self.h, _p(out))
        return out

    def metric_log(self):
        out = np.zeros(self.L.orc_model_size(self.h), dtype=np.float32)
        self.L.orc_get_metric_log(self.h, _p(out))
        return out

    def rows_built(self):
        return self.L.orc_rows_built(self.h)


def cut_points(val, col, F, max_bin):
    L = lib()
    val = np.ascontiguousarray(val, dtype=np.float32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    cap = max(len(val), 1)
    cv = np.zeros(cap, dtype=np.float32)
    crp = np.zeros(F + 1, dtype=np.int32)
    cf = np.zeros(cap, dtype=np.int32)
    nb = L.orc_cut_points(F, len(val), _p(val), _p(col), max_bin, _p(cv), _p(crp), _p(cf))
    return cv[:nb].copy(), crp, cf[:nb].copy()


def bin_ids(val, col, cut_val, cut_row_ptr):
    L = lib()
    val = np.ascontiguousarray(val, dtype=np.float32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    cut_val = np.ascontiguousarray(cut_val, dtype=np.float32)
    cut_row_ptr = np.ascontiguousarray(cut_row_ptr, dtype=np.int32)
    out = np.zeros(len(val), dtype=np.int32)
    L.orc_bin_ids(len(val), _p(val), _p(col), _p(cut_val), _p(cut_row_ptr), _p(out))
    return out


def gradient(objective, y, yp, num_class=1):
    L = lib()
    y = np.ascontiguousarray(y, dtype=np.float32)
    yp = np.ascontiguousarray(yp, dtype=np.float32)
    n = len(y)
    out = np.zeros((yp.size, 2), dtype=np.float32)
    L.orc_gradient(objective.encode(), n, num_class, _p(y), _p(yp), _p(out))
    return out


def bagging_draws(seed, N, count=None):
    """The indices RowSampler::do_bagging draws for entries 0..count-1 of an N-entry gradient array."""
    L = lib()
    count = N if count is None else count
    out = np.zeros(count, dtype=np.int32)
    L.orc_bagging_draws(int(seed), int(N), int(count), _p(out))
    return out


def rank_gradient(objective, y, score, groups, seed):
    """One LambdaRank pass: (gh [n, 2], order [n] = row at every position of the (label, score) order of its
    group, pair [n] = partner position of every drawing position or -1)."""
    L = lib()
    y = np.ascontiguousarray(y, dtype=np.float32)
    score = np.ascontiguousarray(score, dtype=np.float32)
    grp = np.ascontiguousarray(groups, dtype=np.int32)
    n = len(y)
    gh = np.zeros((n, 2), dtype=np.float32)
    order = np.zeros(n, dtype=np.int32)
    pair = np.zeros(n, dtype=np.int32)
    L.orc_rank_gradient(int(objective == "rank:ndcg"), n, _p(y), _p(score), _p(grp), len(grp), int(seed), _p(gh),
                        _p(order), _p(pair))
    return gh, order, pair


def rank_metric(objective, y, score, groups):
    L = lib()
    y = np.ascontiguousarray(y, dtype=np.float32)
    score = np.ascontiguousarray(score, dtype=np.float32)
    grp = np.ascontiguousarray(groups, dtype=np.int32)
    return L.orc_rank_metric(int(objective == "rank:ndcg"), len(y), _p(y), _p(score), _p(grp), len(grp))


def metric_score(objective, y, yp, num_class=1):
    L = lib()
    y = np.ascontiguousarray(y, dtype=np.float32)
    yp = np.ascontiguousarray(yp, dtype=np.float32)
    return L.orc_metric_score(objective.encode(), len(y), num_class, _p(y), _p(yp))


def prune_nodes(nodes, gamma):
    L = lib()
    nodes = np.ascontiguousarray(nodes, dtype=NODE_DTYPE).copy()
    npr = L.orc_prune_nodes(_p(nodes), len(nodes), gamma)
    return nodes, npr


def group_label(y):
    L = lib()
    y = np.ascontiguousarray(y, dtype=np.float32).copy()
    lab = np.zeros(len(y), dtype=np.float32)
    nl = C.c_int(0)
    L.orc_group_label(len(y), _p(y), _p(lab), C.byref(nl))
    return y, lab[: nl.value].copy()


def predict_raw(val, row_ptr, col, F, model, lr, base_score):
    """model: NODE_DTYPE array [n_iter, n_class_trees, n_nodes]; returns class-major raw scores."""
    L = lib()
    val = np.ascontiguousarray(val, dtype=np.float32)
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    model = np.ascontiguousarray(model, dtype=NODE_DTYPE)
    n = len(row_ptr) - 1
    n_iter, nct, n_nodes = model.shape
    out = np.zeros(nct * n, dtype=np.float32)
    L.orc_predict_raw(n, F, _p(val), _p(row_ptr), _p(col), _p(model), n_iter, nct, n_nodes, lr, base_score, _p(out))
    return out


def predict_transform(objective, y, n, num_class, label):
    L = lib()
    y = np.ascontiguousarray(y, dtype=np.float32).copy()
    label = np.ascontiguousarray(label, dtype=np.float32)
    m = L.orc_predict_transform(objective.encode(), n, num_class, _p(label), _p(y))
    return y[:m]
