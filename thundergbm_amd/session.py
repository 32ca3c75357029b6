"""Python view of the session API (tgbm_trainer_*) used by the benchmark and the parity tests."""
import ctypes as C

import numpy as np

from . import _lib

NODE_DTYPE = np.dtype(
    [
        ("final_id", "<i4"), ("lch", "<i4"), ("rch", "<i4"), ("parent", "<i4"),
        ("gain", "<f4"), ("base_weight", "<f4"), ("split_fid", "<i4"), ("split_value", "<f4"),
        ("split_bid", "u1"), ("default_right", "u1"), ("is_leaf", "u1"), ("is_valid", "u1"),
        ("is_pruned", "u1"), ("pad", "u1", (3,)), ("sum_g", "<f4"), ("sum_h", "<f4"),
    ]
)
SPLIT_DTYPE = np.dtype(
    [
        ("gain", "<f4"), ("miss_g", "<f4"), ("miss_h", "<f4"), ("lch_g", "<f4"), ("lch_h", "<f4"),
        ("default_right", "<i4"), ("nid", "<i4"), ("fid", "<i4"), ("fval", "<f4"), ("bid", "<i4"),
        ("best_index", "<i4"), ("pad", "<i4"),
    ]
)
QUANT_DTYPE = np.dtype([("scale_g", "<f4"), ("scale_h", "<f4"), ("inv_g", "<f4"), ("inv_h", "<f4"),
                        ("gq_max", "<f4"), ("hq_max", "<f4"), ("h_bits", "<i4"), ("h_integer", "<i4"),
                        ("flush_rows", "<i4")])
CTL_DTYPE = np.dtype([("hchunk", "<i4"), ("n_hitems", "<i4"), ("n_pitems", "<i4"), ("rows_built", "<i4")])


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class Session:
    """One training session on the GPU: CSR input is copied to HBM once, then boosted in place."""

    def __init__(self, val, row_ptr, col, y, depth=6, n_trees=40, min_child_weight=1.0, lambda_=1.0, gamma=1.0,
                 max_num_bin=255, learning_rate=1.0, objective="reg:linear", num_class=1, verbose=0, groups=None):
        self.L = _lib.load()
        val = np.ascontiguousarray(val, dtype=np.float32)
        row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
        col = np.ascontiguousarray(col, dtype=np.int32)
        y = np.ascontiguousarray(y, dtype=np.float32)
        self.n = len(row_ptr) - 1
        self.nnz = int(row_ptr[-1])
        self.depth = depth
        # groups: sizes of the query groups (consecutive rows) of the ranking objectives
        grp = np.ascontiguousarray(groups if groups is not None else [], dtype=np.int32)
        self.h = self.L.tgbm_trainer_create_grouped(self.n, _p(val), _p(row_ptr), _p(col), _p(y), depth, n_trees,
                                                    min_child_weight, lambda_, gamma, max_num_bin, learning_rate,
                                                    objective.encode(), num_class, verbose,
                                                    _p(grp) if len(grp) else None, len(grp))
        self.F = self.info("n_features")
        self.n_bins = self.info("n_bins")
        self.num_class = self.info("num_class")
        self.tree_per_rounds = self.info("tree_per_rounds")
        self.n_nodes = self.info("n_nodes")

    def close(self):
        if getattr(self, "h", None):
            self.L.tgbm_trainer_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def info(self, key):
        return self.L.tgbm_trainer_info(self.h, key.encode())

    @property
    def base_score(self):
        return self.L.tgbm_trainer_base_score(self.h)

    def set_option(self, key, value):
        self.L.tgbm_trainer_set_option(self.h, key.encode(), float(value))

    def sample_columns(self):
        self.L.tgbm_trainer_sample_columns(self.h)

    def boost(self, rounds=1):
        self.L.tgbm_trainer_boost(self.h, rounds)

    def gradient(self):
        self.L.tgbm_trainer_gradient(self.h)

    def tree_init(self, k=0):
        self.L.tgbm_trainer_tree_init(self.h, k)

    def find_split(self, level):
        self.L.tgbm_trainer_find_split(self.h, level)

    def partition(self, level):
        self.L.tgbm_trainer_partition(self.h, level)

    def finish_tree(self, k=0):
        self.L.tgbm_trainer_finish_tree(self.h, k)

    def metric(self):
        return self.L.tgbm_trainer_metric(self.h)

    def get(self, name, dtype, shape=None):
        nbytes = self.L.tgbm_trainer_get(self.h, name.encode(), None, 0)
        out = np.zeros(nbytes // np.dtype(dtype).itemsize, dtype=dtype)
        if nbytes:
            self.L.tgbm_trainer_get(self.h, name.encode(), _p(out), nbytes)
        return out.reshape(shape) if shape is not None else out

    def set(self, name, arr):
        arr = np.ascontiguousarray(arr)
        self.L.tgbm_trainer_set(self.h, name.encode(), _p(arr), arr.nbytes)

    # typed views
    def cuts(self):
        return self.get("cut_val", np.float32), self.get("cut_row_ptr", np.int32), self.get("cut_fid", np.int32)

    def binmat(self):
        """Local bin of every (block, row, feature in block), 255 / 65535 where a row stores no value of the feature.
        Features that share a column of the device matrix (runs of features that never meet in a row) are taken
        apart here, so the result does not depend on that."""
        W, nb = self.info("dense_W"), self.info("dense_blocks")
        m = self.get("binmat", np.uint16 if self.info("dense_bin_bytes") == 2 else np.uint8, (nb, self.n, W))
        F, P = self.F, self.info("dense_cols")
        if P == F:
            return m
        cols = m.transpose(1, 0, 2).reshape(self.n, nb * W).astype(np.int32)
        fc, lo = self.get("feat_col", np.int32), self.get("feat_lo", np.uint8).astype(np.int32)
        _, crp, _ = self.cuts()
        t = cols[:, fc] - lo[None, :]
        logical = np.where((t >= 0) & (t < np.diff(crp)[None, :]), t, 255).astype(np.uint8)
        nbl = (F + W - 1) // W
        out = np.full((self.n, nbl * W), 255, np.uint8)
        out[:, :F] = logical
        return np.ascontiguousarray(out.reshape(self.n, nbl, W).transpose(1, 0, 2))

    def global_bin_ids(self, row_ptr, col):
        """Global bin id of every stored value (the reference's csr_bin_id) and its local bin id."""
        if self.info("sparse"):
            gb = self.get("csr_bin", np.int32)
            _, crp, _ = self.cuts()
            return gb, gb - crp[col]
        W = self.info("dense_W")
        m = self.binmat()
        _, crp, _ = self.cuts()
        rows = np.repeat(np.arange(self.n), np.diff(row_ptr))
        local = m[col // W, rows, col % W].astype(np.int32)
        return local + crp[col], local

    def nid(self):
        return self.get("nid", np.int32)

    def gh(self):
        return self.get("gh", np.float32, (-1, 2))

    def y_pred(self):
        return self.get("y_pred", np.float32)

    def y(self):
        return self.get("y", np.float32)

    def labels(self):
        return self.get("labels", np.float32)

    def nodes(self):
        return self.get("nodes", NODE_DTYPE)

    def splits(self, level):
        return self.get("sp", SPLIT_DTYPE)[: 1 << level]

    def level_hist(self, level):
        """Raw histograms of the nodes of `level`: [2^level, n_bins, 2] (exact fixed-point sums as float64)."""
        q = self.get("hist_q%d" % (level & 1), np.int64)
        q = q[: (1 << level) * self.n_bins * 2].reshape(1 << level, self.n_bins, 2)
        sc = self.quant()
        return q.astype(np.float64) * np.array([float(sc["inv_g"]), float(sc["inv_h"])])

    def quant(self):
        """Fixed-point plan of the current tree (QuantCtl)."""
        return self.get("quant", QUANT_DTYPE)[0]

    def ctl(self):
        return self.get("ctl", CTL_DTYPE)

    def model(self):
        m = self.get("model", NODE_DTYPE)
        return m.reshape(-1, self.tree_per_rounds, self.n_nodes)

    def metric_log(self):
        return self.get("metric_log", np.float32)

    def set_profiling(self, on):
        self.L.tgbm_trainer_set_profiling(self.h, int(on))

    def profile(self):
        out = np.zeros(4, dtype=np.float64)
        self.L.tgbm_trainer_get_profile(self.h, _p(out))
        return {"hist_ms": out[0], "launches": int(out[1]), "rows_built": int(out[2]), "bytes": int(out[3])}

    PHASES = ("gradient_tree_init", "hist", "merge_subtract", "split_update", "partition", "tree_end", "metric", "reorder")

    def phase_profile(self):
        """Per-stage milliseconds of the rounds boosted with profiling on, and the histogram launches split into the
        root level and the levels below it."""
        out = np.zeros(15, dtype=np.float64)
        self.L.tgbm_trainer_get_phase_profile(self.h, _p(out), 15)
        split = {}
        for i, name in enumerate(("root", "below_root")):
            ms, launches, nbytes = out[9 + 3 * i:12 + 3 * i]
            split[name] = {"ms": float(ms), "launches": int(launches), "bytes": int(nbytes)}
        return {"rounds": int(out[0]), "phase_ms": {k: float(v) for k, v in zip(self.PHASES, out[1:9])}, "hist": split}

    def export_model(self):
        return self.L.tgbm_trainer_export_model(self.h)
