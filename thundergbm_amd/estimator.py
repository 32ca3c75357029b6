"""scikit-learn style estimators over the C ABI, with the constructor arguments, method names and
data handling of the reference wrapper (python/thundergbm/thundergbm.py): dense inputs lose their
exact zeros on the way to CSR (zeros are missing values), values go in as float32 with ascending
column indices, classifier predictions come back as the original labels."""
import ctypes as C

import numpy as np
import scipy.sparse as sp
from sklearn.base import BaseEstimator, ClassifierMixin, RegressorMixin

from . import _lib

_PARAMS = ("depth", "n_trees", "n_gpus", "min_child_weight", "lambda_tgbm", "gamma", "max_num_bin", "verbose",
           "column_sampling_rate", "bagging", "n_parallel_trees", "learning_rate", "objective", "num_class",
           "tree_method")


def _csr(X):
    """CSR view of X with float32 values and ascending column indices; the caller's matrix is only copied
    when it has to be changed."""
    if not sp.issparse(X):
        X = sp.csr_matrix(np.asarray(X))
    elif X.format != "csr":
        X = X.tocsr()
    if X.data.dtype != np.float32 or not X.data.flags.c_contiguous:
        X = sp.csr_matrix((np.ascontiguousarray(X.data, dtype=np.float32), X.indices, X.indptr), shape=X.shape)
    if not X.has_sorted_indices:
        X = X.copy()
        X.sort_indices()
    return X


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def _stored_label_count(model_path):
    """Number of labels a model file stores (read from its header, nothing else is parsed)."""
    import struct
    with open(model_path, "rb") as f:
        (olen,) = struct.unpack("<i", f.read(4))
        if olen < 0 or olen >= 4096:
            raise ValueError("model file %s: bad objective length" % model_path)
        f.seek(olen + 16, 1)
        raw = f.read(4)
        if len(raw) != 4:
            raise ValueError("model file %s is truncated" % model_path)
        (n_label,) = struct.unpack("<i", raw)
    if n_label < 0:
        raise ValueError("model file %s: bad label count" % model_path)
    return n_label


class TGBMModel(BaseEstimator):
    def __init__(self, depth=6, n_trees=40, n_gpus=1, min_child_weight=1.0, lambda_tgbm=1.0, gamma=1.0,
                 max_num_bin=255, verbose=1, column_sampling_rate=1.0, bagging=0, n_parallel_trees=1,
                 learning_rate=1.0, objective="reg:linear", num_class=1, tree_method="auto"):
        for name in _PARAMS:
            setattr(self, name, locals()[name])
        self.model = None
        self.tree_per_iter = -1
        self.group_label = None

    def __del__(self):
        self._release()

    def _release(self):
        if getattr(self, "model", None) is not None:
            _lib.load().model_free(C.byref(self.model))
            self.model = None

    def fit(self, X, y, groups=None):
        lib = _lib.load()
        self._release()
        X = _csr(X)
        y = np.ascontiguousarray(y, dtype=np.float32)
        if X.shape[0] != len(y):
            raise ValueError("X and y have different numbers of rows")
        indptr = np.ascontiguousarray(X.indptr, dtype=np.int32)
        indices = np.ascontiguousarray(X.indices, dtype=np.int32)
        n_labels = len(np.unique(y))
        group_label = (C.c_float * max(n_labels, 1))()
        n_class = (C.c_int * 1)(self.num_class)
        per_iter = (C.c_int * 1)(0)
        self.model = C.c_void_p(None)
        grp = None if groups is None else np.ascontiguousarray(groups, dtype=np.int32)
        lib.sparse_train_scikit(X.shape[0], _ptr(X.data), _ptr(indptr), _ptr(indices), _ptr(y), self.depth,
                                self.n_trees, self.n_gpus, self.min_child_weight, self.lambda_tgbm, self.gamma,
                                self.max_num_bin, self.verbose, self.column_sampling_rate, int(self.bagging),
                                self.n_parallel_trees, self.learning_rate, self.objective.encode("utf-8"),
                                C.cast(n_class, C.c_void_p), self.tree_method.encode("utf-8"),
                                C.cast(C.byref(self.model), C.c_void_p), C.cast(per_iter, C.c_void_p),
                                C.cast(group_label, C.c_void_p), None if grp is None else _ptr(grp),
                                0 if grp is None else len(grp))
        self.num_class = n_class[0]
        self.tree_per_iter = per_iter[0]
        self.group_label = [group_label[i] for i in range(n_labels)]
        if not self.model:
            raise RuntimeError("The model returned is empty!")
        return self

    def predict(self, X, groups=None):
        if not self.model:
            raise ValueError("Please train the model first or load model from file!")
        lib = _lib.load()
        X = _csr(X)
        indptr = np.ascontiguousarray(X.indptr, dtype=np.int32)
        indices = np.ascontiguousarray(X.indices, dtype=np.int32)
        n = X.shape[0]
        n_out = n * self.num_class if self.objective == "multi:softprob" else n
        out = np.zeros(max(n_out, n * max(self.tree_per_iter, 1)), dtype=np.float32)
        labels = np.asarray(self.group_label if self.group_label else [0.0], dtype=np.float32)
        grp = None if groups is None else np.ascontiguousarray(groups, dtype=np.int32)
        lib.sparse_predict_scikit(n, _ptr(X.data), _ptr(indptr), _ptr(indices), _ptr(out),
                                  C.cast(C.byref(self.model), C.c_void_p), self.n_trees, self.tree_per_iter,
                                  self.objective.encode("utf-8"), self.num_class, self.learning_rate, _ptr(labels),
                                  None if grp is None else _ptr(grp), 0 if grp is None else len(grp), self.verbose)
        if self.objective == "multi:softprob":
            # the library returns class-major probabilities; the reference wrapper reshapes them as
            # [-1, num_class] without transposing (thundergbm.py:169-171) and so does this one
            self.predict_label = out[:n_out].reshape([-1, self.num_class])
        else:
            self.predict_label = out[:n].copy()
        return self.predict_label

    def predict_proba_class_major(self, X):
        """multi:softprob probabilities as [num_class, n_rows] (the layout the library produces)."""
        p = self.predict(X)
        return p.reshape(self.num_class, -1)

    def save_model(self, model_path):
        if not self.model:
            raise ValueError("Please train the model first or load model from file!")
        labels = np.asarray(self.group_label if self.group_label else [0.0], dtype=np.float32)
        _lib.load().save(model_path.encode("utf-8"), self.objective.encode("utf-8"), self.learning_rate,
                         self.num_class, self.n_trees, self.tree_per_iter, C.cast(C.byref(self.model), C.c_void_p),
                         _ptr(labels))

    def load_model(self, model_path):
        lib = _lib.load()
        self._release()
        self.model = C.c_void_p(None)
        lr = (C.c_float * 1)()
        n_class = (C.c_int * 1)()
        n_trees = (C.c_int * 1)()
        per_iter = (C.c_int * 1)()
        lib.load_model(model_path.encode("utf-8"), C.cast(lr, C.c_void_p), C.cast(n_class, C.c_void_p),
                       C.cast(n_trees, C.c_void_p), C.cast(per_iter, C.c_void_p),
                       C.cast(C.byref(self.model), C.c_void_p))
        if not self.model:
            raise ValueError("Model is None.")
        self.learning_rate = lr[0]
        self.num_class = n_class[0]
        self.n_trees = n_trees[0]
        self.tree_per_iter = per_iter[0]
        # load_config copies every label the file stores (scikit_tgbm.cpp:173-182) and has no capacity argument:
        # files written by the CLI for reg:* / rank:* objectives hold one label per training row, so the buffer is
        # sized from the file's own label count (header: i32 objective length, objective, f32 learning rate,
        # i32 num_class, i32 n_trees, f32 base_score, i32 label count; parser.cpp:146-157)
        n_stored = _stored_label_count(model_path)
        labels = (C.c_float * max(n_stored, self.num_class, 1))()
        lib.load_config(model_path.encode("utf-8"), C.cast(labels, C.c_void_p))
        self.group_label = [labels[i] for i in range(self.num_class)]

    def get_trees(self):
        """Every tree as parallel heap-ordered arrays (the dictionaries the reference hands to shap)."""
        if not self.model:
            raise ValueError("Please train the model first or load model from file!")
        lib = _lib.load()
        total = self.n_trees * self.tree_per_iter
        n_nodes = np.zeros(total, dtype=np.int32)
        mp = C.cast(C.byref(self.model), C.c_void_p)
        lib.get_n_nodes(mp, _ptr(n_nodes), self.n_trees, self.tree_per_iter)
        trees = []
        for t in range(total):
            nn = int(n_nodes[t])
            d = {"children_left": np.empty(nn, np.int32), "children_right": np.empty(nn, np.int32),
                 "children_default": np.empty(nn, np.int32), "feature": np.empty(nn, np.int32),
                 "threshold": np.empty(nn, np.float32), "value": np.empty(nn, np.float32),
                 "node_sample_weight": np.empty(nn, np.float32)}
            lib.get_a_tree(mp, t, nn, _ptr(d["children_left"]), _ptr(d["children_right"]),
                           _ptr(d["children_default"]), _ptr(d["feature"]), _ptr(d["threshold"]), _ptr(d["value"]),
                           _ptr(d["node_sample_weight"]))
            d["value"] = d["value"].reshape(-1, 1)
            trees.append(d)
        return trees

    def get_shap_trees(self):
        """The trees as shap.explainers.tree.Tree objects (python/thundergbm/thundergbm.py:284-348); like
        the reference only for models with one tree per iteration, and only when shap is installed."""
        if self.objective != "binary:logistic" and self.tree_per_iter != 1:
            raise RuntimeError("not supported yet!")
        import shap.explainers.tree as shap_tree
        return [shap_tree.Tree(t) for t in self.get_trees()[:: max(self.tree_per_iter, 1)]]

    def cv(self, X, y, folds=None, nfold=5, shuffle=True, seed=0):
        """k-fold cross-validation with the reference's fold construction and result keys
        (python/thundergbm/thundergbm.py:223-282): fold size int(n / nfold), folds cut from a seeded
        permutation, accuracy for classifiers and mean squared error (reported under the RMSE keys, as
        there) for regressors."""
        import statistics

        X = _csr(X)
        y = np.ascontiguousarray(y, dtype=np.float32)
        n = X.shape[0]
        if folds is not None:
            train_ids = [f[0] for f in folds]
            test_ids = [f[1] for f in folds]
            nfold = len(folds)
        else:
            order = np.random.RandomState(seed).permutation(n) if shuffle else np.arange(n)
            step = int(n / nfold)
            test_ids = [order[i:i + step] for i in range(0, n, step)]
            train_ids = [np.concatenate([test_ids[i] for i in range(nfold) if i != k]) for k in range(nfold)]
        classifier = getattr(self, "_impl", "") == "classifier"
        train_scores, test_scores = [], []
        for k in range(nfold):
            self.fit(X[train_ids[k], :], y[train_ids[k]])
            for ids, scores in ((train_ids[k], train_scores), (test_ids[k], test_scores)):
                pred = self.predict(X[ids, :])
                if classifier:
                    scores.append(float(np.mean(pred == y[ids])))
                else:
                    scores.append(float(np.mean((pred - y[ids]) ** 2)))
        name = "accuracy" if classifier else "RMSE"
        self.eval_res = {
            "train-%s-mean" % name: statistics.mean(train_scores), "train-%s-std" % name: statistics.stdev(train_scores),
            "test-%s-mean" % name: statistics.mean(test_scores), "test-%s-std" % name: statistics.stdev(test_scores)}
        return self.eval_res


class TGBMClassifier(TGBMModel, ClassifierMixin):
    _impl = "classifier"

    def __init__(self, depth=6, n_trees=40, n_gpus=1, min_child_weight=1.0, lambda_tgbm=1.0, gamma=1.0,
                 max_num_bin=255, verbose=1, column_sampling_rate=1.0, bagging=0, n_parallel_trees=1,
                 learning_rate=1.0, objective="multi:softmax", num_class=2, tree_method="auto"):
        super().__init__(depth, n_trees, n_gpus, min_child_weight, lambda_tgbm, gamma, max_num_bin, verbose,
                         column_sampling_rate, bagging, n_parallel_trees, learning_rate, objective, num_class,
                         tree_method)


class TGBMRegressor(TGBMModel, RegressorMixin):
    _impl = "regressor"

    def __init__(self, depth=6, n_trees=40, n_gpus=1, min_child_weight=1.0, lambda_tgbm=1.0, gamma=1.0,
                 max_num_bin=255, verbose=1, column_sampling_rate=1.0, bagging=0, n_parallel_trees=1,
                 learning_rate=1.0, objective="reg:linear", num_class=1, tree_method="auto"):
        super().__init__(depth, n_trees, n_gpus, min_child_weight, lambda_tgbm, gamma, max_num_bin, verbose,
                         column_sampling_rate, bagging, n_parallel_trees, learning_rate, objective, num_class,
                         tree_method)
