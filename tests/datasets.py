"""Seeded synthetic inputs shared by the CPU and GPU tests and by bench.py (small versions of the
benchmark configurations) plus a LIBSVM reader for the golden fixture."""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
A1A = os.path.join(HERE, "golden", "a1a_test_dataset.txt")


def read_libsvm(path):
    """1-based `label idx:val ...` lines -> (val, row_ptr, col, y) with 0-based columns."""
    vals, cols, row_ptr, ys = [], [], [0], []
    with open(path) as f:
        for line in f:
            parts = line.split()
            if not parts:
                continue
            ys.append(float(parts[0]))
            for tok in parts[1:]:
                i, v = tok.split(":")
                cols.append(int(i) - 1)
                vals.append(float(v))
            row_ptr.append(len(vals))
    return (np.asarray(vals, np.float32), np.asarray(row_ptr, np.int32), np.asarray(cols, np.int32),
            np.asarray(ys, np.float32))


def dense_to_csr(X):
    """Dense -> CSR with the reference wrapper's rule: exact zeros are dropped (they become missing)."""
    X = np.asarray(X, dtype=np.float32)
    n, F = X.shape
    if np.count_nonzero(X) == X.size:  # nothing to drop: skip the index gymnastics on big matrices
        row_ptr = (np.arange(n + 1, dtype=np.int64) * F).astype(np.int32)
        col = np.tile(np.arange(F, dtype=np.int32), n)
        return np.ascontiguousarray(X).reshape(-1), row_ptr, col
    mask = X != 0
    row_ptr = np.zeros(X.shape[0] + 1, dtype=np.int32)
    np.cumsum(mask.sum(axis=1), out=row_ptr[1:])
    col = np.nonzero(mask)[1].astype(np.int32)
    val = X[mask].astype(np.float32)
    return val, row_ptr, col


def config1(n=10000, F=8, seed=0):
    """Regression: X ~ U[0,1], y = Xw + 0.5 sin(6 x0) + N(0,0.1)."""
    rng = np.random.default_rng(seed)
    X = rng.random((n, F), dtype=np.float32)
    w = rng.standard_normal(F).astype(np.float32)
    y = X @ w + 0.5 * np.sin(6 * X[:, 0]) + 0.1 * rng.standard_normal(n).astype(np.float32)
    return X, y.astype(np.float32)


def config2(n=10_000_000, seed=1):
    """Binary: 21 N(0,1) columns + 7 derived (products / abs of pairs); Bernoulli(sigmoid(logit))."""
    rng = np.random.default_rng(seed)
    X = np.empty((n, 28), dtype=np.float32)
    X[:, :21] = rng.standard_normal((n, 21), dtype=np.float32)
    for j in range(7):
        a, b = X[:, 2 * j], X[:, 2 * j + 1]
        X[:, 21 + j] = a * b if j % 2 == 0 else np.abs(a - b)
    w = np.zeros(28, dtype=np.float32)
    idx = rng.choice(28, size=10, replace=False)
    w[idx] = rng.standard_normal(10).astype(np.float32)
    logit = X @ w
    for j in range(4):
        logit += 0.3 * X[:, j] * X[:, j + 5]
    logit += 0.15
    p = 1.0 / (1.0 + np.exp(-logit))
    y = (rng.random(n, dtype=np.float32) < p).astype(np.float32)
    return X, y


def config3(n=500_000, F=2000, seed=2):
    """Wide regression: N(0,1), 5% of columns Student-t(df=2); 50 informative columns."""
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((n, F), dtype=np.float32)
    heavy = rng.choice(F, size=max(1, F // 20), replace=False)
    for c in heavy:
        X[:, c] = rng.standard_t(2, size=n).astype(np.float32)
    inf = rng.choice(F, size=min(50, F), replace=False)
    w = rng.standard_normal(len(inf)).astype(np.float32)
    y = X[:, inf] @ w + rng.standard_normal(n).astype(np.float32)
    return X, y.astype(np.float32)


def config4(n=2_000_000, F=100_000, nnz_per_row=40, seed=3):
    """Sparse CSR binary: Zipf(1.1) feature ids, lognormal values, sparse logistic labels."""
    rng = np.random.default_rng(seed)
    raw = rng.zipf(1.1, size=(n, nnz_per_row)) - 1
    raw = np.where(raw >= F, rng.integers(0, F, size=raw.shape), raw).astype(np.int64)
    raw.sort(axis=1)
    keep = np.ones_like(raw, dtype=bool)
    keep[:, 1:] = raw[:, 1:] != raw[:, :-1]
    row_ptr = np.zeros(n + 1, dtype=np.int32)
    np.cumsum(keep.sum(axis=1), out=row_ptr[1:])
    col = raw[keep].astype(np.int32)
    val = rng.lognormal(0.0, 1.0, size=len(col)).astype(np.float32)
    wf = rng.choice(F, size=min(500, F), replace=False)
    w = np.zeros(F, dtype=np.float32)
    w[wf] = rng.standard_normal(len(wf)).astype(np.float32)
    w[:20] = rng.standard_normal(20).astype(np.float32)
    contrib = w[col] * np.log1p(val)
    logit = np.add.reduceat(contrib, row_ptr[:-1].astype(np.int64))
    logit[np.diff(row_ptr) == 0] = 0
    logit = logit - np.median(logit)
    p = 1.0 / (1.0 + np.exp(-logit))
    y = (rng.random(n) < p).astype(np.float32)
    return val, row_ptr, col, y


def config5(n=1_000_000, seed=4):
    """8-class softmax: 10 quantised-int columns in [0,3000), one-hot groups of 4 and 40."""
    rng = np.random.default_rng(seed)
    X = np.zeros((n, 54), dtype=np.float32)
    X[:, :10] = np.floor(rng.random((n, 10)) * 3000).astype(np.float32)
    g1 = rng.integers(0, 4, size=n)
    g2 = rng.integers(0, 40, size=n)
    X[np.arange(n), 10 + g1] = 1
    X[np.arange(n), 14 + g2] = 1
    W = rng.standard_normal((54, 8)).astype(np.float32)
    Z = (X / np.maximum(X.max(axis=0), 1)) @ W
    bias = np.log(np.array([0.40, 0.25, 0.15, 0.08, 0.05, 0.03, 0.02, 0.02]))
    Z = Z + bias + rng.gumbel(size=Z.shape)
    y = Z.argmax(axis=1).astype(np.float32)
    return X, y


def warm_up(T):
    """One tiny training session: the first GPU call of a process initialises the runtime (which may draw from
    rand() itself), so the tests' random streams do not depend on which of them runs first."""
    X, y = config1(64, 3, seed=0)
    val, rp, col = dense_to_csr(X)
    s = T.Session(val, rp, col, y, depth=2, n_trees=1, max_num_bin=8)
    s.boost(1)
    s.close()
