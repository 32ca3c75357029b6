"""The entry point that allocates nothing (tgbm_predict_raw_noalloc) against tgbm_predict_raw, through the C ABI:
same scores bit for bit on two calls in a row, the second with a smaller input (the device array keeps the first
call's contents), and a clear rejection beyond the limits."""
import ctypes as C
import os

import numpy as np
import pytest

import datasets as D

pytestmark = pytest.mark.gpu


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _rows(n, F, seed, frac_missing=0.3):
    rng = np.random.default_rng(seed)
    X = np.round(rng.standard_normal((n, F)) * 2, 2).astype(np.float32)
    X[X == 0] = 0.5
    X[rng.random((n, F)) < frac_missing] = 0
    return X


@pytest.mark.parametrize("objective,K", [("binary:logistic", 1), ("multi:softmax", 4)])
def test_no_alloc_predict_equals_predict_raw(objective, K):
    os.environ.pop("TGBM_LAYOUT", None)
    import thundergbm_amd as T
    L = T.load()
    n, F = 6000, 23
    X = _rows(n, F, 5)
    rng = np.random.default_rng(6)
    score = X[:, 0] - 0.7 * X[:, 4] + 0.2 * rng.standard_normal(n)
    y = (score > 0).astype(np.float32) if K == 1 else np.digitize(score, np.quantile(score, [0.25, 0.5, 0.75])).astype(np.float32)
    val, rp, col = D.dense_to_csr(X)
    s = T.Session(val, rp, col, y, depth=5, n_trees=7, learning_rate=0.3, objective=objective, max_num_bin=64)
    s.boost(7)
    model = C.c_void_p(s.export_model())
    base = s.base_score if K == 1 else 0.0
    s.close()
    # two calls in a row on unseen rows: 5000 rows, then 1200 other rows
    for m, seed in ((5000, 11), (1200, 12)):
        Xt = _rows(m, F, seed, 0.4)
        tv, trp, tc = D.dense_to_csr(Xt)
        ref = np.full(m * K, -7.0, np.float32)
        got = np.full(m * K, 9.0, np.float32)
        L.tgbm_predict_raw(m, _p(tv), _p(trp), _p(tc), model, 7, K, 0.3, base, _p(ref))
        rc = L.tgbm_predict_raw_noalloc(m, _p(tv), _p(trp), _p(tc), model, 7, K, 0.3, base, _p(got))
        assert rc == 0
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), "scores differ at %d rows" % m
        assert np.unique(got).size > 10  # real scores, not a constant
    # beyond the limits: a clear rejection, nothing written
    big = 70000
    tv = np.ones(big, np.float32)
    trp = np.arange(big + 1, dtype=np.int32)
    tc = np.zeros(big, np.int32)
    out = np.full(big * K, 3.0, np.float32)
    assert L.tgbm_predict_raw_noalloc(big, _p(tv), _p(trp), _p(tc), model, 7, K, 0.3, base, _p(out)) == 1
    assert np.all(out == 3.0)
    L.model_free(C.byref(model))
