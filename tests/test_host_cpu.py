"""CPU-side checks of the shipped library: the C ABI surface, the model file format and the CLI
argument handling. No kernel is launched here."""
import ctypes as C
import os
import re
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "thundergbm.h")
LIB = os.path.join(ROOT, "thundergbm_amd", "libthundergbm.so")
TRAIN = os.path.join(ROOT, "thundergbm_amd", "bin", "thundergbm-train")

NODE = np.dtype([("final_id", "<i4"), ("lch", "<i4"), ("rch", "<i4"), ("parent", "<i4"), ("gain", "<f4"),
                 ("base_weight", "<f4"), ("split_fid", "<i4"), ("split_value", "<f4"), ("split_bid", "u1"),
                 ("default_right", "u1"), ("is_leaf", "u1"), ("is_valid", "u1"), ("is_pruned", "u1"),
                 ("pad", "u1", (3,)), ("sum_g", "<f4"), ("sum_h", "<f4")])


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        subprocess.check_call(["python", os.path.join(ROOT, "thundergbm_amd", "build.py")])
    import sys
    sys.path.insert(0, ROOT)
    import thundergbm_amd
    return thundergbm_amd.load()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text)) - {"defined"})


def test_header_symbols_are_exported(lib):
    names = _declared_functions()
    # the nine entry points of the reference's scikit_tgbm.cpp must all be there
    for ref in ("set_logger", "sparse_train_scikit", "sparse_predict_scikit", "save", "load_model", "load_config",
                "get_n_nodes", "get_a_tree", "model_free"):
        assert ref in names
    for ref in ("train_R", "predict_R"):  # gbm_R_interface.cpp
        assert ref in names
    for n in names:
        assert hasattr(lib, n), "declared in the header but not exported: %s" % n


def test_python_signature_table_matches_header():
    import sys
    sys.path.insert(0, ROOT)
    from thundergbm_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared_functions()


def test_tree_node_is_48_bytes():
    assert NODE.itemsize == 48
    assert NODE.fields["split_bid"][1] == 32 and NODE.fields["sum_g"][1] == 40


def _toy_model_bytes(objective=b"binary:logistic", labels=(-1.0, 1.0), n_iter=3):
    nodes = np.zeros(7, dtype=NODE)
    for i in range(7):
        nodes[i]["final_id"] = i
        nodes[i]["parent"] = -1 if i == 0 else (i - 1) // 2
        nodes[i]["is_valid"] = 1
        nodes[i]["split_fid"] = -1
        if i < 3:
            nodes[i]["lch"], nodes[i]["rch"] = 2 * i + 1, 2 * i + 2
            nodes[i]["split_fid"], nodes[i]["split_value"], nodes[i]["gain"] = i, 0.5 * i, 2.0
            nodes[i]["default_right"] = i % 2
        else:
            nodes[i]["lch"] = nodes[i]["rch"] = -1
            nodes[i]["is_leaf"] = 1
            nodes[i]["base_weight"] = 0.1 * i
        nodes[i]["sum_h"] = 10 + i
    out = struct.pack("<i", len(objective)) + objective
    out += struct.pack("<fiif", 0.25, len(labels), n_iter, 0.0)
    out += struct.pack("<i", len(labels)) + struct.pack("<%df" % len(labels), *labels)
    out += struct.pack("<i", n_iter)
    for _ in range(n_iter):
        out += struct.pack("<i", 1) + struct.pack("<Q", 7) + nodes.tobytes()
    return out, nodes


def test_model_file_round_trip(lib, tmp_path):
    """load_model / load_config / get_n_nodes / get_a_tree / save on the raw format of the reference's
    Parser (src/thundergbm/parser.cpp:102-171)."""
    data, nodes = _toy_model_bytes()
    src = tmp_path / "in.model"
    src.write_bytes(data)
    model = C.c_void_p(None)
    lr, nc, nt, per = (C.c_float * 1)(), (C.c_int * 1)(), (C.c_int * 1)(), (C.c_int * 1)()
    vp = lambda a: C.cast(a, C.c_void_p)
    lib.load_model(str(src).encode(), vp(lr), vp(nc), vp(nt), vp(per), vp(C.byref(model)))
    assert model.value and abs(lr[0] - 0.25) < 1e-7 and nc[0] == 2 and nt[0] == 3 and per[0] == 1
    labels = (C.c_float * 2)()
    lib.load_config(str(src).encode(), vp(labels))
    assert list(labels) == [-1.0, 1.0]
    nn = np.zeros(3, np.int32)
    lib.get_n_nodes(vp(C.byref(model)), nn.ctypes.data_as(C.c_void_p), 3, 1)
    assert nn.tolist() == [7, 7, 7]
    arr = {k: np.zeros(7, np.int32) for k in ("l", "r", "d", "f")}
    thr, val, w = np.zeros(7, np.float32), np.zeros(7, np.float32), np.zeros(7, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    lib.get_a_tree(vp(C.byref(model)), 1, 7, p(arr["l"]), p(arr["r"]), p(arr["d"]), p(arr["f"]), p(thr), p(val), p(w))
    assert arr["l"].tolist() == [1, 3, 5, -1, -1, -1, -1] and arr["r"].tolist() == [2, 4, 6, -1, -1, -1, -1]
    assert arr["d"].tolist() == [1, 4, 5, -1, -1, -1, -1]  # default child follows default_right
    assert arr["f"].tolist() == [0, 1, 2, -1, -1, -1, -1]
    np.testing.assert_allclose(val, [0, 0, 0, 0.3, 0.4, 0.5, 0.6], rtol=1e-6)
    np.testing.assert_allclose(w, 10 + np.arange(7))
    dst = tmp_path / "out.model"
    lab = np.array([-1.0, 1.0], np.float32)
    lib.save(str(dst).encode(), b"binary:logistic", 0.25, 2, 3, 1, vp(C.byref(model)), p(lab))
    assert dst.read_bytes() == data
    lib.model_free(vp(C.byref(model)))
    assert model.value is None
    lib.model_free(vp(C.byref(model)))  # freeing an empty slot is a no-op


def test_set_logger_and_cli_usage(lib):
    lib.set_logger(0)
    lib.set_logger(1)
    if os.path.exists(TRAIN):
        out = subprocess.run([TRAIN], capture_output=True, text=True)
        assert out.returncode == 0 and "Usage" in out.stdout


def test_estimator_parameters_follow_the_reference_defaults():
    import sys
    sys.path.insert(0, ROOT)
    import thundergbm_amd as T
    r = T.TGBMRegressor()
    c = T.TGBMClassifier()
    # python/thundergbm/thundergbm.py:355-380
    assert (r.depth, r.n_trees, r.max_num_bin, r.learning_rate, r.objective, r.tree_method) == \
        (6, 40, 255, 1.0, "reg:linear", "auto")
    assert (c.objective, c.num_class, c.gamma, c.lambda_tgbm, c.min_child_weight) == ("multi:softmax", 2, 1.0, 1.0, 1.0)
    assert set(r.get_params()) >= {"depth", "n_trees", "n_gpus", "bagging", "column_sampling_rate"}
    with pytest.raises(ValueError):
        r.predict(np.zeros((2, 2)))


def test_zero_based_libsvm_file_is_rejected_with_its_line(tmp_path):
    """LIBSVM feature ids are 1-based (dataset.cpp:243 stores fid - 1); a 0-based file (what sklearn's
    dump_svmlight_file writes by default) must stop on the host with the offending line, not index column -1."""
    if not os.path.exists(TRAIN):
        pytest.skip("CLI not built")
    data = tmp_path / "zero_based.txt"
    data.write_text("# comment line\n1 1:0.5 3:1.5\n0 2:1.0\n1 0:2.0 4:1.0\n0 1:1.0\n")
    out = subprocess.run([TRAIN, "data=%s" % data, "n_trees=1"], capture_output=True, text=True, cwd=str(tmp_path))
    assert out.returncode != 0
    assert "line 4" in out.stderr and "feature id 0" in out.stderr and "1-based" in out.stderr


_BAD_CSR = r"""
import ctypes as C, sys
import numpy as np
sys.path.insert(0, %r)
import thundergbm_amd
L = thundergbm_amd.load()
val = np.ones(4, np.float32); col = np.array([0, 1, 0, 1], np.int32); y = np.zeros(3, np.float32)
rp = np.array(%s, np.int32)
p = lambda a: a.ctypes.data_as(C.c_void_p)
L.tgbm_trainer_create_grouped(3, p(val), p(rp), p(col), p(y), 3, 1, 1.0, 1.0, 1.0, 16, 1.0, b"reg:linear", 1, 0, None, 0)
"""


@pytest.mark.parametrize("row_ptr,msg", [("[0, 2, 1, 4]", "row_ptr decreases at row 1"), ("[1, 2, 3, 4]", "row_ptr[0] is 1")])
def test_malformed_row_ptr_is_rejected_on_the_host(lib, row_ptr, msg):
    import sys
    out = subprocess.run([sys.executable, "-c", _BAD_CSR % (ROOT, row_ptr)], capture_output=True, text=True)
    assert out.returncode != 0 and msg in out.stderr, out.stderr


def test_load_model_with_one_label_per_training_row(lib, tmp_path):
    """Model files written by the CLI for reg:* objectives store every training label (dataset.cpp:290-291,
    parser.cpp:156-157); load_config copies them all, so the Python side must size its buffer from the file."""
    import sys
    sys.path.insert(0, ROOT)
    import thundergbm_amd as T
    labels = tuple(float(i % 7) for i in range(5000))
    data, _ = _toy_model_bytes(objective=b"reg:linear", labels=labels, n_iter=2)
    # num_class of a regression model is 1 whatever the label count
    olen = 4 + len(b"reg:linear")
    data = data[:olen + 4] + struct.pack("<i", 1) + data[olen + 8:]
    path = tmp_path / "cli_reg.model"
    path.write_bytes(data)
    m = T.TGBMRegressor()
    m.load_model(str(path))
    assert m.num_class == 1 and m.n_trees == 2 and m.group_label == [0.0]
    assert len(m.get_trees()) == 2
