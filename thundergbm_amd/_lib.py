"""ctypes loader of the in-tree libthundergbm.so. There is no fallback: a missing library is an error."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libthundergbm.so")

_lib = None

# name -> (restype, argtypes); exactly the declarations of include/thundergbm.h
_P = C.c_void_p
SIGNATURES = {
    "set_logger": (None, [C.c_int]),
    "sparse_train_scikit": (None, [C.c_int, _P, _P, _P, _P, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                                   C.c_float, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, C.c_float, C.c_char_p,
                                   _P, C.c_char_p, _P, _P, _P, _P, C.c_int]),
    "sparse_predict_scikit": (None, [C.c_int, _P, _P, _P, _P, _P, C.c_int, C.c_int, C.c_char_p, C.c_int, C.c_float,
                                     _P, _P, C.c_int, C.c_int]),
    "save": (None, [C.c_char_p, C.c_char_p, C.c_float, C.c_int, C.c_int, C.c_int, _P, _P]),
    "load_model": (None, [C.c_char_p, _P, _P, _P, _P, _P]),
    "load_config": (None, [C.c_char_p, _P]),
    "get_n_nodes": (None, [_P, _P, C.c_int, C.c_int]),
    "get_a_tree": (None, [_P, C.c_int, C.c_int, _P, _P, _P, _P, _P, _P, _P]),
    "model_free": (None, [_P]),
    "train_R": (None, [_P] * 18),
    "predict_R": (None, [_P] * 3),
    "tgbm_trainer_create": (_P, [C.c_int, _P, _P, _P, _P, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_int,
                                 C.c_float, C.c_char_p, C.c_int, C.c_int]),
    "tgbm_trainer_create_grouped": (_P, [C.c_int, _P, _P, _P, _P, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float,
                                         C.c_int, C.c_float, C.c_char_p, C.c_int, C.c_int, _P, C.c_int]),
    "tgbm_trainer_destroy": (None, [_P]),
    "tgbm_trainer_set_option": (None, [_P, C.c_char_p, C.c_double]),
    "tgbm_trainer_sample_columns": (None, [_P]),
    "tgbm_trainer_boost": (None, [_P, C.c_int]),
    "tgbm_trainer_gradient": (None, [_P]),
    "tgbm_trainer_tree_init": (None, [_P, C.c_int]),
    "tgbm_trainer_find_split": (None, [_P, C.c_int]),
    "tgbm_trainer_partition": (None, [_P, C.c_int]),
    "tgbm_trainer_finish_tree": (None, [_P, C.c_int]),
    "tgbm_trainer_metric": (C.c_float, [_P]),
    "tgbm_trainer_info": (C.c_int, [_P, C.c_char_p]),
    "tgbm_trainer_base_score": (C.c_float, [_P]),
    "tgbm_trainer_get": (C.c_size_t, [_P, C.c_char_p, _P, C.c_size_t]),
    "tgbm_trainer_set": (None, [_P, C.c_char_p, _P, C.c_size_t]),
    "tgbm_trainer_set_profiling": (None, [_P, C.c_int]),
    "tgbm_trainer_get_profile": (None, [_P, _P]),
    "tgbm_trainer_get_phase_profile": (C.c_int, [_P, _P, C.c_int]),
    "tgbm_trainer_export_model": (_P, [_P]),
    "tgbm_predict_raw": (None, [C.c_int, _P, _P, _P, _P, C.c_int, C.c_int, C.c_float, C.c_float, _P]),
    "tgbm_predict_raw_noalloc": (C.c_int, [C.c_int, _P, _P, _P, _P, C.c_int, C.c_int, C.c_float, C.c_float, _P]),
    "tgbm_cut_points": (C.c_int, [C.c_int, C.c_int, _P, _P, _P, C.c_int, _P, _P, _P, _P]),
}


def load():
    """Returns the CDLL with typed signatures; raises if the HIP library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libthundergbm.so is missing: build it with `python thundergbm_amd/build.py` "
                "(hipcc, gfx950). There is no CPU fallback.")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
