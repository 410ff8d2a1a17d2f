"""ctypes binding of oracle/libcpu_variant.so: the restated CPU variant of the
reference (timing baseline; test infrastructure)."""
import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
_SO = os.path.join(_DIR, "libcpu_variant.so")
if not os.path.exists(_SO):
    subprocess.check_call(["make", "-C", _DIR, "libcpu_variant.so"], stdout=subprocess.DEVNULL)
lib = C.CDLL(_SO)
lib.cpuv_build_tree.restype = C.c_int
lib.cpuv_build_tree.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                C.c_int, C.c_double, C.c_double, C.c_double, C.c_int, C.c_void_p, C.c_void_p,
                                C.c_void_p, C.c_void_p, C.c_void_p]
lib.cpuv_predict.restype = None
lib.cpuv_predict.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                             C.c_int, C.c_void_p]
lib.cpuv_max_threads.restype = C.c_int


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def build_tree(X, g, h, *, max_depth, split_samples, seed, l1=0.0, l2=1.0, min_split_gain=0.0, n_threads=1):
    X = np.ascontiguousarray(X, np.float32)
    g = np.ascontiguousarray(g, np.float64)
    h = np.ascontiguousarray(h, np.float64)
    n, f = X.shape
    k = g.shape[1]
    m = 2 ** (max_depth + 1) - 1
    leaf = np.empty((m, k))
    feature = np.empty(m, np.int32)
    split = np.empty(m)
    gain = np.empty(m)
    hess = np.empty((m, k))
    lib.cpuv_build_tree(_p(X), n, f, _p(g), _p(h), k, max_depth, split_samples, seed, l1, l2, min_split_gain,
                        n_threads, _p(leaf), _p(feature), _p(split), _p(gain), _p(hess))
    return leaf, feature, split, gain, hess


def predict(X, trees, n_outputs, n_threads=1):
    X = np.ascontiguousarray(X, np.float32)
    n, f = X.shape
    nt = len(trees)
    lp = (C.c_void_p * max(nt, 1))()
    fp = (C.c_void_p * max(nt, 1))()
    sp = (C.c_void_p * max(nt, 1))()
    keep = []
    for i, (lv, ft, sv) in enumerate(trees):
        lv = np.ascontiguousarray(lv, np.float64)
        ft = np.ascontiguousarray(ft, np.int32)
        sv = np.ascontiguousarray(sv, np.float64)
        keep.append((lv, ft, sv))
        lp[i], fp[i], sp[i] = lv.ctypes.data, ft.ctypes.data, sv.ctypes.data
    out = np.empty((n, n_outputs))
    lib.cpuv_predict(_p(X), n, f, nt, lp, fp, sp, n_outputs, n_threads, _p(out))
    return out
