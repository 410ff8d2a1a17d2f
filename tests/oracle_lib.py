"""ctypes binding of the CPU oracle (oracle/liblbt_oracle.so) for the tests.

The oracle is test infrastructure: only tests, the smoke check and the
benchmark's CPU-baseline leg load it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_SO = os.path.join(_ORACLE_DIR, "liblbt_oracle.so")


class OrcParams(C.Structure):
    _fields_ = [
        ("max_depth", C.c_int32),
        ("max_nodes", C.c_int32),
        ("split_samples", C.c_int32),
        ("seed", C.c_int32),
        ("dataset_rows", C.c_int64),
        ("l1", C.c_double),
        ("l2", C.c_double),
        ("min_split_gain", C.c_double),
        ("hist_cache_bytes", C.c_int64),
    ]


class OrcTaps(C.Structure):
    _fields_ = [
        ("proposals", C.c_void_p),
        ("row_pointers", C.c_void_p),
        ("n_bins", C.c_int32),
        ("scales", C.c_double * 4),
        ("quantised", C.c_void_p),
        ("node_sums", C.c_void_p),
        ("positions", C.c_void_p),
        ("positions_per_level", C.c_void_p),
        ("histogram", C.c_void_p),
        ("histogram_capacity", C.c_int64),
        ("hist_node_begin", C.c_int32),
        ("hist_node_end", C.c_int32),
        ("level_instances", C.c_void_p),
        ("level_built_instances", C.c_void_p),
        ("level_built_nodes", C.c_void_p),
    ]


def _load():
    if not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_ORACLE_DIR, "lbt_oracle.c")
    ):
        subprocess.check_call(["make", "-C", _ORACLE_DIR, "liblbt_oracle.so"], stdout=subprocess.DEVNULL)
    lib = C.CDLL(_SO)
    lib.orc_minstd_seed.restype = C.c_uint32
    lib.orc_minstd_seed.argtypes = [C.c_uint32]
    lib.orc_minstd_next.restype = C.c_uint32
    lib.orc_minstd_next.argtypes = [C.c_uint32]
    lib.orc_minstd_discard.restype = C.c_uint32
    lib.orc_minstd_discard.argtypes = [C.c_uint32, C.c_uint64]
    lib.orc_uniform01.restype = C.c_double
    lib.orc_uniform01.argtypes = [C.c_uint32]
    lib.orc_hash.restype = C.c_int64
    lib.orc_hash.argtypes = [C.c_int64]
    lib.orc_hash_combine2.restype = C.c_int64
    lib.orc_hash_combine2.argtypes = [C.c_int64, C.c_int64, C.c_int64]
    lib.orc_quantise_one.restype = None
    lib.orc_quantise_one.argtypes = [C.c_double, C.c_double, C.c_double, C.c_double, C.c_int64, C.c_void_p]
    lib.orc_calculate_gain.restype = C.c_double
    lib.orc_calculate_gain.argtypes = [C.c_double] * 9
    lib.orc_calculate_leaf_value.restype = C.c_double
    lib.orc_calculate_leaf_value.argtypes = [C.c_double] * 4
    lib.orc_row_samples.restype = None
    lib.orc_row_samples.argtypes = [C.c_int32, C.c_int64, C.c_int32, C.c_void_p]
    lib.orc_split_proposals.restype = C.c_int32
    lib.orc_split_proposals.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int32, C.c_int32,
                                        C.c_int32, C.c_int64, C.c_void_p, C.c_void_p]
    lib.orc_abs_sums.restype = None
    lib.orc_abs_sums.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    lib.orc_scales.restype = None
    lib.orc_scales.argtypes = [C.c_void_p, C.c_void_p]
    lib.orc_quantise_all.restype = None
    lib.orc_quantise_all.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int64, C.c_int32,
                                     C.c_void_p, C.c_void_p]
    lib.orc_build_tree.restype = C.c_int
    lib.orc_build_tree.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int32, C.c_void_p,
                                   C.c_void_p, C.c_int32, C.c_void_p, C.POINTER(OrcParams), C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(OrcTaps)]
    lib.orc_predict.restype = None
    lib.orc_predict.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                C.c_void_p, C.c_int32, C.c_void_p]
    lib.orc_update_tree.restype = None
    lib.orc_update_tree.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p,
                                    C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_double, C.c_double,
                                    C.c_void_p, C.c_void_p]
    lib.orc_weighted_gradient.restype = None
    lib.orc_weighted_gradient.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_int64,
                                          C.c_int32, C.c_void_p, C.c_void_p]
    lib.orc_add_leaf_values.restype = None
    lib.orc_add_leaf_values.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]
    lib.orc_gather_rows.restype = None
    lib.orc_gather_rows.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_int64,
                                    C.c_void_p]
    lib.orc_histogram_level.restype = None
    lib.orc_histogram_level.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p,
                                        C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_int32, C.c_int32,
                                        C.c_void_p]
    lib.orc_scan.restype = None
    lib.orc_scan.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32,
                             C.c_int32]
    lib.orc_best_split.restype = None
    lib.orc_best_split.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int,
                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_double, C.c_double,
                                   C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.orc_update_positions.restype = None
    lib.orc_update_positions.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_int32]
    return lib


lib = _load()


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _check_x(X):
    X = np.ascontiguousarray(X)
    assert X.dtype in (np.float32, np.float64) and X.ndim == 2
    return X, int(X.dtype == np.float64)


def row_samples(seed, dataset_rows, split_samples):
    out = np.empty(split_samples, np.int64)
    lib.orc_row_samples(seed, dataset_rows, split_samples, _p(out))
    return out


def split_proposals(X, seed, split_samples, dataset_rows=None, row_offset=0):
    X, is64 = _check_x(X)
    n, f = X.shape
    props = np.empty(f * split_samples, X.dtype)
    rp = np.empty(f + 1, np.int32)
    nb = lib.orc_split_proposals(_p(X), is64, row_offset, n, f, seed, split_samples,
                                 dataset_rows if dataset_rows is not None else n, _p(props), _p(rp))
    return props[:nb].copy(), rp


def abs_sums(g, h):
    g = np.ascontiguousarray(g, np.float64).ravel()
    h = np.ascontiguousarray(h, np.float64).ravel()
    out = np.empty(2, np.float64)
    lib.orc_abs_sums(_p(g), _p(h), g.size, _p(out))
    return out


def scales(sums):
    sums = np.ascontiguousarray(sums, np.float64)
    out = np.empty(4, np.float64)
    lib.orc_scales(_p(sums), _p(out))
    return out


def quantise_all(g, h, seed, sc, row_offset=0):
    g = np.ascontiguousarray(g, np.float64)
    h = np.ascontiguousarray(h, np.float64)
    n, k = g.shape
    q = np.empty((n, k, 2), np.int64)
    sc = np.ascontiguousarray(sc, np.float64)
    lib.orc_quantise_all(_p(g), _p(h), n, k, row_offset, seed, _p(sc), _p(q))
    return q


class TreeResult:
    pass


def build_tree(X, g, h, *, max_depth, split_samples, seed, l1=0.0, l2=1.0, min_split_gain=0.0,
               feature_set=None, dataset_rows=None, row_offset=0, hist_cache_bytes=0,
               want_levels=False, want_hist=True):
    """Runs the oracle's BuildTreeTask restatement; returns outputs and taps."""
    X, is64 = _check_x(X)
    g = np.ascontiguousarray(g, np.float64)
    h = np.ascontiguousarray(h, np.float64)
    n, f = X.shape
    k = g.shape[1]
    max_nodes = 2 ** (max_depth + 1) - 1
    prm = OrcParams(max_depth, max_nodes, split_samples, seed, dataset_rows if dataset_rows is not None else n,
                    l1, l2, min_split_gain, hist_cache_bytes)
    r = TreeResult()
    r.leaf_value = np.empty((max_nodes, k), np.float64)
    r.feature = np.empty(max_nodes, np.int32)
    r.split_value = np.empty(max_nodes, np.float64)
    r.gain = np.empty(max_nodes, np.float64)
    r.hessian = np.empty((max_nodes, k), np.float64)
    taps = OrcTaps()
    props = np.empty(f * split_samples, X.dtype)
    rp = np.empty(f + 1, np.int32)
    q = np.empty((n, k, 2), np.int64)
    ns = np.empty((max_nodes, k, 2), np.int64)
    pos = np.empty((n, 2), np.int32)
    taps.proposals = props.ctypes.data
    taps.row_pointers = rp.ctypes.data
    taps.quantised = q.ctypes.data
    taps.node_sums = ns.ctypes.data
    taps.positions = pos.ctypes.data
    lvl = None
    if want_levels and max_depth > 0:
        lvl = np.empty((max_depth, n, 2), np.int32)
        taps.positions_per_level = lvl.ctypes.data
    li = np.zeros(max(max_depth, 1), np.int64)
    lbi = np.zeros(max(max_depth, 1), np.int64)
    lbn = np.zeros(max(max_depth, 1), np.int32)
    taps.level_instances = li.ctypes.data
    taps.level_built_instances = lbi.ctypes.data
    taps.level_built_nodes = lbn.ctypes.data
    hist = None
    if want_hist:
        # upper bound: the cache never exceeds max(1 GB rule, one node)
        cache = hist_cache_bytes if hist_cache_bytes > 0 else 1000000000
        cap = max(cache, f * split_samples * k * 16) // 8 + 16
        cap = min(cap, (2 ** (max_depth + 2)) * f * split_samples * k * 2)
        hist = np.zeros(cap, np.int64)
        taps.histogram = hist.ctypes.data
        taps.histogram_capacity = cap
    fs = None
    if feature_set is not None:
        fs = np.ascontiguousarray(feature_set).astype(np.uint8)
    rc = lib.orc_build_tree(_p(X), is64, row_offset, n, f, _p(g), _p(h), k, _p(fs) if fs is not None else None,
                            C.byref(prm), _p(r.leaf_value), _p(r.feature), _p(r.split_value), _p(r.gain),
                            _p(r.hessian), C.byref(taps))
    if rc != 0:
        raise ValueError("orc_build_tree failed: %d" % rc)
    nb = taps.n_bins
    r.n_bins = nb
    r.proposals = props[:nb].copy()
    r.row_pointers = rp
    r.scales = np.array(list(taps.scales))
    r.quantised = q
    r.node_sums = ns
    r.positions = pos
    r.positions_per_level = lvl
    r.hist_node_begin = taps.hist_node_begin
    r.hist_node_end = taps.hist_node_end
    if hist is not None:
        nn = r.hist_node_end - r.hist_node_begin
        r.histogram = hist[: nn * k * nb * 2].reshape(nn, k, nb, 2).copy()
    r.level_instances = li[:max_depth]
    r.level_built_instances = lbi[:max_depth]
    r.level_built_nodes = lbn[:max_depth]
    return r


def predict(X, trees, n_outputs):
    """trees: list of (leaf[max_nodes,K] f64, feature[max_nodes] i32, split[max_nodes] f64)."""
    X, is64 = _check_x(X)
    n, f = X.shape
    nt = len(trees)
    keep = []
    leaf_p = (C.c_void_p * max(nt, 1))()
    feat_p = (C.c_void_p * max(nt, 1))()
    split_p = (C.c_void_p * max(nt, 1))()
    for i, (lv, ft, sp) in enumerate(trees):
        lv = np.ascontiguousarray(lv, np.float64)
        ft = np.ascontiguousarray(ft, np.int32)
        sp = np.ascontiguousarray(sp, np.float64)
        keep.append((lv, ft, sp))
        leaf_p[i], feat_p[i], split_p[i] = lv.ctypes.data, ft.ctypes.data, sp.ctypes.data
    out = np.empty((n, n_outputs), np.float64)
    lib.orc_predict(_p(X), is64, n, f, nt, leaf_p, feat_p, split_p, n_outputs, _p(out))
    return out


def update_tree(X, g, h, feature, split, l1, l2):
    X, is64 = _check_x(X)
    g = np.ascontiguousarray(g, np.float64)
    h = np.ascontiguousarray(h, np.float64)
    feature = np.ascontiguousarray(feature, np.int32)
    split = np.ascontiguousarray(split, np.float64)
    n, f = X.shape
    k = g.shape[1]
    m = feature.shape[0]
    leaf = np.empty((m, k), np.float64)
    hess = np.empty((m, k), np.float64)
    lib.orc_update_tree(_p(X), is64, n, f, _p(g), _p(h), k, _p(feature), _p(split), m, l1, l2, _p(leaf), _p(hess))
    return leaf, hess


OBJECTIVES = {"squared_error": 0, "log_loss": 1}


def weighted_gradient(objective, y, pred, weight=None, learning_rate=1.0):
    pred = np.ascontiguousarray(pred, np.float64)
    y = np.ascontiguousarray(y, np.float64)
    n, k = pred.shape
    w = None if weight is None else np.ascontiguousarray(weight, np.float64)
    g = np.empty_like(pred)
    h = np.empty_like(pred)
    lib.orc_weighted_gradient(OBJECTIVES[objective], _p(pred), _p(y), None if w is None else _p(w),
                              learning_rate, n, k, _p(g), _p(h))
    return g, h


def add_leaf_values(pred, leaf, row_leaf):
    pred = np.array(pred, np.float64, order="C")
    leaf = np.ascontiguousarray(leaf, np.float64)
    row_leaf = np.ascontiguousarray(row_leaf, np.int32)
    lib.orc_add_leaf_values(_p(leaf), _p(row_leaf), pred.shape[0], pred.shape[1], _p(pred))
    return pred


def gather_rows(X, rows, row_offset=0):
    X, is64 = _check_x(X)
    rows = np.ascontiguousarray(rows, np.int64)
    out = np.empty((rows.shape[0], X.shape[1]), X.dtype)
    lib.orc_gather_rows(_p(X), is64, row_offset, X.shape[0], X.shape[1], _p(rows), rows.shape[0], _p(out))
    return out


# ---- the stages of one level (orc_build_tree runs these four in a loop); arrays are updated in place

def histogram_level(X, quantised, proposals, row_pointers, positions, batch, node_sums, hist_nodes, histogram):
    X, is64 = _check_x(X)
    n, f = X.shape
    assert quantised.dtype == np.int64 and positions.dtype == np.int32 and histogram.dtype == np.int64
    assert proposals.dtype == X.dtype and node_sums.dtype == np.int64 and row_pointers.dtype == np.int32
    lib.orc_histogram_level(_p(X), is64, n, f, _p(quantised), quantised.shape[1], _p(proposals), _p(row_pointers),
                            _p(positions), batch[0], batch[1], _p(node_sums), hist_nodes[0], hist_nodes[1],
                            _p(histogram))


def scan(histogram, hist_nodes, row_pointers, node_sums, batch):
    assert histogram.dtype == np.int64 and node_sums.dtype == np.int64
    lib.orc_scan(_p(histogram), hist_nodes[0], hist_nodes[1], histogram.shape[1], len(row_pointers) - 1,
                 _p(row_pointers), _p(node_sums), batch[0], batch[1])


def best_split(histogram, hist_nodes, proposals, row_pointers, node_sums, scales4, batch, leaf, feature, split, gain,
               l1=0.0, l2=1.0, min_split_gain=0.0, feature_set=None):
    fs = None if feature_set is None else np.ascontiguousarray(feature_set, np.uint8)
    scales4 = np.ascontiguousarray(scales4, np.float64)
    lib.orc_best_split(_p(histogram), hist_nodes[0], hist_nodes[1], histogram.shape[1], len(row_pointers) - 1,
                       _p(proposals), int(proposals.dtype == np.float64), _p(row_pointers),
                       _p(fs) if fs is not None else None, _p(node_sums), _p(scales4), l1, l2, min_split_gain,
                       batch[0], batch[1], _p(leaf), _p(feature), _p(split), _p(gain))


def update_positions(X, positions, feature, split, max_nodes):
    X, is64 = _check_x(X)
    n, f = X.shape
    assert positions.dtype == np.int32 and feature.dtype == np.int32 and split.dtype == np.float64
    lib.orc_update_positions(_p(X), is64, n, f, _p(positions), _p(feature), _p(split), max_nodes)
