"""Thin, allocation-owning wrappers over the C ABI. torch only provides device
memory and the current stream; all computation happens in liblbtree.so."""
import ctypes as C

import numpy as np
import torch

from . import _lib

_DT = {torch.float32: _lib.LBT_F32, torch.float64: _lib.LBT_F64}


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def as_device(a, dtype=None):
    """numpy / torch (any device) -> contiguous CUDA tensor, dtype preserved unless given."""
    if isinstance(a, torch.Tensor):
        t = a
    else:
        t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None and t.dtype != dtype:
        t = t.to(dtype)
    if not t.is_cuda:
        t = t.cuda()
    return t.contiguous()


def _check_x(X):
    X = as_device(X)
    if X.dtype not in _DT:
        # src/cpp_utils/cpp_utils.h:131-136: only float and double are dispatched
        raise _lib.LbtError("X must be float32 or float64, got %s" % X.dtype)
    if X.dim() != 2:
        raise _lib.LbtError("X must be 2-dimensional")
    return X


_workspace = {}


def _get_workspace(nbytes, device):
    """One grow-only scratch buffer per device, reused by successive calls."""
    ws = _workspace.get(device)
    if ws is None or ws.numel() < nbytes:
        _workspace[device] = None
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _workspace[device] = ws
    return ws


class BuildResult:
    pass


def build_tree(X, g, h, *, max_depth, split_samples, seed, l1_regularization=0.0, l2_regularization=1.0,
               min_split_gain=0.0, feature_set=None, dataset_rows=None, row_offset=0, hist_cache_bytes=0,
               taps=False, taps_levels=False, row_leaf=False):
    """BUILD_TREE (legateboost/models/tree.py:104-191). Returns a BuildResult with the five task
    outputs as CUDA tensors; with taps=True also the observation points."""
    X = _check_x(X)
    g = as_device(g, torch.float64)
    h = as_device(h, torch.float64)
    if g.dim() != 2 or g.shape != h.shape or g.shape[0] != X.shape[0]:
        raise _lib.LbtError("g and h must be [n_rows, n_outputs] and aligned with X")
    n, f = X.shape
    k = g.shape[1]
    dev = X.device
    max_nodes = 2 ** (max_depth + 1) - 1
    prm = _lib.BuildParams(max_depth, max_nodes, split_samples, seed,
                           dataset_rows if dataset_rows is not None else n, l1_regularization,
                           l2_regularization, min_split_gain, hist_cache_bytes)
    nbytes = _lib.lib.lbt_build_tree_workspace_bytes(n, f, k, max_depth, split_samples, _DT[X.dtype], hist_cache_bytes)
    if nbytes == 0:
        # let the library produce the message for the offending argument
        ws = None
    else:
        ws = _get_workspace(nbytes, dev)
    r = BuildResult()
    r.leaf_value = torch.empty((max(max_nodes, 1), k), dtype=torch.float64, device=dev)
    r.feature = torch.empty(max(max_nodes, 1), dtype=torch.int32, device=dev)
    r.split_value = torch.empty(max(max_nodes, 1), dtype=torch.float64, device=dev)
    r.gain = torch.empty(max(max_nodes, 1), dtype=torch.float64, device=dev)
    r.hessian = torch.empty((max(max_nodes, 1), k), dtype=torch.float64, device=dev)
    fs = None
    if feature_set is not None:
        fs = as_device(feature_set).to(torch.uint8)
        if fs.shape != (f,):
            raise _lib.LbtError("feature_set must have shape (n_features,)")
    tp = None
    keep = []
    if taps or row_leaf:
        tp = _lib.BuildTaps()
    if row_leaf:
        # leaf of every training row, so that the caller can update its predictions without a traversal
        r.row_leaf = torch.empty(n, dtype=torch.int32, device=dev)
        tp.row_leaf = r.row_leaf.data_ptr()
    if taps:
        r.proposals_buf = torch.empty(f * split_samples, dtype=X.dtype, device=dev)
        r.row_pointers = torch.empty(f + 1, dtype=torch.int32, device=dev)
        r.quantised = torch.empty((n, k, 2), dtype=torch.int32, device=dev)
        r.node_sums = torch.empty((max_nodes, k, 2), dtype=torch.int64, device=dev)
        r.positions = torch.empty((n, 2), dtype=torch.int32, device=dev)
        tp.proposals = r.proposals_buf.data_ptr()
        tp.row_pointers = r.row_pointers.data_ptr()
        tp.quantised = r.quantised.data_ptr()
        tp.node_sums = r.node_sums.data_ptr()
        tp.positions = r.positions.data_ptr()
        if taps_levels and max_depth > 0:
            r.positions_per_level = torch.empty((max_depth, n, 2), dtype=torch.int32, device=dev)
            tp.positions_per_level = r.positions_per_level.data_ptr()
        cache = hist_cache_bytes if hist_cache_bytes > 0 else 1000000000
        used_nodes = 2 ** max_depth - 1
        cap = min(max(cache, f * split_samples * k * 16) // 8 + 16, used_nodes * f * split_samples * k * 2)
        r.hist_buf = torch.zeros(max(cap, 1), dtype=torch.int64, device=dev)
        tp.histogram = r.hist_buf.data_ptr()
        tp.histogram_capacity = r.hist_buf.numel()
        li = np.zeros(max(max_depth, 1), np.int64)
        lbi = np.zeros(max(max_depth, 1), np.int64)
        lbn = np.zeros(max(max_depth, 1), np.int32)
        keep += [li, lbi, lbn]
        tp.level_instances = li.ctypes.data
        tp.level_built_instances = lbi.ctypes.data
        tp.level_built_nodes = lbn.ctypes.data
    rc = _lib.lib.lbt_build_tree(_stream(), X.data_ptr(), _DT[X.dtype], row_offset, n, f, g.data_ptr(), h.data_ptr(),
                                 k, fs.data_ptr() if fs is not None else None, C.byref(prm), r.leaf_value.data_ptr(),
                                 r.feature.data_ptr(), r.split_value.data_ptr(), r.gain.data_ptr(),
                                 r.hessian.data_ptr(), ws.data_ptr() if ws is not None else None,
                                 ws.numel() if ws is not None else 0, C.byref(tp) if tp is not None else None)
    _lib.check(rc)
    if taps:
        r.n_bins = tp.n_bins
        r.proposals = r.proposals_buf[: tp.n_bins]
        r.scales = np.array(list(tp.scales))
        r.hist_node_begin = tp.hist_node_begin
        r.hist_node_end = tp.hist_node_end
        nn = r.hist_node_end - r.hist_node_begin
        need = nn * k * tp.n_bins * 2
        r.histogram = r.hist_buf[:need].view(nn, k, tp.n_bins, 2) if need <= r.hist_buf.numel() else None
        r.level_instances = li[:max_depth]
        r.level_built_instances = lbi[:max_depth]
        r.level_built_nodes = lbn[:max_depth]
    return r


def predict(X, trees, n_outputs, tiled=True):
    """PREDICT (legateboost/models/tree.py:245-280). trees: sequence of
    (leaf_value [nodes,K] f64, feature [nodes] i32, split_value [nodes] f64) CUDA tensors."""
    X = _check_x(X)
    n, f = X.shape
    nt = len(trees)
    out = torch.empty((n, n_outputs), dtype=torch.float64, device=X.device)
    leaf_p = (C.c_void_p * max(nt, 1))()
    feat_p = (C.c_void_p * max(nt, 1))()
    split_p = (C.c_void_p * max(nt, 1))()
    nodes = (C.c_int32 * max(nt, 1))()
    keep = []
    for i, (lv, ft, sp) in enumerate(trees):
        lv = as_device(lv, torch.float64)
        ft = as_device(ft, torch.int32)
        sp = as_device(sp, torch.float64)
        if lv.dim() != 2 or lv.shape[1] != n_outputs or ft.shape[0] != lv.shape[0] or sp.shape[0] != lv.shape[0]:
            raise _lib.LbtError("tree %d has inconsistent shapes" % i)
        keep.append((lv, ft, sp))
        leaf_p[i], feat_p[i], split_p[i], nodes[i] = lv.data_ptr(), ft.data_ptr(), sp.data_ptr(), ft.shape[0]
    total_nodes = sum(int(nodes[i]) for i in range(nt))
    ws = None
    if tiled:
        ws = torch.empty(int(_lib.lib.lbt_predict_workspace_bytes(nt, total_nodes, n_outputs, _DT[X.dtype])), dtype=torch.uint8,
                         device=X.device)
    rc = _lib.lib.lbt_predict(_stream(), X.data_ptr(), _DT[X.dtype], n, f, nt, leaf_p, feat_p, split_p, nodes,
                              n_outputs, out.data_ptr(), ws.data_ptr() if ws is not None else None,
                              ws.numel() if ws is not None else 0)
    _lib.check(rc)
    return out


def update_tree(X, g, h, feature, split_value, l1_regularization, l2_regularization):
    """UPDATE_TREE (legateboost/models/tree.py:197-240). Returns (leaf_value, hessian)."""
    X = _check_x(X)
    g = as_device(g, torch.float64)
    h = as_device(h, torch.float64)
    feature = as_device(feature, torch.int32)
    split_value = as_device(split_value, torch.float64)
    n, f = X.shape
    k = g.shape[1]
    m = feature.shape[0]
    leaf = torch.empty((m, k), dtype=torch.float64, device=X.device)
    hess = torch.empty((m, k), dtype=torch.float64, device=X.device)
    nbytes = _lib.lib.lbt_update_tree_workspace_bytes(n, k, m)
    ws = torch.empty(int(nbytes), dtype=torch.uint8, device=X.device)
    rc = _lib.lib.lbt_update_tree(_stream(), X.data_ptr(), _DT[X.dtype], n, f, g.data_ptr(), h.data_ptr(), k,
                                  feature.data_ptr(), split_value.data_ptr(), m, l1_regularization,
                                  l2_regularization, leaf.data_ptr(), hess.data_ptr(), ws.data_ptr(), ws.numel())
    _lib.check(rc)
    return leaf, hess
