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
               taps=False, taps_levels=False, row_leaf=False, wait=True, abs_sum_chunks=None):
    """BUILD_TREE (legateboost/models/tree.py:104-191). Returns a BuildResult with the five task
    outputs as CUDA tensors; with taps=True also the observation points. wait=False returns
    without synchronising the stream (lbt_build_tree_async; not together with taps=True).
    abs_sum_chunks: the chunk sums weighted_gradient(..., sums=True) returned for these g and h."""
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
    if abs_sum_chunks is not None:
        if not (abs_sum_chunks.is_cuda and abs_sum_chunks.dtype == torch.float64 and abs_sum_chunks.is_contiguous()
                and abs_sum_chunks.numel() == 2 * _lib.lib.lbt_abs_sum_chunks(n, k)):
            raise _lib.LbtError("abs_sum_chunks must be the [2][chunks] float64 CUDA tensor of weighted_gradient")
        prm.abs_sum_chunks = abs_sum_chunks.data_ptr()
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
    if taps and not wait:
        raise _lib.LbtError("the observation points need the synchronising call")
    call = _lib.lib.lbt_build_tree if wait else _lib.lib.lbt_build_tree_async
    rc = call(_stream(), X.data_ptr(), _DT[X.dtype], row_offset, n, f, g.data_ptr(), h.data_ptr(),
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


def _tree_arrays(trees, n_outputs):
    nt = len(trees)
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
    return leaf_p, feat_p, split_p, nodes, keep


class PackedEnsemble:
    """An ensemble packed once for repeated prediction (lbt_pack_ensemble): owns the device
    buffer and the descriptor; tied to the dtype and width of the X it will be applied to."""

    def __init__(self, trees, n_outputs, n_features, dtype=torch.float32, device=None):
        if dtype not in _DT:
            raise _lib.LbtError("X must be float32 or float64, got %s" % dtype)
        leaf_p, feat_p, split_p, nodes, keep = _tree_arrays(trees, n_outputs)
        nt = len(trees)
        total = sum(int(nodes[i]) for i in range(nt))
        device = device if device is not None else (keep[0][0].device if keep else "cuda")
        nbytes = int(_lib.lib.lbt_predict_workspace_bytes(nt, total, n_outputs, _DT[dtype]))
        self.buffer = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        self.desc = _lib.PackedEnsemble()
        self.dtype, self.n_features, self.n_outputs = dtype, n_features, n_outputs
        rc = _lib.lib.lbt_pack_ensemble(_stream(), _DT[dtype], n_features, nt, leaf_p, feat_p, split_p, nodes,
                                        n_outputs, self.buffer.data_ptr(), nbytes, C.byref(self.desc))
        _lib.check(rc)

    def predict(self, X):
        X = _check_x(X)
        n, f = X.shape
        out = torch.empty((n, self.n_outputs), dtype=torch.float64, device=X.device)
        rc = _lib.lib.lbt_predict_packed(_stream(), X.data_ptr(), _DT[X.dtype], n, f, C.byref(self.desc),
                                         out.data_ptr())
        _lib.check(rc)
        return out


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


_OBJECTIVES = {"squared_error": _lib.LBT_OBJ_SQUARED_ERROR, "log_loss": _lib.LBT_OBJ_LOG_LOSS}


def weighted_gradient(objective, y, pred, sample_weight=None, learning_rate=1.0, out=None, sums=False):
    """LBBase._get_weighted_gradient (legateboost/legateboost.py:189-224) for "squared_error" or
    "log_loss" in one pass. pred: raw predictions [n, K]; y: [n, K], or [n] / [n, 1] class labels
    for log loss with K > 1. Returns (g, h); `out=(g, h)` reuses two buffers of pred's shape.
    sums=True (or a [2][chunks] float64 tensor to fill): also the chunk sums of |g| and |h| that
    build_tree(abs_sum_chunks=...) takes in place of its own pass over g and h; returns (g, h, sums)."""
    pred = as_device(pred, torch.float64)
    y = as_device(y, torch.float64)
    if pred.dim() != 2:
        raise _lib.LbtError("pred must be [n_rows, n_outputs]")
    n, k = pred.shape
    labels = objective == "log_loss" and k > 1
    if y.numel() != (n if labels else n * k):
        raise _lib.LbtError("y has %d elements, expected %d" % (y.numel(), n if labels else n * k))
    w = None
    if sample_weight is not None:
        w = as_device(sample_weight, torch.float64)
        if w.numel() != n:
            raise _lib.LbtError("sample_weight must have one entry per row")
    if objective not in _OBJECTIVES:
        raise _lib.LbtError("unknown objective %r" % (objective,))
    g, h = out if out is not None else (torch.empty_like(pred), torch.empty_like(pred))
    if sums is not False and sums is not None:
        m = int(_lib.lib.lbt_abs_sum_chunks(n, k))
        part = sums if isinstance(sums, torch.Tensor) else torch.empty((2, m), dtype=torch.float64, device=pred.device)
        if part.numel() != 2 * m or part.dtype != torch.float64 or not part.is_cuda:
            raise _lib.LbtError("sums must be a float64 CUDA tensor of 2 x %d entries" % m)
        rc = _lib.lib.lbt_weighted_gradient_sums(_stream(), _OBJECTIVES[objective], pred.data_ptr(), y.data_ptr(),
                                                 w.data_ptr() if w is not None else None, float(learning_rate), n, k,
                                                 g.data_ptr(), h.data_ptr(), part.data_ptr())
        _lib.check(rc)
        return g, h, part
    rc = _lib.lib.lbt_weighted_gradient(_stream(), _OBJECTIVES[objective], pred.data_ptr(), y.data_ptr(),
                                        w.data_ptr() if w is not None else None, float(learning_rate), n, k,
                                        g.data_ptr(), h.data_ptr())
    _lib.check(rc)
    return g, h


def add_leaf_values(pred, leaf_value, row_leaf):
    """pred += leaf_value[row_leaf], in place: the caller's `train_pred += tree.predict(X)`
    (legateboost/legateboost.py:268) from the rows' leaves recorded by build_tree(row_leaf=True)."""
    if not (pred.is_cuda and pred.dtype == torch.float64 and pred.is_contiguous() and pred.dim() == 2):
        raise _lib.LbtError("pred must be a contiguous CUDA float64 [n_rows, n_outputs] tensor")
    leaf_value = as_device(leaf_value, torch.float64)
    row_leaf = as_device(row_leaf, torch.int32)
    n, k = pred.shape
    if leaf_value.dim() != 2 or leaf_value.shape[1] != k or row_leaf.numel() != n:
        raise _lib.LbtError("leaf_value must be [n_nodes, n_outputs] and row_leaf [n_rows]")
    rc = _lib.lib.lbt_add_leaf_values(_stream(), leaf_value.data_ptr(), leaf_value.shape[0], row_leaf.data_ptr(), n, k,
                                      pred.data_ptr())
    _lib.check(rc)
    return pred


def gather_rows(X, samples, row_offset=0):
    """GATHER (legateboost/utils.py:412-460, src/utils/gather.cu:26-91): rows `samples` (global
    numbers) of X; rows this shard does not hold come back as zeros. samples: a tuple / numpy
    array (sent as the task's host scalar) or a CUDA int64 tensor."""
    X = _check_x(X)
    n, f = X.shape
    on_host = not (isinstance(samples, torch.Tensor) and samples.is_cuda)
    if on_host:
        rows = np.ascontiguousarray(np.asarray(samples, dtype=np.int64).reshape(-1))
        m = rows.shape[0]
        staging = torch.empty(max(m, 1), dtype=torch.int64, device=X.device)
        rows_p, staging_p = rows.ctypes.data, staging.data_ptr()
    else:
        rows = samples.to(torch.int64).contiguous().reshape(-1)
        m = rows.shape[0]
        rows_p, staging_p = rows.data_ptr(), None
    out = torch.empty((m, f), dtype=X.dtype, device=X.device)
    rc = _lib.lib.lbt_gather_rows(_stream(), X.data_ptr(), _DT[X.dtype], row_offset, n, f, rows_p, m, int(on_host),
                                  staging_p, out.data_ptr())
    _lib.check(rc)
    if on_host:
        torch.cuda.current_stream().synchronize()  # the host array is read by the copy on the stream
    return out


def select_split_samples(X, split_samples, seed, dataset_rows=None, row_offset=0):
    """SelectSplitSamples on its own (build_tree.cu:867-964): returns (proposals, row_pointers),
    the proposals of feature f at proposals[row_pointers[f]:row_pointers[f + 1]], ascending,
    the last one +inf."""
    X = _check_x(X)
    n, f = X.shape
    dt = _DT[X.dtype]
    ws = torch.empty(_lib.lib.lbt_select_split_samples_workspace_bytes(f, split_samples, dt), dtype=torch.uint8,
                     device=X.device)
    props = torch.empty(f * split_samples, dtype=X.dtype, device=X.device)
    rp = torch.empty(f + 1, dtype=torch.int32, device=X.device)
    rc = _lib.lib.lbt_select_split_samples(_stream(), X.data_ptr(), dt, row_offset, n, f, split_samples, seed,
                                           n if dataset_rows is None else dataset_rows, props.data_ptr(),
                                           rp.data_ptr(), ws.data_ptr(), ws.numel())
    _lib.check(rc)
    return props[: int(rp[-1])], rp


def quantise_gradients(g, h, seed, row_offset=0):
    """GradientQuantiser and the root sums on their own (build_tree.cu:51-140, :168-204): returns
    (quantised int32 [n][K][2], root_sums int64 [K][2], scales f64 [4])."""
    g = g.contiguous()
    h = h.contiguous()
    if g.dtype != torch.float64 or h.dtype != torch.float64 or g.shape != h.shape or g.dim() != 2:
        raise ValueError("g and h must be float64 [n_rows][n_outputs] of the same shape")
    n, k = g.shape
    ws = torch.empty(_lib.lib.lbt_quantise_gradients_workspace_bytes(n, k), dtype=torch.uint8, device=g.device)
    q = torch.empty((n, k, 2), dtype=torch.int32, device=g.device)
    sums = torch.empty((k, 2), dtype=torch.int64, device=g.device)
    scales = torch.empty(4, dtype=torch.float64, device=g.device)
    rc = _lib.lib.lbt_quantise_gradients(_stream(), g.data_ptr(), h.data_ptr(), n, k, row_offset, seed, q.data_ptr(),
                                         sums.data_ptr(), scales.data_ptr(), ws.data_ptr(), ws.numel())
    _lib.check(rc)
    return q, sums, scales


# ---- the stages of one level on the reference's layouts (include/lbtree.h) -----------------------

def _stage_ws(nbytes, device):
    return torch.empty(int(nbytes), dtype=torch.uint8, device=device)


def histogram_level(X, quantised, proposals, row_pointers, split_samples, positions, level, batch, node_sums,
                    hist_nodes, histogram, workspace=None, reuse_bins=False, deepest_level=None):
    """HistogramKernel of one batch (build_tree.cu:213-577): adds to `histogram`
    [hist_nodes[1] - hist_nodes[0]][K][n_bins][2] int64. Returns the workspace, which holds the
    cached bins for a later call with reuse_bins=True; a workspace allocated here is sized for
    levels up to deepest_level (the part that depends on the level lies behind the cache)."""
    X = _check_x(X)
    n, f = X.shape
    k = quantised.shape[1]
    dt = _DT[X.dtype]
    need = _lib.lib.lbt_histogram_level_workspace_bytes(n, f, split_samples, dt, level)
    if workspace is None:
        need = max(need, _lib.lib.lbt_histogram_level_workspace_bytes(n, f, split_samples, dt,
                                                                      max(level, deepest_level or 0)))
    if workspace is None or workspace.numel() < need:
        if reuse_bins:
            raise _lib.LbtError("reuse_bins needs the workspace of the call that cached the bins")
        workspace = _stage_ws(need, X.device)
    rc = _lib.lib.lbt_histogram_level(_stream(), X.data_ptr(), dt, n, f, quantised.data_ptr(), k, proposals.data_ptr(),
                                      row_pointers.data_ptr(), split_samples, positions.data_ptr(), level, batch[0],
                                      batch[1], node_sums.data_ptr(), hist_nodes[0], hist_nodes[1],
                                      histogram.data_ptr(), workspace.data_ptr(), workspace.numel(), int(reuse_bins))
    _lib.check(rc)
    return workspace


def scan(histogram, hist_nodes, row_pointers, n_bins, node_sums, batch):
    """scan_kernel of one batch (build_tree.cu:597-668), in place."""
    k = histogram.shape[1]
    f = row_pointers.numel() - 1
    rc = _lib.lib.lbt_scan(_stream(), histogram.data_ptr(), hist_nodes[0], hist_nodes[1], k, f, row_pointers.data_ptr(),
                           n_bins, node_sums.data_ptr(), batch[0], batch[1])
    _lib.check(rc)


def best_split(histogram, hist_nodes, proposals, row_pointers, n_bins, node_sums, scales, batch, leaf, feature, split,
               gain, l1_regularization=0.0, l2_regularization=1.0, min_split_gain=0.0, feature_set=None):
    """perform_best_split of one batch (build_tree.cu:682-782): updates node_sums, leaf, feature,
    split and gain in place."""
    k = histogram.shape[1]
    f = row_pointers.numel() - 1
    ws = _stage_ws(_lib.lib.lbt_best_split_workspace_bytes(f, n_bins, batch[0], batch[1]), histogram.device)
    fs = None
    if feature_set is not None:
        fs = as_device(np.asarray(feature_set, dtype=np.uint8) if not isinstance(feature_set, torch.Tensor)
                       else feature_set.to(torch.uint8))
    rc = _lib.lib.lbt_best_split(_stream(), histogram.data_ptr(), hist_nodes[0], hist_nodes[1], k, f,
                                 proposals.data_ptr(), _DT[proposals.dtype], row_pointers.data_ptr(), n_bins,
                                 fs.data_ptr() if fs is not None else None, node_sums.data_ptr(), scales.data_ptr(),
                                 l1_regularization, l2_regularization, min_split_gain, batch[0], batch[1],
                                 leaf.data_ptr(), feature.data_ptr(), split.data_ptr(), gain.data_ptr(), ws.data_ptr(),
                                 ws.numel())
    _lib.check(rc)
    torch.cuda.current_stream().synchronize()  # ws and fs are released when this returns


def update_positions(X, positions, feature, split, level):
    """UpdatePositions (build_tree.cu:1026-1080), in place on the (node, row) pairs."""
    X = _check_x(X)
    n, f = X.shape
    ws = _stage_ws(_lib.lib.lbt_update_positions_workspace_bytes(n, level), X.device)
    rc = _lib.lib.lbt_update_positions(_stream(), X.data_ptr(), _DT[X.dtype], n, f, positions.data_ptr(),
                                       feature.data_ptr(), split.data_ptr(), level, ws.data_ptr(), ws.numel())
    _lib.check(rc)
    torch.cuda.current_stream().synchronize()
