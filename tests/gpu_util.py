"""Helpers shared by the GPU parity tests: run liblbtree.so and the CPU oracle
on the same inputs and compare every observable."""
import numpy as np
import torch

import oracle_lib as orc
from lbtree import ops


def gpu_build(X, g, h, **kw):
    kw.setdefault("taps", True)
    return ops.build_tree(X, g, h, **kw)


def cpu(t):
    return t.cpu().numpy() if isinstance(t, torch.Tensor) else t


def assert_same_floats(a, b, what):
    a, b = np.asarray(a), np.asarray(b)
    assert a.shape == b.shape, what
    # bit patterns must agree except that -0.0 and +0.0 are interchangeable
    same = (a == b) | (np.isnan(a) & np.isnan(b))
    assert same.all(), "%s differs at %s" % (what, np.argwhere(~same)[:5].tolist())


def assert_tree_parity(gr, cr, *, levels=False, leaf_exact=True):
    """gr: ops.BuildResult with taps; cr: oracle TreeResult."""
    assert gr.n_bins == cr.n_bins
    assert np.array_equal(cpu(gr.row_pointers), cr.row_pointers)
    assert_same_floats(cpu(gr.proposals), cr.proposals, "proposals")
    assert np.array_equal(gr.scales, cr.scales), (gr.scales, cr.scales)
    assert np.array_equal(cpu(gr.quantised).astype(np.int64), cr.quantised)
    assert np.array_equal(cpu(gr.node_sums), cr.node_sums)
    assert np.array_equal(cpu(gr.feature), cr.feature)
    assert_same_floats(cpu(gr.split_value), cr.split_value, "split_value")
    if leaf_exact:
        assert_same_floats(cpu(gr.gain), cr.gain, "gain")
        assert_same_floats(cpu(gr.leaf_value), cr.leaf_value, "leaf_value")
        assert_same_floats(cpu(gr.hessian), cr.hessian, "hessian")
    # stated tolerance of the task: leaf values within 1e-6 relative
    assert np.allclose(cpu(gr.leaf_value), cr.leaf_value, rtol=1e-6, atol=0)
    assert np.array_equal(cpu(gr.positions), cr.positions)
    if levels and cr.positions_per_level is not None:
        assert np.array_equal(cpu(gr.positions_per_level), cr.positions_per_level)
    # histograms: compare the nodes both sides hold (the library does not keep
    # levels that are never built)
    lo = max(gr.hist_node_begin, cr.hist_node_begin)
    hi = min(gr.hist_node_end, cr.hist_node_end)
    if hi > lo and gr.histogram is not None and hasattr(cr, "histogram"):
        gh = cpu(gr.histogram)[lo - gr.hist_node_begin: hi - gr.hist_node_begin]
        ch = cr.histogram[lo - cr.hist_node_begin: hi - cr.hist_node_begin]
        assert np.array_equal(gh, ch), "histogram differs"
    assert np.array_equal(gr.level_built_instances, cr.level_built_instances)
    assert np.array_equal(gr.level_built_nodes, cr.level_built_nodes)


def check_row_leaf(gr, X):
    """leaf_value[row_leaf] must be exactly what PredictTask returns for the training rows."""
    from lbtree import ops

    want = ops.predict(X, [(gr.leaf_value, gr.feature, gr.split_value)], gr.leaf_value.shape[1])
    got = gr.leaf_value[gr.row_leaf.long()]
    assert torch.equal(got, want)


def both(X, g, h, *, levels=False, **kw):
    cr = orc.build_tree(X, g, h, max_depth=kw["max_depth"], split_samples=kw["split_samples"], seed=kw["seed"],
                        l1=kw.get("l1_regularization", 0.0), l2=kw.get("l2_regularization", 1.0),
                        min_split_gain=kw.get("min_split_gain", 0.0), feature_set=kw.get("feature_set"),
                        hist_cache_bytes=kw.get("hist_cache_bytes", 0), want_levels=levels)
    gr = gpu_build(X, g, h, taps_levels=levels, row_leaf=True, **kw)
    torch.cuda.synchronize()
    check_row_leaf(gr, X)
    return gr, cr
