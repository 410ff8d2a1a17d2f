"""CPU-side checks of the drop-in boundary: the shared library loads, exports
every symbol that include/lbtree.h declares, and rejects bad arguments before
touching a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "lbtree.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lbt_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from lbtree import _lib

    names = declared_symbols()
    assert "lbt_build_tree" in names and "lbt_predict" in names and "lbt_update_tree" in names
    for n in names:
        assert hasattr(_lib.lib, n), n
    assert sorted(_lib.EXPORTS) == names
    assert _lib.lib.lbt_version() >= 3
    assert _lib.lib.lbt_release_thread_resources() == 0  # nothing held yet: nothing to do, no GPU call


def test_workspace_query():
    from lbtree import _lib

    q = _lib.lib.lbt_build_tree_workspace_bytes
    a = q(100000, 32, 1, 6, 256, _lib.LBT_F32, 0)
    b = q(200000, 32, 1, 6, 256, _lib.LBT_F32, 0)
    c = q(100000, 32, 4, 6, 256, _lib.LBT_F32, 0)
    assert 0 < a < b and a < c
    # config 2 of the benchmark (4 GB of X) needs about as much scratch again: bin cache,
    # its feature-major copy, positions and the 1e9-byte histogram budget
    assert q(10_000_000, 100, 1, 8, 256, _lib.LBT_F32, 0) < 5_000_000_000
    # invalid shapes give 0
    assert q(0, 32, 1, 6, 256, _lib.LBT_F32, 0) == 0
    assert q(1000, 32, 1, 6, 4096, _lib.LBT_F32, 0) == 0
    assert q(1000, 32, 1, 40, 256, _lib.LBT_F32, 0) == 0
    assert q(1000, 32, 1, 6, 256, 7, 0) == 0
    assert _lib.lib.lbt_update_tree_workspace_bytes(1000, 2, 127) >= 127 * 2 * 16
    # packed ensemble: 8 bytes per node for float X plus the leaf values
    pw = _lib.lib.lbt_predict_workspace_bytes(1000, 511000, 1, _lib.LBT_F32)
    assert 511000 * 16 <= pw < 511000 * 16 + (1 << 20)
    assert _lib.lib.lbt_predict_workspace_bytes(10, 100, 0, _lib.LBT_F32) == 0


def test_bad_arguments_are_rejected_without_a_gpu():
    from lbtree import _lib

    prm = _lib.BuildParams(3, 15, 16, 0, 10, 0.0, 1.0, 0.0, 0)
    one = C.c_void_p(16)  # never dereferenced: validation fails first
    rc = _lib.lib.lbt_build_tree(None, one, _lib.LBT_F32, 0, 10, 2, one, one, 1, None, C.byref(prm), one, one, one,
                                 one, one, None, 0, None)
    assert rc == -3 and b"workspace" in _lib.lib.lbt_last_error()
    prm.max_nodes = 14
    rc = _lib.lib.lbt_build_tree(None, one, _lib.LBT_F32, 0, 10, 2, one, one, 1, None, C.byref(prm), one, one, one,
                                 one, one, one, 1 << 20, None)
    assert rc == -1 and b"max_nodes" in _lib.lib.lbt_last_error()
    prm.max_nodes = 15
    prm.struct_bytes = 48  # a struct of another version of the header, or one that was never filled in
    rc = _lib.lib.lbt_build_tree(None, one, _lib.LBT_F32, 0, 10, 2, one, one, 1, None, C.byref(prm), one, one, one,
                                 one, one, one, 1 << 20, None)
    assert rc == -1 and b"struct_bytes" in _lib.lib.lbt_last_error()
    prm.struct_bytes = C.sizeof(_lib.BuildParams)
    prm.abs_sum_chunks = 16 + 8  # inside g
    rc = _lib.lib.lbt_build_tree(None, one, _lib.LBT_F32, 0, 10, 2, one, one, 1, None, C.byref(prm), one, one, one,
                                 one, one, one, 1 << 20, None)
    assert rc == -1 and b"overlaps" in _lib.lib.lbt_last_error()
    prm.abs_sum_chunks = None
    prm.split_samples = 4096
    rc = _lib.lib.lbt_build_tree(None, one, _lib.LBT_F32, 0, 10, 2, one, one, 1, None, C.byref(prm), one, one, one,
                                 one, one, one, 1 << 20, None)
    assert rc == -1 and b"split_samples" in _lib.lib.lbt_last_error()
    rc = _lib.lib.lbt_build_tree(None, one, 5, 0, 10, 2, one, one, 1, None, C.byref(prm), one, one, one, one, one,
                                 one, 1 << 20, None)
    assert rc == -1
    rc = _lib.lib.lbt_predict(None, one, 9, 10, 2, 0, None, None, None, None, 1, one, None, 0)
    assert rc == -1
    two = C.c_void_p(32)
    ens = _lib.PackedEnsemble()
    assert _lib.lib.lbt_predict_packed(None, one, _lib.LBT_F32, 10, 2, C.byref(ens), one) == -1
    assert b"not packed" in _lib.lib.lbt_last_error()
    assert _lib.lib.lbt_pack_ensemble(None, _lib.LBT_F32, 2, 0, None, None, None, None, 1, one, 64, C.byref(ens)) == -1
    rc = _lib.lib.lbt_weighted_gradient(None, 7, one, one, None, 1.0, 10, 1, two, two)
    assert rc == -1 and b"objective" in _lib.lib.lbt_last_error()
    rc = _lib.lib.lbt_weighted_gradient(None, _lib.LBT_OBJ_SQUARED_ERROR, one, two, None, 1.0, 10, 1, one, two)
    assert rc == -1 and b"alias" in _lib.lib.lbt_last_error()
    assert _lib.lib.lbt_weighted_gradient(None, _lib.LBT_OBJ_LOG_LOSS, None, None, None, 1.0, 0, 3, None, None) == 0
    assert _lib.lib.lbt_add_leaf_values(None, one, 0, one, 10, 1, one) == -1
    assert _lib.lib.lbt_add_leaf_values(None, None, 3, None, 0, 1, None) == 0
    assert _lib.lib.lbt_gather_rows(None, one, 3, 0, 10, 2, one, 4, 0, None, one) == -1
    rc = _lib.lib.lbt_gather_rows(None, one, _lib.LBT_F32, 0, 10, 2, one, 4, 1, None, one)
    assert rc == -1 and b"staging" in _lib.lib.lbt_last_error()
    q = _lib.lib.lbt_select_split_samples_workspace_bytes
    assert 0 < q(4, 16, _lib.LBT_F32) <= q(4, 16, _lib.LBT_F64) and q(4, 4096, _lib.LBT_F32) == 0
    sel = _lib.lib.lbt_select_split_samples
    assert sel(None, one, _lib.LBT_F32, 0, 10, 2, 4096, 1, 10, one, one, one, 1 << 20) == -1
    assert b"split_samples" in _lib.lib.lbt_last_error()
    assert sel(None, one, _lib.LBT_F32, 0, 10, 2, 16, 1, 0, one, one, one, 1 << 20) == -1
    assert sel(None, one, _lib.LBT_F32, 0, 10, 2, 16, 1, 10, one, one, one, 8) == -3
    assert _lib.lib.lbt_quantise_gradients_workspace_bytes(1000, 2) > 0
    assert _lib.lib.lbt_quantise_gradients_workspace_bytes(0, 2) == 0
    qg = _lib.lib.lbt_quantise_gradients
    assert qg(None, one, one, 10, 0, 0, 1, one, one, one, one, 1 << 20) == -1
    assert qg(None, one, one, 10, 1, 0, 1, one, None, one, one, 1 << 20) == -1
    assert qg(None, one, one, 10, 1, 0, 1, one, one, one, one, 8) == -3
    assert qg(None, one, one, 10, 1, 0, 1, one, C.c_void_p(24), one, one, 1 << 20) == -1
    assert b"16-byte aligned" in _lib.lib.lbt_last_error()
    ws = _lib.lib.lbt_weighted_gradient_sums
    assert ws(None, _lib.LBT_OBJ_SQUARED_ERROR, one, two, None, 1.0, 10, 1, C.c_void_p(1024), C.c_void_p(2048),
              C.c_void_p(1024 + 16)) == -1
    assert b"alias" in _lib.lib.lbt_last_error()
    with pytest.raises(_lib.LbtError):
        _lib.check(rc)
    # the stages of a level
    hw = _lib.lib.lbt_histogram_level_workspace_bytes
    assert 0 < hw(1000, 4, 16, _lib.LBT_F32, 0) < hw(1000, 4, 16, _lib.LBT_F32, 12)
    assert hw(1000, 4, 4096, _lib.LBT_F32, 0) == 0 and hw(0, 4, 16, _lib.LBT_F32, 0) == 0
    hl = _lib.lib.lbt_histogram_level
    assert hl(None, one, _lib.LBT_F32, 10, 2, one, 1, one, one, 16, one, 1, 0, 1, one, 0, 3, one, one, 1 << 20, 0) == -1
    assert b"not a batch of level" in _lib.lib.lbt_last_error()
    assert hl(None, one, _lib.LBT_F32, 10, 2, one, 1, one, one, 16, one, 1, 1, 3, one, 2, 3, one, one, 1 << 20, 0) == -1
    assert b"does not hold the batch" in _lib.lib.lbt_last_error()
    assert hl(None, one, _lib.LBT_F32, 10, 2, one, 1, one, one, 16, one, 0, 0, 1, one, 0, 1, one, one, 8, 0) == -3
    assert _lib.lib.lbt_scan(None, one, 0, 3, 1, 2, one, 32, one, 1, 4) == -1
    assert _lib.lib.lbt_scan(None, None, 0, 3, 1, 2, one, 32, one, 1, 3) == -1
    assert _lib.lib.lbt_best_split_workspace_bytes(2, 32, 1, 3) > 0
    assert _lib.lib.lbt_best_split_workspace_bytes(2, 1, 1, 3) == 0
    bs = _lib.lib.lbt_best_split
    assert bs(None, one, 0, 3, 1, 2, one, _lib.LBT_F32, one, 32, None, one, one, 0.0, 1.0, 0.0, 1, 3, one, one, one, one,
              one, 8) == -3
    assert bs(None, one, 0, 3, 1, 2, one, 9, one, 32, None, one, one, 0.0, 1.0, 0.0, 1, 3, one, one, one, one, one,
              1 << 20) == -1
    assert _lib.lib.lbt_update_positions_workspace_bytes(1000, 3) > 0
    assert _lib.lib.lbt_update_positions_workspace_bytes(1000, 30) == 0
    assert _lib.lib.lbt_update_positions(None, one, _lib.LBT_F32, 10, 2, None, one, one, 0, one, 1 << 20) == -1
    assert _lib.lib.lbt_update_positions(None, one, _lib.LBT_F32, 10, 2, one, one, one, 0, one, 8) == -3


def test_tree_constructor_mirrors_reference_checks():
    from lbtree.models import Tree

    with pytest.raises(ValueError, match="split_samples must be <= 2048"):
        Tree(split_samples=4096)
    with pytest.warns(FutureWarning):
        t = Tree(alpha=3.0)
    assert t.l2_regularization == 3.0
    t = Tree()
    assert (t.max_depth, t.split_samples, t.feature_fraction, t.l1_regularization, t.l2_regularization,
            t.min_split_gain) == (8, 256, 1.0, 0.0, 1.0, 0.0)
