"""The four stages of a tree level through their own entry points (lbt_histogram_level, lbt_scan,
lbt_best_split, lbt_update_positions), each compared bit for bit with its oracle twin on the
reference's layouts, level after level, and the tree they produce with lbt_build_tree's."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(n, f, k, dtype, seed):
    rs = np.random.RandomState(seed)
    X = rs.normal(size=(n, f)).astype(dtype)
    X[:, 0] = rs.randint(0, 5, n)  # few distinct values: duplicate proposals collapse
    y = np.sin(X[:, 1]) + (X[:, 0] > 2) + 0.1 * rs.normal(size=n)
    g = np.stack([(0.3 * j - y) * 0.1 for j in range(k)], axis=1) + 0.01 * rs.normal(size=(n, k))
    h = np.abs(rs.normal(size=(n, k))) + 0.5
    return X, g, h


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("n,f,k,depth,s,dtype,cache_nodes", [
    (30000, 9, 1, 5, 64, np.float32, None),
    (20000, 20, 3, 4, 256, np.float32, None),
    (12000, 7, 2, 5, 300, np.float64, None),     # two-byte bins
    (25000, 12, 1, 5, 32, np.float32, 16),        # room for 16 nodes: levels 0..3 share a buffer, level 4 gets its own
])
def test_a_tree_stage_by_stage(n, f, k, depth, s, dtype, cache_nodes):
    import oracle_lib as orc
    from lbtree import ops

    seed = 11
    X, g, h = _inputs(n, f, k, dtype, seed)
    max_nodes = 2 ** (depth + 1) - 1
    Xd = _dev(X)
    # proposals and quantised gradients from the stage calls that exist already (checked elsewhere)
    props_d, rp_d = ops.select_split_samples(Xd, s, seed)
    q_d, root_d, scales_d = ops.quantise_gradients(_dev(g), _dev(h), seed)
    props = props_d.cpu().numpy()
    rp = rp_d.cpu().numpy()
    B = int(rp[-1])
    q = q_d.cpu().numpy().astype(np.int64)
    scales = scales_d.cpu().numpy()
    # both sides keep their own state
    c_sums = np.zeros((max_nodes, k, 2), np.int64)
    c_sums[0] = root_d.cpu().numpy()
    c_leaf = np.zeros((max_nodes, k))
    c_feature = -np.ones(max_nodes, np.int32)
    c_split = np.zeros(max_nodes)
    c_gain = np.zeros(max_nodes)
    c_pos = np.stack([np.zeros(n, np.int32), np.arange(n, dtype=np.int32)], axis=1).copy()
    g_sums, g_leaf, g_feature, g_split, g_gain, g_pos = (_dev(a) for a in (c_sums, c_leaf, c_feature, c_split, c_gain, c_pos))
    # one histogram buffer for the cached levels, a fresh one per level beyond them (GetHistogram,
    # build_tree.cu:1191-1205)
    hist_nodes = (0, 2 ** depth - 1)
    if cache_nodes is not None:
        # TreeBuilder's constructor, build_tree.cu:1004-1011
        cdepth = 0
        while 2 ** (cdepth + 2) - 1 <= cache_nodes and cdepth <= depth:
            cdepth += 1
        hist_nodes = (0, 2 ** (cdepth + 1) - 1)
        assert hist_nodes == (0, 15)
    c_hist = np.zeros((hist_nodes[1] - hist_nodes[0], k, B, 2), np.int64)
    g_hist = _dev(c_hist)
    ws = None
    for level in range(depth):
        batch = (2 ** level - 1, 2 ** (level + 1) - 1)
        if not (batch[0] >= hist_nodes[0] and batch[1] <= hist_nodes[1]):
            hist_nodes = batch
            c_hist = np.zeros((batch[1] - batch[0], k, B, 2), np.int64)
            g_hist = _dev(c_hist)
        ws = ops.histogram_level(Xd, q_d, props_d, rp_d, s, g_pos, level, batch, g_sums, hist_nodes, g_hist,
                                 workspace=ws, reuse_bins=level > 0 and level % 2 == 0, deepest_level=depth - 1)
        orc.histogram_level(X, q, props, rp, c_pos, batch, c_sums, hist_nodes, c_hist)
        assert np.array_equal(g_hist.cpu().numpy(), c_hist), ("histogram", level)
        ops.scan(g_hist, hist_nodes, rp_d, B, g_sums, batch)
        orc.scan(c_hist, hist_nodes, rp, c_sums, batch)
        assert np.array_equal(g_hist.cpu().numpy(), c_hist), ("scan", level)
        ops.best_split(g_hist, hist_nodes, props_d, rp_d, B, g_sums, scales_d, batch, g_leaf, g_feature, g_split, g_gain)
        orc.best_split(c_hist, hist_nodes, props, rp, c_sums, scales, batch, c_leaf, c_feature, c_split, c_gain)
        assert np.array_equal(g_feature.cpu().numpy(), c_feature), ("feature", level)
        assert np.array_equal(g_split.cpu().numpy(), c_split), ("split", level)
        assert np.array_equal(g_gain.cpu().numpy(), c_gain), ("gain", level)
        assert np.array_equal(g_sums.cpu().numpy(), c_sums), ("node_sums", level)
        assert np.array_equal(g_leaf.cpu().numpy(), c_leaf), ("leaf", level)
        if level < depth - 1:
            ops.update_positions(Xd, g_pos, g_feature, g_split, level)
            orc.update_positions(X, c_pos, c_feature, c_split, max_nodes)
            assert np.array_equal(g_pos.cpu().numpy(), c_pos), ("positions", level)
    assert (c_feature != -1).sum() >= 2 ** (depth - 1)
    # the same tree as the whole task gives (root leaf aside, which InitialiseRoot writes)
    cache = 0 if cache_nodes is None else cache_nodes * k * B * 16
    r = ops.build_tree(Xd, _dev(g), _dev(h), max_depth=depth, split_samples=s, seed=seed, taps=True,
                       hist_cache_bytes=cache)
    assert np.array_equal(r.feature.cpu().numpy(), c_feature)
    assert np.array_equal(r.split_value.cpu().numpy(), c_split)
    assert np.array_equal(r.gain.cpu().numpy(), c_gain)
    assert np.array_equal(r.node_sums.cpu().numpy(), c_sums)
    assert np.array_equal(r.leaf_value.cpu().numpy()[1:], c_leaf[1:])
    assert np.array_equal(r.positions.cpu().numpy(), c_pos)
    if cache_nodes is not None:
        assert (r.hist_node_begin, r.hist_node_end) == hist_nodes == (15, 31)


def test_stage_calls_reject_what_they_cannot_take():
    from lbtree import _lib, ops

    X, g, h = _inputs(3000, 4, 1, np.float32, 3)
    Xd = _dev(X)
    props_d, rp_d = ops.select_split_samples(Xd, 16, 1)
    q_d, root_d, _ = ops.quantise_gradients(_dev(g), _dev(h), 1)
    B = int(rp_d[-1])
    sums = torch.zeros((7, 1, 2), dtype=torch.int64, device="cuda")
    hist = torch.zeros((3, 1, B, 2), dtype=torch.int64, device="cuda")
    pos = torch.stack([torch.zeros(3000, dtype=torch.int32), torch.arange(3000, dtype=torch.int32)], dim=1).cuda()
    with pytest.raises(_lib.LbtError, match="not a batch of level"):
        ops.histogram_level(Xd, q_d, props_d, rp_d, 16, pos, 1, (0, 1), sums, (0, 3), hist)
    with pytest.raises(_lib.LbtError, match="does not hold the batch"):
        ops.histogram_level(Xd, q_d, props_d, rp_d, 16, pos, 0, (0, 1), sums, (1, 3), hist)
    with pytest.raises(_lib.LbtError, match="sorted by node"):
        ops.histogram_level(Xd, q_d, props_d, rp_d, 16, pos, 1, (1, 3), sums, (0, 3), hist)  # pairs of level 0
    with pytest.raises(_lib.LbtError, match="proposals"):
        ops.histogram_level(Xd, q_d, props_d, rp_d, 2, pos, 0, (0, 1), sums, (0, 3), hist)  # more than split_samples
