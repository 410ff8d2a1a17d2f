"""Benchmark configurations 3, 4 and 5 at their own shape (features, outputs, depth, split samples).

Each training configuration is checked twice: the first rows of its matrix bit-exact against the
CPU oracle, level by level, at a size the single-threaded oracle finishes in seconds; and the
whole matrix through identities that hold at any size (exact integer sums, a direct count of
histograms, the stable order of the row positions, the row->leaf map against PredictTask,
bit-identical repeats). Configuration 3 crosses the histogram re-allocation of
build_tree.cu:1191-1205 at level 7 (152 nodes of 8 x 51200 bins fit the 1e9-byte cache),
configuration 4 at level 11 (2048-node batches), where no parent histogram exists and both
children are built."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

LR = 0.1


def _softmax_gradients(y, n_classes):
    """Round-0 gradients of LBClassifier: raw predictions start at log(class frequency)
    (objectives.py:489-531), then LBBase._get_weighted_gradient (legateboost.py:189-224)."""
    from lbtree import ops

    prob = torch.bincount(y.to(torch.int64), minlength=n_classes).to(torch.float64) / y.numel()
    pred = torch.log(prob).reshape(1, -1).repeat(y.shape[0], 1).contiguous()
    return ops.weighted_gradient("log_loss", y, pred, None, LR)


def _squared_error_gradients(y):
    pred = torch.full((y.shape[0], 1), float(y.mean()), dtype=torch.float64, device=y.device)
    return (pred - y.reshape(-1, 1)) * LR, torch.ones_like(pred)


@pytest.fixture(scope="module")
def config3():
    from lbtree import datasets

    X, y = datasets.config3()
    assert X.shape == (2_000_000, 200)
    g, h = _softmax_gradients(y, 8)
    return X, g, h


@pytest.fixture(scope="module")
def config4():
    from lbtree import datasets

    X, y = datasets.config4()
    assert X.shape == (1_000_000, 50)
    g, h = _squared_error_gradients(y)
    return X, g, h


def _subsample_parity(X, g, h, rows, **kw):
    import gpu_util as gu

    Xs = X[:rows].cpu().numpy()
    gs = g[:rows].cpu().numpy()
    hs = h[:rows].cpu().numpy()
    gr, cr = gu.both(Xs, gs, hs, levels=True, **kw)
    gu.assert_tree_parity(gr, cr, levels=True)
    return gr, cr


def test_config2_first_rows_bit_exact():
    """The headline shape: 100 features (two feature groups of 52 and 48 whose records carry the
    gradient pair), one output, depth 8, 256 split samples, on the first 200,000 rows of the
    10,000,000 x 100 matrix, level by level against the oracle."""
    from lbtree import datasets

    X, y = datasets.config2(10_000_000, 100)
    assert X.shape == (10_000_000, 100)
    g, h = _squared_error_gradients(y)
    gr, cr = _subsample_parity(X, g, h, 200_000, max_depth=8, split_samples=256, seed=24680)
    assert (cr.hist_node_begin, cr.hist_node_end) == (0, 1023)  # 2441 nodes of 25,600 bins fit the cache
    assert np.diff(cr.row_pointers).max() == 256
    assert (cr.feature != -1).sum() > 200
    # siblings are derived by subtraction from level 1 on
    for d in range(1, 8):
        assert cr.level_built_instances[d] < (cr.positions_per_level[d][:, 0] >= 0).sum()


def test_config3_first_rows_bit_exact(config3):
    """200 features, 8 softmax outputs, depth 8, 256 split samples; the oracle takes about 20 s."""
    X, g, h = config3
    gr, cr = _subsample_parity(X, g, h, 150_000, max_depth=8, split_samples=256, seed=1234567)
    # level 7 works on a re-allocated buffer: every node with rows is built, none by subtraction
    assert (cr.hist_node_begin, cr.hist_node_end) == (127, 255)
    assert cr.level_built_instances[7] == (cr.positions_per_level[7][:, 0] >= 0).sum()
    assert cr.level_built_instances[6] < (cr.positions_per_level[6][:, 0] >= 0).sum()
    assert (cr.feature != -1).sum() > 150


def test_config4_first_rows_bit_exact(config4):
    """50 features (15 of them with 16 levels), one output, depth 12, 512 split samples."""
    X, g, h = config4
    gr, cr = _subsample_parity(X, g, h, 200_000, max_depth=12, split_samples=512, seed=7654321)
    assert (cr.hist_node_begin, cr.hist_node_end) == (2047, 4095)
    assert cr.level_built_instances[11] == (cr.positions_per_level[11][:, 0] >= 0).sum()
    assert cr.level_built_instances[10] < (cr.positions_per_level[10][:, 0] >= 0).sum()
    rp = cr.row_pointers
    assert (np.diff(rp)[:15] <= 16).all() and np.diff(rp).max() > 256  # duplicates collapse; two-byte bins
    assert (cr.feature != -1).sum() > 300


def _direct_histogram_check(X, r, node, features, outputs):
    """Scanned histogram of `node` (which must be in the buffer) against a direct count over its rows."""
    rp = r.row_pointers.cpu().numpy()
    pos = r.positions_of_level.to(torch.int64)
    rows = pos[pos[:, 0] == node, 1]
    assert rows.numel() > 0
    for f in features:
        p = r.proposals[rp[f]: rp[f + 1]]
        bins = torch.searchsorted(p, X[rows, f].contiguous(), right=False)  # first proposal >= x
        n = int(rp[f + 1] - rp[f])
        assert int(bins.max()) < n
        for k in outputs:
            q = r.quantised[rows, k, :].to(torch.int64)
            want = torch.cumsum(torch.zeros((n, 2), dtype=torch.int64, device=X.device).index_add_(0, bins, q), 0)
            got = r.histogram[node - r.hist_node_begin, k, rp[f]: rp[f + 1], :]
            # the scan leaves the raw bin where neither running sum is positive (build_tree.cu:645)
            keep = (want[:, 0] > 0) | (want[:, 1] > 0)
            assert int(keep.sum()) > 0
            assert torch.equal(got[keep], want[keep]), (node, f, k)


def _full_size_properties(X, g, h, depth, s, seed, features):
    from lbtree import ops

    n, k = X.shape[0], g.shape[1]
    r = ops.build_tree(X, g, h, max_depth=depth, split_samples=s, seed=seed, taps=True, taps_levels=True,
                       row_leaf=True)
    torch.cuda.synchronize()
    feature = r.feature.cpu().numpy()
    sums = r.node_sums.cpu().numpy()
    split = np.flatnonzero(feature >= 0)
    # children add up to their parent, the root to the quantised gradients (exact integers)
    assert np.array_equal(sums[2 * split + 1] + sums[2 * split + 2], sums[split])
    assert np.array_equal(r.quantised.to(torch.int64).sum(dim=0).cpu().numpy(), sums[0])
    # every scanned feature of a node in the buffer ends in the node's sums
    rp = r.row_pointers.cpu().numpy()
    last = torch.as_tensor(rp[1:] - 1, device=X.device, dtype=torch.long)
    node_sums = r.node_sums[r.hist_node_begin: r.hist_node_end]
    for kk in range(k):
        ends = r.histogram[:, kk, last, :]
        reached = node_sums[:, kk, 1] > 0
        assert torch.equal(ends[reached], node_sums[reached, kk].unsqueeze(1).expand(-1, len(rp) - 1, -1)), kk
    # a direct count of two nodes of the deepest level (built without a parent histogram here)
    r.positions_of_level = r.positions_per_level[depth - 1]
    level_first = 2 ** (depth - 1) - 1
    counts = torch.bincount(r.positions_of_level[:, 0].to(torch.int64) + 1, minlength=2 ** depth + 1)[1:]
    held = torch.nonzero(counts[level_first:] > 0).reshape(-1)
    assert held.numel() >= 2
    for j in (int(held[0]), int(held[-1])):
        _direct_histogram_check(X, r, level_first + j, features, sorted({0, k - 1}))
    # positions: a permutation, nodes ascending (-1 first), rows ascending inside a node; the
    # retired rows keep the order in which they retired (the sort of build_tree.cu:1050-1073 is
    # stable): what was retired at one level is the head of the next level's order, unchanged,
    # followed by the rows that retire now
    pos = r.positions.to(torch.int64)
    assert torch.equal(pos, r.positions_per_level[depth - 1].to(torch.int64))
    assert torch.equal(torch.sort(pos[:, 1]).values, torch.arange(n, device=X.device))
    retired_before = 0
    for d in range(depth):
        lv = r.positions_per_level[d].to(torch.int64)
        node, row = lv[:, 0], lv[:, 1]
        assert bool((node[1:] >= node[:-1]).all()), d
        retired = int((node < 0).sum())
        live = node[retired:] * (1 << 32) + row[retired:]
        assert bool((live[1:] > live[:-1]).all()), d
        assert int(node[retired:].min()) >= 2 ** d - 1 and int(node.max()) < 2 ** (d + 1) - 1
        if d > 0:
            prev = r.positions_per_level[d - 1][:, 1]
            assert retired >= retired_before
            assert torch.equal(lv[:retired_before, 1], prev[:retired_before].to(torch.int64)), d
            # the rows that retire now stand in the order they had at the level before
            where = torch.empty(n, dtype=torch.int64, device=X.device)
            where[prev.to(torch.int64)] = torch.arange(n, device=X.device)
            fresh = where[row[retired_before:retired]]
            assert bool((fresh[1:] > fresh[:-1]).all()), d
        retired_before = retired
    # the row -> leaf map against PredictTask, tiled and per node
    tree = (r.leaf_value, r.feature, r.split_value)
    want = ops.predict(X, [tree], k)
    assert torch.equal(r.leaf_value[r.row_leaf.long()], want)
    assert torch.equal(ops.predict(X, [tree], k, tiled=False), want)
    # a second build gives the same bits
    r2 = ops.build_tree(X, g, h, max_depth=depth, split_samples=s, seed=seed)
    for name in ("feature", "split_value", "gain", "leaf_value", "hessian"):
        assert torch.equal(getattr(r, name), getattr(r2, name)), name
    return r


def test_config3_full_size_properties(config3):
    X, g, h = config3
    r = _full_size_properties(X, g, h, 8, 256, 99, (0, 101, 199))
    assert (r.hist_node_begin, r.hist_node_end) == (127, 255)
    assert int((r.feature >= 0).sum()) > 150


def test_config4_full_size_properties(config4):
    X, g, h = config4
    r = _full_size_properties(X, g, h, 12, 512, 77, (0, 14, 15, 49))
    assert (r.hist_node_begin, r.hist_node_end) == (2047, 4095)
    assert int((r.feature >= 0).sum()) > 500


def test_config5_all_trees_all_rows():
    """1000 complete depth-8 trees over 64 features, 20,000,000 rows: the tiled traversal equals the
    per-node one on every row, and the oracle on a sample of rows from both ends."""
    import oracle_lib as orc
    from lbtree import datasets, ops

    trees = datasets.config5_ensemble()
    assert len(trees) == 1000
    X = datasets.config5_X()
    assert X.shape == (20_000_000, 64)
    tiled = ops.predict(X, trees, 1)
    plain = ops.predict(X, trees, 1, tiled=False)
    assert torch.equal(tiled, plain)
    del plain
    ens = ops.PackedEnsemble(trees, 1, 64)
    assert torch.equal(ens.predict(X), tiled)
    th = [(a.cpu().numpy(), b.cpu().numpy(), c.cpu().numpy()) for a, b, c in trees]
    for lo, hi in ((0, 1500), (X.shape[0] - 1500, X.shape[0])):
        want = orc.predict(X[lo:hi].cpu().numpy(), th, 1)
        assert np.array_equal(tiled[lo:hi].cpu().numpy(), want)
        assert np.abs(tiled[lo:hi].cpu().numpy() - want).max() <= 1e-5  # the task's stated tolerance
