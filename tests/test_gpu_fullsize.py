"""The headline workload at full size (10,000,000 x 100 f32, depth 8, 256 split samples), where the
single-threaded oracle would take hours: the build is checked through properties that do not depend
on the size -- exact integer identities of the histograms and node sums, the order of the row
positions, agreement of the row->leaf map with PredictTask, and bit-identical repeats."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def built():
    from lbtree import datasets, ops

    X, y = datasets.config2(10_000_000, 100)
    pred = torch.full((X.shape[0], 1), float(y.mean()), dtype=torch.float64, device=X.device)
    g = (pred - y.reshape(-1, 1)) * 0.1
    h = torch.ones_like(pred)
    r = ops.build_tree(X, g, h, max_depth=8, split_samples=256, seed=2024, taps=True, row_leaf=True)
    torch.cuda.synchronize()
    return X, g, h, r


def test_children_sums_add_up_to_their_parent(built):
    _, _, _, r = built
    feature = r.feature.cpu().numpy()
    sums = r.node_sums.cpu().numpy()  # [nodes][k][2] int64
    split = np.flatnonzero(feature >= 0)
    assert len(split) > 100
    assert np.array_equal(sums[2 * split + 1] + sums[2 * split + 2], sums[split])
    q = r.quantised.to(torch.int64).sum(dim=0).cpu().numpy()
    assert np.array_equal(q, sums[0])


def test_root_histogram_equals_a_direct_count(built):
    X, _, _, r = built
    rp = r.row_pointers.cpu().numpy()
    assert r.hist_node_begin == 0
    q = r.quantised[:, 0, :].to(torch.int64)
    for f in (0, 57, 99):
        p = r.proposals[rp[f]: rp[f + 1]]
        bins = torch.searchsorted(p, X[:, f].contiguous(), right=False)  # first proposal >= x
        n = int(rp[f + 1] - rp[f])
        assert int(bins.max()) < n
        for c in range(2):
            direct = torch.zeros(n, dtype=torch.int64, device=X.device).index_add_(0, bins, q[:, c])
            # the buffer holds the scanned histogram
            assert torch.equal(torch.cumsum(direct, 0), r.histogram[0, 0, rp[f]: rp[f + 1], c])


def test_every_scanned_feature_ends_in_the_node_sum(built):
    _, _, _, r = built
    rp = r.row_pointers.cpu().numpy()
    last = torch.as_tensor(rp[1:] - 1, device=r.histogram.device, dtype=torch.long)
    ends = r.histogram[:, 0, last, :]  # [nodes in buffer][features][2]
    sums = r.node_sums[r.hist_node_begin: r.hist_node_end, 0, :]
    reached = sums[:, 1] > 0
    assert int(reached.sum()) > 100
    assert torch.equal(ends[reached], sums[reached].unsqueeze(1).expand(-1, len(rp) - 1, -1))


def _best_split_on_the_host(hist, sums, rp, scales):
    """perform_best_split (build_tree.cu:682-782) of one node from its scanned histogram
    [bins][2] and its sums [2], one output, no feature set, l1 = 0, l2 = 1, min_split_gain = 0:
    the gain of every bin with the oracle's scalar, zero where a child has no hessian, then the
    arg-max under the reference's order (strictly greater gain wins inside each of its 512 strided
    threads, so the lowest bin of a residue class; the rank-ordered reduce keeps the later class on
    ties, so the highest residue). Returns (bin, gain) or (-1, 0.0)."""
    import oracle_lib as orc

    lib = orc._load()
    ng, nh = int(sums[0]), int(sums[1])
    gains = np.zeros(len(hist))
    for b in range(len(hist)):
        lg, lh = int(hist[b, 0]), int(hist[b, 1])
        rg, rh = ng - lg, nh - lh
        if lh <= 0 or rh <= 0:
            continue
        gains[b] = lib.orc_calculate_gain(lg * scales[2], lh * scales[3], rg * scales[2], rh * scales[3],
                                          ng * scales[2], nh * scales[3], 0.0, 1.0, 0.0)
    top = gains.max()
    if not top > 1e-5:
        return -1, 0.0
    tied = np.flatnonzero(gains == top)
    residue = (tied % 512).max()
    return int(tied[tied % 512 == residue].min()), float(top)


def test_split_decisions_follow_from_the_histograms(built):
    """Root and two nodes of each deeper level: feature, threshold and gain recomputed on the
    host from the node's scanned histogram (itself checked against a direct count above)."""
    _, _, _, r = built
    rp = r.row_pointers.cpu().numpy()
    feature = r.feature.cpu().numpy()
    split = r.split_value.cpu().numpy()
    gain = r.gain.cpu().numpy()
    sums = r.node_sums.cpu().numpy()
    proposals = r.proposals.cpu().numpy()
    assert r.hist_node_begin == 0
    checked = 0
    for d in range(8):
        first = 2 ** d - 1
        level = [n for n in range(first, 2 * first + 1) if sums[n, 0, 1] > 0]
        for node in sorted({level[0], level[len(level) // 2], level[-1]}):
            hist = r.histogram[node, 0].cpu().numpy()
            b, top = _best_split_on_the_host(hist, sums[node, 0], rp, r.scales)
            if b < 0:
                assert feature[node] == -1
                continue
            f = int(np.searchsorted(rp, b, side="right") - 1)
            assert feature[node] == f, (node, feature[node], f)
            assert split[node] == float(proposals[b]), node
            assert gain[node] == top, node
            # the children's sums are the chosen bin and what is left of the node
            assert np.array_equal(sums[2 * node + 1, 0], hist[b])
            assert np.array_equal(sums[2 * node + 2, 0], sums[node, 0] - hist[b])
            checked += 1
    assert checked >= 15


def test_positions_are_a_stable_partition(built):
    X, _, _, r = built
    pos = r.positions.to(torch.int64)
    node, row = pos[:, 0], pos[:, 1]
    assert torch.equal(torch.sort(row).values, torch.arange(X.shape[0], device=X.device))
    key = node * (1 << 32) + row  # nodes ascending (-1 first), rows ascending inside a node
    assert bool((key[1:] > key[:-1]).all())


def test_row_leaf_is_what_predict_returns(built):
    from lbtree import ops

    X, _, _, r = built
    want = ops.predict(X, [(r.leaf_value, r.feature, r.split_value)], 1)
    assert torch.equal(r.leaf_value[r.row_leaf.long()], want)
    plain = ops.predict(X, [(r.leaf_value, r.feature, r.split_value)], 1, tiled=False)
    assert torch.equal(plain, want)


def test_a_second_build_is_bit_identical(built):
    from lbtree import ops

    X, g, h, r = built
    r2 = ops.build_tree(X, g, h, max_depth=8, split_samples=256, seed=2024)
    for name in ("feature", "split_value", "gain", "leaf_value", "hessian"):
        assert torch.equal(getattr(r, name), getattr(r2, name)), name


def test_ensemble_prediction_tiled_equals_per_node_and_oracle_on_a_sample():
    """The prediction-only workload (complete depth-8 trees over 64 features), 200 trees on 2M rows."""
    import oracle_lib as orc
    from lbtree import datasets, ops

    trees = datasets.config5_ensemble()[:200]
    X = datasets.config5_X(2_000_000)
    tiled = ops.predict(X, trees, 1)
    plain = ops.predict(X, trees, 1, tiled=False)
    assert torch.equal(tiled, plain)
    ns = 3000
    th = [(a.cpu().numpy(), b.cpu().numpy(), c.cpu().numpy()) for a, b, c in trees]
    want = orc.predict(X[:ns].cpu().numpy(), th, 1)
    assert np.array_equal(tiled[:ns].cpu().numpy(), want)
