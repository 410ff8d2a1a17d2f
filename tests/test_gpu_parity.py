"""GPU parity: liblbtree.so (through the C ABI) against the CPU oracle on the
same seeded inputs. Integer results (quantised gradients, histograms, node
sums, splits, positions) must be bit-exact; leaf values are additionally
checked against the 1e-6 relative tolerance, predictions against 1e-5 absolute."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _problem(seed, n, f, k, dtype=np.float32, lowcard=True):
    rs = np.random.RandomState(seed)
    X = rs.randn(n, f).astype(dtype)
    if lowcard and f > 2:
        X[:, 1] = rs.randint(0, 4, n)
        X[:, 2] = 0.25
    g = rs.randn(n, k)
    h = rs.rand(n, k) + 0.1
    return X, g, h


@pytest.mark.parametrize("n,f,k,depth,s,dtype", [
    (1000, 4, 1, 3, 16, np.float32),
    (5000, 10, 1, 5, 64, np.float32),
    (5000, 10, 3, 4, 64, np.float64),
    (20000, 33, 2, 6, 256, np.float32),
    (3000, 7, 1, 8, 2048, np.float32),
    (2, 1, 1, 1, 256, np.float64),
    (1, 3, 2, 2, 8, np.float32),
    (700, 300, 1, 3, 5, np.float32),
    (4000, 150, 1, 4, 256, np.float32),   # several feature groups, two features per lane
    (6000, 64, 1, 5, 256, np.float32),    # one group, gradients embedded in the bin records
    (2500, 18, 1, 4, 300, np.float64),    # two-byte bins with double features
    (4000, 5, 1, 4, 64, np.float32),      # feature counts that are no multiple of a lane's four: the
    (4000, 6, 1, 4, 64, np.float32),      # last lane of a row owns 1, 2 or 3 features
    (4000, 103, 2, 4, 256, np.float32),
    (3000, 9, 1, 4, 64, np.float64),      # ... or of a lane's two doubles
    (3000, 11, 1, 3, 400, np.float32),    # ... with two-byte bins
    (2000, 200, 8, 3, 256, np.float32),   # 3 groups x 8 outputs would leave CUs idle: a fourth group is taken
    (2000, 300, 5, 3, 256, np.float32),
    (20000, 100, 1, 9, 64, np.float32),   # four lanes per 64-byte record in two groups (52 + 48 features), down to
    (3000, 52, 1, 6, 32, np.float32),     # nodes of a few rows, whose sums go to the histogram directly
])
def test_build_tree_bit_exact(n, f, k, depth, s, dtype):
    import gpu_util as gu

    X, g, h = _problem(n * 7 + f, n, f, k, dtype)
    gr, cr = gu.both(X, g, h, levels=True, max_depth=depth, split_samples=s, seed=12345)
    gu.assert_tree_parity(gr, cr, levels=True)


def test_depth_zero_and_regularisation_variants():
    import gpu_util as gu

    X, g, h = _problem(5, 4000, 6, 2)
    for kw in [dict(max_depth=0, split_samples=16, seed=1),
               dict(max_depth=4, split_samples=32, seed=2, l1_regularization=0.7, l2_regularization=0.0),
               dict(max_depth=4, split_samples=32, seed=3, l2_regularization=5.0, min_split_gain=0.05),
               dict(max_depth=5, split_samples=32, seed=2**31 - 1)]:
        gr, cr = gu.both(X, g, h, **kw)
        gu.assert_tree_parity(gr, cr)


@pytest.mark.parametrize("n,f,k,depth,s", [(30000, 20, 1, 6, 256), (20000, 70, 2, 5, 64), (9000, 6, 3, 4, 300)])
def test_negative_hessians_bit_exact(n, f, k, depth, s):
    """A custom objective may hand over negative hessians; the reference rounds and sums them as
    int64 like any other value (build_tree.cu:112-129). Embedded and gathered gradient pairs,
    one- and two-byte bins."""
    import gpu_util as gu

    X, g, h = _problem(n + k, n, f, k)
    rs = np.random.RandomState(n)
    h = np.where(rs.rand(n, k) < 0.15, -h, h)
    h[:5] = -3.0
    gr, cr = gu.both(X, g, h, levels=True, max_depth=depth, split_samples=s, seed=99)
    gu.assert_tree_parity(gr, cr, levels=True)
    assert (cr.quantised[:, :, 1] < 0).any() and (cr.feature != -1).sum() > 5
    # all hessians negative: the root's sum is not positive, nothing splits (build_tree.cu:712)
    gr, cr = gu.both(X, g, -np.abs(h), max_depth=3, split_samples=s, seed=5)
    gu.assert_tree_parity(gr, cr)
    assert (cr.feature == -1).all()


@pytest.mark.parametrize("wait", [True, False])
def test_error_raised_inside_a_build_reaches_the_caller(wait):
    """One entry holds the whole absolute gradient sum and the stochastic rounding takes it up to
    2^31 (seed, row and value chosen for that: the oracle confirms the value), which the packed
    32-bit pairs cannot hold. The library notices after the first level is queued: the call must
    return the status, the synchronising form with the stream drained, and later calls work."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import _lib, ops

    n, seed, row = 4096, 308, 1068
    g = np.zeros((n, 1))
    g[row, 0] = 4.236547993389047
    h = np.zeros((n, 1))
    h[0, 0] = 1.0
    q = orc.quantise_all(g, h, seed, orc.scales(orc.abs_sums(g, h)))
    assert q[row, 0, 0] == 2 ** 31
    X, _, _ = _problem(3, n, 7, 1)
    with pytest.raises(_lib.LbtError, match="2\\^31"):
        ops.build_tree(X, g, h, max_depth=4, split_samples=32, seed=seed, wait=wait)
    if wait:
        assert torch.cuda.current_stream().query()  # nothing of the failed call is still queued
    torch.cuda.synchronize()
    # the same thread and workspace serve the next call, also after the thread's pinned buffers
    # and events have been released
    X2, g2, h2 = _problem(4, n, 7, 1)
    for _ in range(2):
        gr, cr = gu.both(X2, g2, h2, max_depth=4, split_samples=32, seed=seed)
        gu.assert_tree_parity(gr, cr)
        assert _lib.lib.lbt_release_thread_resources() == 0


def test_feature_set():
    import gpu_util as gu

    X, g, h = _problem(6, 3000, 8, 1)
    fs = np.array([0, 1, 0, 0, 1, 0, 0, 1], bool)
    gr, cr = gu.both(X, g, h, max_depth=5, split_samples=32, seed=4, feature_set=fs)
    gu.assert_tree_parity(gr, cr)
    used = set(gu.cpu(gr.feature)[gu.cpu(gr.feature) >= 0].tolist())
    assert used and used <= {1, 4, 7}


def test_small_histogram_budget_batches():
    import gpu_util as gu

    X, g, h = _problem(8, 3000, 5, 2)
    ref = None
    for budget in [0, 40000, 6000, 1]:
        gr, cr = gu.both(X, g, h, max_depth=5, split_samples=16, seed=9, hist_cache_bytes=budget)
        gu.assert_tree_parity(gr, cr)
        if ref is None:
            ref = gu.cpu(gr.feature).copy()
        assert np.array_equal(gu.cpu(gr.feature), ref)


@pytest.mark.parametrize("k,depth,budget", [(1, 5, 0), (3, 4, 0), (2, 5, 6000), (1, 6, 40000), (4, 1, 0), (2, 3, 1)])
def test_tree_without_histogram_tap_matches_oracle(k, depth, budget):
    """A caller that does not ask for the histograms lets the last level (and a level before a new
    histogram buffer) keep its running sums to itself: the tree must be the one the oracle builds, with
    l1 regularisation, a minimum gain, outputs whose hessian sums vanish in some nodes and empty nodes."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    X, g, h = _problem(40 + k, 4000, 9, k)
    # a few rows carry all the hessian mass of the last output: its sums vanish in most nodes
    if k > 1:
        h[:, k - 1] = 0.0
        h[:40, k - 1] = 1.0
    kw = dict(max_depth=depth, split_samples=32, seed=77, l1_regularization=0.01, min_split_gain=1e-4,
              hist_cache_bytes=budget)
    cr = orc.build_tree(X, g, h, max_depth=depth, split_samples=32, seed=77, l1=0.01, l2=1.0, min_split_gain=1e-4,
                        hist_cache_bytes=budget)
    plain = ops.build_tree(X, g, h, row_leaf=True, **kw)
    tapped = ops.build_tree(X, g, h, taps=True, row_leaf=True, **kw)
    gu.assert_tree_parity(tapped, cr)
    for got in (plain, tapped):
        assert np.array_equal(gu.cpu(got.feature), cr.feature)
        gu.assert_same_floats(gu.cpu(got.split_value), cr.split_value, "split_value")
        gu.assert_same_floats(gu.cpu(got.gain), cr.gain, "gain")
        gu.assert_same_floats(gu.cpu(got.leaf_value), cr.leaf_value, "leaf_value")
        gu.assert_same_floats(gu.cpu(got.hessian), cr.hessian, "hessian")
    assert np.array_equal(gu.cpu(plain.row_leaf), gu.cpu(tapped.row_leaf))


def test_deep_tree_with_duplicates_and_small_nodes():
    import gpu_util as gu

    rs = np.random.RandomState(3)
    n, f = 6000, 12
    X = np.exp(rs.randn(n, f) * 1.5).astype(np.float32)
    X[:, :4] = rs.randint(0, 16, (n, 4))
    y = (X[:, 0] > 7).astype(float) + (X[:, 5] > 1.0) * 2.0 + rs.randn(n) * 0.2
    g = (0.0 - y).reshape(-1, 1)
    h = np.ones((n, 1))
    gr, cr = gu.both(X, g, h, levels=True, max_depth=12, split_samples=512, seed=77)
    gu.assert_tree_parity(gr, cr, levels=True)
    assert (cr.feature != -1).sum() > 100


def test_skewed_features_exercise_every_stage_of_the_bin_search():
    """Heavy tails crowd most proposals into a few lookup cells, so the search runs through its
    probe windows into the binary-search stage; a constant and a two-valued column sit beside them."""
    import gpu_util as gu

    rs = np.random.RandomState(11)
    n, f = 20000, 24
    X = np.exp(rs.randn(n, f) * 2.5).astype(np.float32)
    X[:, 3] = 1.5
    X[:, 4] = rs.randint(0, 2, n)
    X[:, 5] = -np.exp(rs.randn(n) * 3.0)
    X[::97, 6] = np.float32(3.0e38)
    g = rs.randn(n, 1)
    h = rs.rand(n, 1) + 0.5
    gr, cr = gu.both(X, g, h, levels=True, max_depth=6, split_samples=256, seed=31)
    gu.assert_tree_parity(gr, cr, levels=True)


def test_tie_rule_on_gpu():
    import gpu_util as gu

    n = 64
    Xp = np.arange(1, 601, dtype=np.float32).reshape(-1, 1)
    X = np.zeros((n, 1), np.float32)
    X[: n // 2, 0] = 470.0
    X[n // 2:, 0] = 600.0
    Xall = np.concatenate([Xp, X])
    g = np.zeros((len(Xall), 1))
    h = np.full((len(Xall), 1), 1e-300)
    g[600: 600 + n // 2] = -1.0
    g[600 + n // 2:] = 1.0
    h[600:] = 1.0
    gr, cr = gu.both(Xall, g, h, max_depth=1, split_samples=2048, seed=0)
    gu.assert_tree_parity(gr, cr)
    bin_idx = int(np.searchsorted(cr.proposals, np.float32(gu.cpu(gr.split_value)[0])))
    assert bin_idx == 511


def test_config1_boosting_rounds_match_oracle_round_by_round():
    """Benchmark configuration 1: 100000x32, squared error, depth 6, 10 rounds, lr 0.1.
    Each round's task inputs (X, g, h, seed) go to both implementations."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(0)
    n, f = 100000, 32
    X = rs.random_sample((n, f)).astype(np.float32)
    y = np.sin(2 * np.pi * X[:, :4].astype(np.float64)).sum(axis=1) + rs.normal(0, 0.1, n)
    Xd = ops.as_device(X)
    est_rs = np.random.RandomState(0)
    pred = np.full((n, 1), y.mean())
    losses = []
    for rnd in range(10):
        g = (pred - y.reshape(-1, 1)) * 0.1
        h = np.ones((n, 1))
        seed = int(est_rs.randint(0, 2**31))
        gr, cr = gu.both(Xd if False else X, g, h, max_depth=6, split_samples=256, seed=seed)
        gu.assert_tree_parity(gr, cr)
        p_gpu = gu.cpu(ops.predict(Xd, [(gr.leaf_value, gr.feature, gr.split_value)], 1))
        p_cpu = orc.predict(X, [(cr.leaf_value, cr.feature, cr.split_value)], 1)
        assert np.abs(p_gpu - p_cpu).max() <= 1e-5
        assert np.array_equal(p_gpu, p_cpu)
        pred = pred + p_cpu
        losses.append(((pred[:, 0] - y) ** 2).mean())
    assert all(b < a for a, b in zip(losses, losses[1:]))


def test_predict_matches_oracle_multi_tree_multi_output():
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(21)
    X = rs.randn(30000, 16).astype(np.float32)
    trees_c, trees_g = [], []
    for t in range(130):  # more than one launch batch
        m = 2 ** 5 - 1
        feat = -np.ones(m, np.int32)
        feat[: 2 ** 4 - 1] = rs.randint(0, 16, 2 ** 4 - 1)
        # some early leaves
        feat[rs.randint(1, 15, 2)] = -1
        split = rs.randn(m)
        leaf = rs.randn(m, 3) * 0.01
        trees_c.append((leaf, feat, split))
        trees_g.append((ops.as_device(leaf), ops.as_device(feat), ops.as_device(split)))
    want = orc.predict(X, trees_c, 3)
    got = gu.cpu(ops.predict(X, trees_g, 3))
    assert np.array_equal(got, want)
    X64 = X.astype(np.float64)
    got64 = gu.cpu(ops.predict(X64, trees_g[:3], 3))
    assert np.array_equal(got64, orc.predict(X64, trees_c[:3], 3))
    assert np.array_equal(gu.cpu(ops.predict(X, [], 3)), np.zeros((30000, 3)))


@pytest.mark.parametrize("f,k", [(13, 1), (100, 1), (200, 3), (330, 1), (40, 11), (13, 17)])
def test_predict_tiled_and_per_node_paths_agree_with_oracle(f, k):
    """Mixed tree sizes, feature counts that take 4, 8 or 16 lanes per row (one not a multiple of
    four), a row count that is not a multiple of the tile, thresholds that equal feature values or
    sit between two floats."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(5)
    n = 70001 if f < 100 else 9001
    X = rs.rand(n, f).astype(np.float32)
    trees_c, trees_g = [], []
    for t in range(47):
        depth = [3, 8, 5, 10][t % 4]
        m = 2 ** (depth + 1) - 1
        inner = 2 ** depth - 1
        feat = -np.ones(m, np.int32)
        feat[:inner] = rs.randint(0, f, inner)
        if t % 3 == 0:
            feat[rs.randint(1, inner, 3)] = -1
        split = rs.rand(m)
        # every third threshold is an actual (float) feature value, every fifth one lies just above one
        vals = X[rs.randint(0, n, m), np.maximum(feat, 0)].astype(np.float64)
        split[::3] = vals[::3]
        split[::5] = vals[::5] + 1e-12
        leaf = rs.randn(m, k) * 0.01
        trees_c.append((leaf, feat, split))
        trees_g.append((ops.as_device(leaf), ops.as_device(feat), ops.as_device(split)))
    want = orc.predict(X, trees_c, k)
    tiled = gu.cpu(ops.predict(X, trees_g, k))
    plain = gu.cpu(ops.predict(X, trees_g, k, tiled=False))
    assert np.array_equal(tiled, want)
    assert np.array_equal(plain, want)
    X64 = X.astype(np.float64) + 1e-13
    assert np.array_equal(gu.cpu(ops.predict(X64, trees_g, k)), orc.predict(X64, trees_c, k))


@pytest.mark.parametrize("f,k,dtype", [(13, 1, np.float32), (100, 3, np.float32), (330, 1, np.float32),
                                       (40, 2, np.float64), (24, 19, np.float32), (9, 9, np.float64)])
def test_packed_ensemble_predicts_like_the_oracle(f, k, dtype):
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import _lib, ops

    rs = np.random.RandomState(f + k)
    X = rs.normal(size=(4099, f)).astype(dtype)
    trees = []
    for t in range(37):
        depth = 1 + t % 6
        m = 2 ** (depth + 1) - 1
        feature = np.full(m, -1, np.int32)
        inner = 2 ** depth - 1
        feature[:inner] = rs.randint(0, f, inner)
        feature[rs.randint(1, max(inner, 2), 2)] = -1  # early leaves; their subtrees are unreachable
        split = rs.normal(size=m)
        split[:3] = X[:3, feature[0]]  # thresholds that equal feature values: <= goes left
        trees.append((rs.normal(size=(m, k)), feature, split))
    dev = [tuple(ops.as_device(a) for a in t) for t in trees]
    ens = ops.PackedEnsemble(dev, k, f, torch.float32 if dtype == np.float32 else torch.float64)
    want = orc.predict(X, trees, k)
    for rows in (X, X[:1], X[:777]):  # the same packed ensemble serves batch after batch
        got = gu.cpu(ens.predict(rows))
        assert np.array_equal(got, want[: rows.shape[0]])
    assert ens.predict(X[:0]).shape == (0, k)
    with pytest.raises(_lib.LbtError, match="does not match"):
        ens.predict(X[:, : f - 1])
    with pytest.raises(_lib.LbtError, match="does not match"):
        ens.predict(X.astype(np.float64 if dtype == np.float32 else np.float32))


def test_update_tree_matches_oracle_within_rounding():
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    X, g, h = _problem(31, 20000, 6, 2)
    gr, cr = gu.both(X, g, h, max_depth=5, split_samples=64, seed=8)
    leaf_c, hess_c = orc.update_tree(X, g, h, cr.feature, cr.split_value, 0.3, 1.0)
    leaf_g, hess_g = ops.update_tree(X, g, h, gr.feature, gr.split_value, 0.3, 1.0)
    # double sums in a different order: 1e-6 relative, as the task states for leaf values
    assert np.allclose(gu.cpu(leaf_g), leaf_c, rtol=1e-6, atol=1e-12)
    assert np.allclose(gu.cpu(hess_g), hess_c, rtol=1e-9)


@pytest.mark.parametrize("k", [1, 3])
def test_squared_error_gradient_is_bit_exact(k):
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(40 + k)
    n = 100003
    pred, y, w = rs.normal(size=(n, k)), rs.normal(size=(n, k)), rs.gamma(2.0, size=n)
    w[:3] = [0.0, 1e-12, 1e6]
    for weight in (None, w):
        g_c, h_c = orc.weighted_gradient("squared_error", y, pred, weight, 0.3)
        g_g, h_g = ops.weighted_gradient("squared_error", y, pred, weight, 0.3)
        assert np.array_equal(gu.cpu(g_g), g_c) and np.array_equal(gu.cpu(h_g), h_c)


@pytest.mark.parametrize("k", [1, 2, 8, 13])
def test_log_loss_gradient_matches_oracle(k):
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(50 + k)
    n = 50021
    pred = 5 * rs.normal(size=(n, k))
    pred[0] = 700.0 * (1 - 2 * (np.arange(k) % 2))  # saturated row
    y = rs.randint(0, max(k, 2), n).astype(np.float64)
    w = rs.gamma(2.0, size=n)
    g_c, h_c = orc.weighted_gradient("log_loss", y.reshape(-1, 1) if k == 1 else y, pred, w, 0.1)
    g_g, h_g = ops.weighted_gradient("log_loss", y.reshape(-1, 1) if k == 1 else y, pred, w, 0.1)
    # the device's exp and libm's differ in the last bit: 1e-12 of the largest gradient of the row
    scale = np.abs(g_c).max(axis=1, keepdims=True) + 1e-300
    assert (np.abs(gu.cpu(g_g) - g_c) <= 1e-12 * scale).all()
    assert np.allclose(gu.cpu(h_g), h_c, rtol=1e-12, atol=0)
    assert np.isfinite(gu.cpu(g_g)).all() and (gu.cpu(h_g) >= 1e-8).all()


@pytest.mark.parametrize("objective,n,k", [("squared_error", 100003, 1), ("squared_error", 20481, 3),
                                           ("log_loss", 70001, 1), ("log_loss", 30011, 8), ("log_loss", 9001, 5),
                                           ("log_loss", 300, 13)])
def test_gradient_pass_with_the_quantisers_sums(objective, n, k):
    """lbt_weighted_gradient_sums writes the same g and h as lbt_weighted_gradient and the first level
    of the quantiser's absolute sums; a build that is handed those sums skips its own pass over g
    and h and must give the oracle's scales, rounded pairs and tree bit for bit."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(n + k)
    pred = 3 * rs.normal(size=(n, k))
    if objective == "squared_error":
        y = rs.normal(size=(n, k))
    else:
        y = rs.randint(0, max(k, 2), n).astype(np.float64)
        y = y.reshape(-1, 1) if k == 1 else y
    w = rs.gamma(2.0, size=n)
    g0, h0 = ops.weighted_gradient(objective, y, pred, w, 0.3)
    g1, h1, sums = ops.weighted_gradient(objective, y, pred, w, 0.3, sums=True)
    assert torch.equal(g0, g1) and torch.equal(h0, h1)
    # the chunk sums against a plain numpy restatement of the fixed order: 4096 entries per chunk,
    # lane t adds entries t, t + 256, ..., then a binary tree over the 256 lanes
    for arr, got in ((gu.cpu(g1), gu.cpu(sums[0])), (gu.cpu(h1), gu.cpu(sums[1]))):
        flat = np.abs(arr.reshape(-1))
        m = (flat.size + 4095) // 4096
        padded = np.zeros(m * 4096)
        padded[: flat.size] = flat
        lanes = np.zeros((m, 256))
        for j in range(16):
            lanes += padded.reshape(m, 16, 256)[:, j, :]
        stride = 128
        while stride >= 1:
            lanes[:, :stride] += lanes[:, stride: 2 * stride]
            stride //= 2
        assert np.array_equal(got, lanes[:, 0])
    X = rs.normal(size=(n, 6)).astype(np.float32)
    cr = orc.build_tree(X, gu.cpu(g1), gu.cpu(h1), max_depth=4, split_samples=32, seed=11)
    gr = ops.build_tree(X, g1, h1, max_depth=4, split_samples=32, seed=11, taps=True, abs_sum_chunks=sums)
    gu.assert_tree_parity(gr, cr)
    # the asynchronous form, as the boosting loop calls it
    r2 = ops.build_tree(X, g1, h1, max_depth=4, split_samples=32, seed=11, wait=False, abs_sum_chunks=sums)
    assert torch.equal(r2.leaf_value, gr.leaf_value) and torch.equal(r2.feature, gr.feature)


# depth 13 / 14: the last level has 4096 / 8192 segments, either side of what the windowed leaf
# kernel indexes; 600 split samples: two-byte bins; depth 1: no bin cache
@pytest.mark.parametrize("k,depth,s", [(1, 6, 64), (4, 6, 64), (1, 13, 16), (1, 14, 16), (2, 5, 600), (1, 1, 64)])
def test_row_leaf_prediction_update_equals_predict(k, depth, s):
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    X, g, h = _problem(60 + k, 30000, 9, k)
    r = ops.build_tree(X, g, h, max_depth=depth, split_samples=s, seed=3, row_leaf=True)
    base = np.random.RandomState(1).normal(size=(30000, k))
    pred = torch.from_numpy(base.copy()).cuda()
    ops.add_leaf_values(pred, r.leaf_value, r.row_leaf)
    tree = (r.leaf_value, r.feature, r.split_value)
    assert torch.equal(pred, torch.from_numpy(base).cuda() + ops.predict(X, [tree], k))
    assert np.array_equal(gu.cpu(pred), orc.add_leaf_values(base, gu.cpu(r.leaf_value), gu.cpu(r.row_leaf)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gather_rows_matches_oracle(dtype):
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(8)
    X = rs.normal(size=(5000, 17)).astype(dtype)
    rows = rs.randint(900, 6200, 300).astype(np.int64)  # some outside the shard [1000, 6000)
    want = orc.gather_rows(X, rows, row_offset=1000)
    assert (want == 0).all(axis=1).any() and (want != 0).any()
    assert np.array_equal(gu.cpu(ops.gather_rows(X, tuple(rows), row_offset=1000)), want)
    assert np.array_equal(gu.cpu(ops.gather_rows(X, torch.from_numpy(rows).cuda(), row_offset=1000)), want)
    assert ops.gather_rows(X, (), row_offset=0).shape == (0, 17)


def test_async_build_gives_the_same_tree_and_defers_the_profile():
    from lbtree import _lib, ops

    X, g, h = _problem(77, 40000, 12, 2)
    kw = dict(max_depth=6, split_samples=64, seed=11, row_leaf=True)
    a = ops.build_tree(X, g, h, **kw)
    _lib.profile_reset()
    _lib.profile_enable(1)
    try:
        b = [ops.build_tree(X, g, h, wait=False, **kw) for _ in range(3)]  # queued back to back on one workspace
        prof = _lib.profile_get()  # waits for the three calls
    finally:
        _lib.profile_enable(0)
    for r in b:
        for name in ["leaf_value", "feature", "split_value", "gain", "hessian", "row_leaf"]:
            assert torch.equal(getattr(a, name), getattr(r, name)), name
    assert prof["histogram"]["launches"] == 3 * 6 and prof["binning"]["launches"] == 3
    assert len(prof["levels"]) == 6 and prof["levels"][0]["instances"] == 3 * 40000
    assert all(lv["built_instances"] <= lv["instances"] for lv in prof["levels"])
    with pytest.raises(_lib.LbtError):
        ops.build_tree(X, g, h, max_depth=3, split_samples=16, seed=1, taps=True, wait=False)


def test_two_runs_are_bit_identical():
    import gpu_util as gu

    X, g, h = _problem(2, 50000, 20, 1)
    a = gu.gpu_build(X, g, h, max_depth=6, split_samples=256, seed=5)
    b = gu.gpu_build(X, g, h, max_depth=6, split_samples=256, seed=5)
    torch.cuda.synchronize()
    for name in ["leaf_value", "feature", "split_value", "gain", "hessian", "positions", "histogram"]:
        assert torch.equal(getattr(a, name), getattr(b, name)), name


def test_errors_surface_as_exceptions():
    from lbtree import _lib, ops

    X = np.zeros((10, 2), np.float32)
    g = np.zeros((10, 1))
    with pytest.raises(_lib.LbtError):
        ops.build_tree(X, g, g, max_depth=2, split_samples=4096, seed=0)
    with pytest.raises(_lib.LbtError):
        ops.build_tree(X.astype(np.float16), g, g, max_depth=2, split_samples=16, seed=0)
    with pytest.raises(_lib.LbtError):
        ops.build_tree(X, g[:5], g[:5], max_depth=2, split_samples=16, seed=0)


@pytest.mark.parametrize("n,f,s,dtype,offset,total", [
    (5000, 7, 64, np.float32, 0, None),
    (300, 3, 256, np.float64, 0, None),      # more samples than rows: duplicates collapse
    (4000, 12, 2048, np.float32, 0, None),
    (1000, 5, 32, np.float32, 2500, 6000),   # a shard in the middle of a larger dataset: other rows give 0
    (1, 2, 8, np.float64, 0, None),
])
def test_select_split_samples_stage(n, f, s, dtype, offset, total):
    """The stage on its own against the oracle's restatement of SelectSplitSamples
    (build_tree.cu:867-964): proposals bit for bit, and the same ones the whole build uses."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    X, g, h = _problem(n + f, n, f, 1, dtype)
    props, rp = ops.select_split_samples(torch.from_numpy(X).cuda(), s, 77, dataset_rows=total, row_offset=offset)
    want, want_rp = orc.split_proposals(X, 77, s, dataset_rows=total, row_offset=offset)
    assert np.array_equal(gu.cpu(rp), want_rp)
    assert np.array_equal(gu.cpu(props).view(np.uint8), want.view(np.uint8))
    # ascending inside a feature, +inf last
    pr, r = gu.cpu(props), gu.cpu(rp)
    for j in range(f):
        seg = pr[r[j]:r[j + 1]]
        assert seg.size >= 1 and np.isinf(seg[-1]) and np.all(np.diff(seg) > 0)
    if offset == 0 and total is None:
        t = ops.build_tree(torch.from_numpy(X).cuda(), torch.from_numpy(g).cuda(), torch.from_numpy(h).cuda(),
                           max_depth=1, split_samples=s, seed=77, taps=True)
        assert np.array_equal(gu.cpu(t.row_pointers), gu.cpu(rp))
        assert np.array_equal(gu.cpu(t.proposals).view(np.uint8), pr.view(np.uint8))


@pytest.mark.parametrize("n,k,offset", [(5000, 1, 0), (3000, 3, 0), (700, 8, 123456), (1, 1, 0), (9000, 2, 7)])
def test_quantise_gradients_stage(n, k, offset):
    """The quantiser on its own against the oracle (build_tree.cu:51-140, :143-165, :168-204): the
    scales from the absolute sums in the fixed order, every rounded pair and the root sums."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(n + k)
    g = rs.randn(n, k) * np.exp(rs.randn(n, 1))
    h = rs.rand(n, k) + 1e-3
    q, sums, sc = ops.quantise_gradients(torch.from_numpy(g).cuda(), torch.from_numpy(h).cuda(), 4242,
                                         row_offset=offset)
    want_sc = orc.scales(orc.abs_sums(g, h))
    assert np.array_equal(gu.cpu(sc), want_sc)
    want = orc.quantise_all(g, h, 4242, want_sc, row_offset=offset)
    assert np.array_equal(gu.cpu(q).astype(np.int64), want)
    assert np.array_equal(gu.cpu(sums), want.sum(axis=0))
    # each rounded value is within one unit of the scaled input
    assert np.all(np.abs(want[:, :, 0] - g * want_sc[0]) < 1.0)


def test_property_sweep_against_the_oracle():
    """Drawn cases in the ranges of the reference's property tests (test_with_hypothesis.py:26-40,
    148-168: depth 1..8, split_samples 1..500, both dtypes, sample weights, feature fractions), plus
    what the histogram layouts depend on (feature counts either side of a group, two-byte bins, small
    histogram budgets, skewed and low-cardinality columns). Every case is printed before it runs."""
    from hypothesis import HealthCheck, given, settings, strategies as st
    import gpu_util as gu

    @settings(max_examples=60, deadline=None, derandomize=True, database=None,
              suppress_health_check=list(HealthCheck))
    @given(n=st.sampled_from([1, 37, 600, 4000, 25000]), f=st.sampled_from([1, 2, 5, 17, 64, 65, 130]),
           k=st.sampled_from([1, 1, 2, 4]), depth=st.integers(1, 8), s=st.integers(1, 500),
           f64=st.booleans(), kind=st.integers(0, 3), budget=st.sampled_from([0, 0, 150000, 4000000]),
           frac=st.sampled_from([1.0, 1.0, 0.5]), weighted=st.booleans(), seed=st.integers(0, 2**31 - 1))
    def run(n, f, k, depth, s, f64, kind, budget, frac, weighted, seed):
        print("case", dict(n=n, f=f, k=k, depth=depth, s=s, f64=f64, kind=kind, budget=budget, frac=frac,
                           weighted=weighted, seed=seed), flush=True)
        rs = np.random.RandomState(seed % 100003)
        if n * f > 1_500_000:
            n = 1_500_000 // f
        X = rs.randn(n, f).astype(np.float64 if f64 else np.float32)
        if kind == 1:
            X[:, 0] = rs.randint(0, 3, n)             # low cardinality
        elif kind == 2:
            X = np.exp(3 * X).astype(X.dtype)         # skewed
        elif kind == 3:
            X[: n // 2] = np.sort(X[: n // 2], axis=0)  # partly sorted: nodes become row ranges
        w = rs.rand(n, 1) * 3 if weighted else 1.0     # the caller multiplies both by the sample weight
        g = rs.randn(n, k) * w
        h = np.maximum((rs.rand(n, k) + 0.05) * w, 1e-8)
        fs = None
        if frac < 1.0 and f > 1:
            fs = rs.rand(f) < frac
            fs[rs.randint(f)] = True
        gr, cr = gu.both(X, g, h, levels=(n * depth <= 200000), max_depth=depth, split_samples=s, seed=seed,
                         hist_cache_bytes=budget, feature_set=fs)
        gu.assert_tree_parity(gr, cr, levels=(n * depth <= 200000))

    run()


@pytest.mark.parametrize("f,dtype,skip", [(8, np.float32, 1), (6, np.float32, 3), (7, np.float32, 2), (5, np.float64, 1)])
def test_matrix_that_starts_off_a_16_byte_boundary(f, dtype, skip):
    """X as a view that begins `skip` elements into an allocation: rows then start on element
    boundaries only, which the binning pass has to load as such."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    n = 3000
    X, g, h = _problem(f + skip, n, f, 1, dtype)
    base = torch.zeros(n * f + skip, dtype=torch.from_numpy(X).dtype, device="cuda")
    Xd = base[skip:].view(n, f)
    Xd.copy_(torch.from_numpy(X))
    assert Xd.data_ptr() % 16 != 0 and Xd.is_contiguous()
    gr = ops.build_tree(Xd, torch.from_numpy(g).cuda(), torch.from_numpy(h).cuda(), max_depth=5, split_samples=64,
                        seed=31, taps=True, row_leaf=True)
    cr = orc.build_tree(X, g, h, max_depth=5, split_samples=64, seed=31)
    gu.assert_tree_parity(gr, cr)


@pytest.mark.parametrize("f,lanes", [(13, 4), (100, 8), (330, 16)])
@pytest.mark.parametrize("k", [1, 3])
def test_predict_with_a_handful_of_trees(f, lanes, k):
    """Ensembles of at most as many trees as lanes share a row are walked one tree per lane: a
    single tree (what a boosting round predicts with), exactly that many, and one more (the
    general shape again)."""
    import gpu_util as gu
    import oracle_lib as orc
    from lbtree import ops

    rs = np.random.RandomState(f * 7 + k)
    X = rs.rand(5003, f).astype(np.float32)
    trees_c, trees_g = [], []
    for t in range(lanes + 1):
        depth = [6, 2, 8, 4][t % 4]
        m, inner = 2 ** (depth + 1) - 1, 2 ** depth - 1
        feat = -np.ones(m, np.int32)
        feat[:inner] = rs.randint(0, f, inner)
        split = rs.rand(m)
        leaf = rs.randn(m, k)
        trees_c.append((leaf, feat, split))
        trees_g.append(tuple(ops.as_device(a) for a in (leaf, feat, split)))
    for n_trees in (1, 2, lanes, lanes + 1):
        want = orc.predict(X, trees_c[:n_trees], k)
        assert np.array_equal(gu.cpu(ops.predict(X, trees_g[:n_trees], k)), want), n_trees
