"""The reference's own model-level tests (legateboost/test/models/test_tree.py,
test_model.py, test_estimator.py) restated against the `Tree` mirror and the
boosting loop, on the GPU."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _np(t):
    return t.cpu().numpy()


def test_basic():
    from lbtree.models import Tree

    X = np.array([[0.0], [1.0]])
    g = np.array([[0.0], [-1.0]])
    h = np.array([[1.0], [1.0]])
    model = Tree(max_depth=1, l2_regularization=0.0).set_random_state(np.random.RandomState(2)).fit(X, g, h)
    assert np.allclose(_np(model.predict(X)), np.array([[0.0], [1.0]]))


@pytest.mark.parametrize("num_outputs", [1, 5])
def test_improving_with_depth(num_outputs):
    from lbtree.models import Tree

    rs = np.random.RandomState(0)
    X = rs.random_sample((10000, 100))
    g = rs.normal(size=(X.shape[0], num_outputs))
    h = rs.random_sample(g.shape) + 0.1
    y = -g / h
    metrics = []
    for max_depth in range(0, 12):
        model = Tree(max_depth=max_depth).set_random_state(np.random.RandomState(2)).fit(X, g, h)
        predict = _np(model.predict(X))
        loss = ((predict - y) ** 2 * h).sum(axis=0) / h.sum(axis=0)
        metrics.append(loss.mean())
    assert all(b <= a + 1e-12 for a, b in zip(metrics, metrics[1:]))
    assert metrics[-1] < metrics[0]


def test_max_depth():
    import lbtree as lb

    X = np.random.RandomState(0).random_sample((2, 1))
    y = np.array([500.0, 500.0])
    model = lb.LBRegressor(init=None, base_models=(lb.models.Tree(max_depth=20),), learning_rate=1.0,
                           n_estimators=1, random_state=0)
    model.fit(X, y)


def test_l2_and_l1_regularization():
    import lbtree as lb

    X = np.array([[0.0], [0.0]])
    y = np.array([500.0, 500.0])
    m = lb.LBRegressor(init=None, base_models=(lb.models.Tree(l2_regularization=10.0, max_depth=0),),
                       learning_rate=1.0, n_estimators=1, random_state=0)
    m.fit(X, y)
    assert np.isclose(_np(m.predict(X))[0], y.sum() / (y.size + 10.0))
    m.update(X, y)
    assert np.isclose(_np(m.predict(X))[0], y.sum() / (y.size + 10.0))
    m = lb.LBRegressor(init=None, base_models=(lb.models.Tree(l2_regularization=0.0, l1_regularization=1.5,
                                                               max_depth=0),),
                       learning_rate=1.0, n_estimators=1, random_state=0)
    m.fit(X, y)
    assert np.isclose(_np(m.predict(X))[0], (y.sum() - 1.5) / y.size)
    m.update(X, y)
    assert np.isclose(_np(m.predict(X))[0], (y.sum() - 1.5) / y.size)
    y = np.array([0.5, 0.5])
    m.fit(X, y)
    assert np.isclose(_np(m.predict(X))[0], 0.0)
    m.update(X, y)
    assert np.isclose(_np(m.predict(X))[0], 0.0)


def test_callable_feature_sample():
    import lbtree as lb

    def feature_fraction():
        return torch.tensor([0, 1, 0, 0, 0, 0, 0, 0, 0, 0], dtype=torch.bool)

    rng = np.random.RandomState(0)
    X = rng.randn(100, 10)
    y = rng.randn(100)
    model = lb.LBRegressor(base_models=(lb.models.Tree(feature_fraction=feature_fraction),), random_state=0,
                           n_estimators=10).fit(X, y)
    used = np.concatenate([_np(m.feature) for m in model])
    assert set(used[used >= 0].tolist()) == {1}

    def feature_fraction_int():
        return torch.tensor([0, 1, 0, 0, 0, 0, 0, 0, 0, 0])

    with pytest.raises(ValueError, match=r"feature_fraction must return a boolean array of shape \(n_features,\)"):
        lb.LBRegressor(base_models=(lb.models.Tree(feature_fraction=feature_fraction_int),), random_state=0).fit(X, y)

    def feature_fraction_wrong_shape():
        return torch.tensor([0, 1, 0, 0, 0, 0, 0, 0, 0], dtype=torch.bool)

    with pytest.raises(ValueError, match=r"feature_fraction must return a boolean array of shape \(n_features,\)"):
        lb.LBRegressor(base_models=(lb.models.Tree(feature_fraction=feature_fraction_wrong_shape),),
                       random_state=0).fit(X, y)


def test_feature_fraction_float_samples_features():
    import lbtree as lb

    rng = np.random.RandomState(0)
    X = rng.randn(300, 10)
    y = X[:, 0] * 3 + rng.randn(300) * 0.1
    base = lb.LBRegressor(base_models=(lb.models.Tree(feature_fraction=1.0, max_depth=3),), random_state=1,
                          n_estimators=10).fit(X, y)
    samp = lb.LBRegressor(base_models=(lb.models.Tree(feature_fraction=0.3, max_depth=3),), random_state=1,
                          n_estimators=10).fit(X, y)
    fb = np.concatenate([_np(m.feature) for m in base])
    fsamp = np.concatenate([_np(m.feature) for m in samp])
    assert len(set(fsamp[fsamp >= 0].tolist())) >= len(set(fb[fb >= 0].tolist()))
    for m in samp:
        assert len(set(_np(m.feature)[_np(m.feature) >= 0].tolist())) <= 3


def test_min_split_gain():
    import lbtree as lb

    rng = np.random.RandomState(0)
    X = rng.random_sample((100, 1))
    y = rng.random_sample(100)
    a = lb.LBRegressor(init=None, base_models=(lb.models.Tree(min_split_gain=0.0, max_depth=12),), learning_rate=1.0,
                       n_estimators=1, random_state=0).fit(X, y)
    b = lb.LBRegressor(init=None, base_models=(lb.models.Tree(min_split_gain=0.03, max_depth=12),),
                       learning_rate=1.0, n_estimators=1, random_state=0).fit(X, y)
    assert int((b[0].hessian > 0).sum()) < int((a[0].hessian > 0).sum())
    assert np.isclose(float(a[0].gain[0]), float(b[0].gain[0]) + 0.03)


def test_wide_deep():
    import lbtree as lb

    rng = np.random.RandomState(0)
    X = rng.randn(5000, 500)
    y = rng.randn(X.shape[0])
    lb.LBRegressor(init=None, n_estimators=3, base_models=(lb.models.Tree(max_depth=10),)).fit(X, y)


def test_batch_inference():
    from lbtree.models import Tree

    rs = np.random.RandomState(0)
    X = rs.random_sample((1000, 10))
    g = rs.normal(size=(1000, 2))
    h = rs.random_sample(g.shape) + 0.1
    a = Tree(max_depth=5).set_random_state(np.random.RandomState(10)).fit(X, g, h)
    b = Tree(max_depth=5).set_random_state(np.random.RandomState(11)).fit(X, g, h)
    assert not (a == b) and a == a and isinstance(str(a), str) and "leaf=" in str(a)
    both = _np(Tree.batch_predict([a, b], X))
    assert np.allclose(both, _np(a.predict(X)) + _np(b.predict(X)))
    assert np.allclose(_np((a * 2.0).predict(X)), 2.0 * _np(a.predict(X)))


def sanity_check_models(model):
    # legateboost/testing/utils.py:22-39
    for m in model:
        feat, hess, gain = _np(m.feature), _np(m.hessian), _np(m.gain)
        split_nodes = feat != -1
        assert (hess[split_nodes] > 0.0).all()
        assert (gain[split_nodes] > 0.0).all()
        leaves = (feat == -1) & (hess[:, 0] > 0.0)
        assert np.isclose(hess[leaves].sum(axis=0), hess[0]).all()


def test_regressor_and_update():
    import lbtree as lb

    rs = np.random.RandomState(2)
    X = rs.random_sample((3000, 10)).astype(np.float32)
    y = np.stack([X[:, 0] * 2 + np.sin(6 * X[:, 1]), X[:, 2] - X[:, 3]], axis=1) + rs.normal(0, 0.05, (3000, 2))
    m = lb.LBRegressor(n_estimators=15, base_models=(lb.models.Tree(max_depth=5),), random_state=3, verbose=0)
    m.fit(X, y)
    sanity_check_models(m)
    pred = _np(m.predict(X))
    assert ((pred - y) ** 2).mean() < 0.25 * ((y - y.mean(axis=0)) ** 2).mean()
    # fit then update on the same data gives the same predictions (test_estimator.py:60-65)
    m.update(X, y)
    assert np.allclose(_np(m.predict(X)), pred, rtol=1e-4, atol=1e-4)


def test_subsample():
    """test_estimator.py:191-227: on data that a deep tree overfits, keeping half of the rows per round
    gives the lower test error (averaged over five data sets); and the seed of the row draw is taken from
    the estimator's RandomState where the reference takes it, so the tree seeds are the reference's."""
    import lbtree as lb
    from sklearn.datasets import make_regression
    from sklearn.model_selection import train_test_split

    sub_mse, full_mse = [], []
    for i in range(5):
        X, y = make_regression(n_samples=1000, n_features=10, noise=10.0, random_state=i)
        X_train, X_test, y_train, y_test = train_test_split(X, y, test_size=0.5, random_state=i)
        params = dict(n_estimators=20, random_state=i, learning_rate=0.5,
                      base_models=(lb.models.Tree(max_depth=12, alpha=0.0),))
        sub = lb.LBRegressor(**params, subsample=0.5).fit(X_train, y_train)
        full = lb.LBRegressor(**params).fit(X_train, y_train)
        sub_mse.append(((_np(sub.predict(X_test)).ravel() - y_test) ** 2).mean())
        full_mse.append(((_np(full.predict(X_test)).ravel() - y_test) ** 2).mean())
    assert np.mean(sub_mse) < np.mean(full_mse)

    # order of the draws from the estimator's RandomState: row-draw seed, then the tree's seed, every round
    m = lb.LBRegressor(n_estimators=3, random_state=11, subsample=0.5, base_models=(lb.models.Tree(max_depth=2),))
    rs = np.random.RandomState(7)
    X = rs.random_sample((500, 4)).astype(np.float32)
    m.fit(X, X[:, 0] + rs.normal(0, 0.1, 500))
    expect = np.random.RandomState(11)
    for _ in m:
        expect.randint(0, 2**32, dtype=np.int64)
        expect.randint(0, 2**31)
    assert m.random_state_.randint(0, 2**31) == expect.randint(0, 2**31)
    with pytest.raises(ValueError):
        lb.LBRegressor(subsample=0.0)


@pytest.mark.parametrize("num_class", [2, 5])
def test_classifier(num_class):
    import lbtree as lb

    rs = np.random.RandomState(4)
    X = rs.randn(4000, 8).astype(np.float32)
    P = rs.randn(8, num_class)
    y = np.argmax(X @ P + rs.gumbel(size=(4000, num_class)) * 0.3, axis=1).astype(np.float64)
    m = lb.LBClassifier(n_estimators=12, base_models=(lb.models.Tree(max_depth=4),), random_state=5)
    m.fit(X, y)
    sanity_check_models(m)
    proba = _np(m.predict_proba(X))
    assert proba.shape == (4000, num_class) and np.allclose(proba.sum(axis=1), 1.0)
    assert (_np(m.predict(X)) == y).mean() > 0.7


def _tree_ensemble_eval(a, X):
    """ai.onnx.ml TreeEnsemble (opset 5) for one tree with BRANCH_LEQ nodes and SUM aggregation."""
    out = np.zeros((X.shape[0], a["n_targets"]))
    for r in range(X.shape[0]):
        i, leaf = a["tree_roots"][0], False
        while not leaf:
            assert a["nodes_modes"][i] == 0
            if X[r, a["nodes_featureids"][i]] <= a["nodes_splits"][i]:
                i, leaf = a["nodes_truenodeids"][i], bool(a["nodes_trueleafs"][i])
            else:
                i, leaf = a["nodes_falsenodeids"][i], bool(a["nodes_falseleafs"][i])
        out[r, a["leaf_targetids"][i]] += a["leaf_weights"][i]
    return out


def test_onnx_attributes_describe_the_same_function():
    import lbtree as lb

    rs = np.random.RandomState(4)
    X = rs.randn(400, 5)
    g, h = rs.randn(400, 2), np.ones((400, 2))
    tree = lb.models.Tree(max_depth=4, split_samples=32).set_random_state(np.random.RandomState(1)).fit(X, g, h)
    assert _np(tree.feature)[0] != -1
    want = _np(tree.predict(X))
    got = sum(_tree_ensemble_eval(tree.onnx_attributes(k), X) for k in range(2))
    assert np.array_equal(got, want)
    try:
        import onnx  # noqa: F401
    except ImportError:
        with pytest.raises(ImportError):
            tree.to_onnx()
    else:
        assert tree.to_onnx().graph.name == "legateboost.models.Tree"
