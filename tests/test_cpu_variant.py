"""Sanity of the CPU-variant timing baseline (oracle/cpu_variant.cpp): it must
be a working tree learner, thread-count independent, and agree with the oracle
wherever the two algorithms coincide (exact leaf statistics of a given tree)."""
import numpy as np

import cpu_variant_lib as cv
import oracle_lib as orc


def test_cpu_variant_learns_and_threads_agree():
    rs = np.random.RandomState(0)
    X = rs.random_sample((20000, 12)).astype(np.float32)
    y = np.sin(6 * X[:, 0]) + X[:, 1] * X[:, 2] + rs.normal(0, 0.05, 20000)
    g = (y.mean() - y).reshape(-1, 1)
    h = np.ones((20000, 1))
    a = cv.build_tree(X, g, h, max_depth=6, split_samples=64, seed=3, n_threads=1)
    b = cv.build_tree(X, g, h, max_depth=6, split_samples=64, seed=3, n_threads=4)
    assert np.array_equal(a[1], b[1]) and np.allclose(a[0], b[0], rtol=1e-9, atol=1e-12)
    pred = cv.predict(X, [(a[0], a[1], a[2])], 1, n_threads=2)
    before = ((y.mean() - y) ** 2).mean()
    after = ((y.mean() + pred[:, 0] - y) ** 2).mean()
    assert after < 0.5 * before
    # same walk as the oracle's predict
    assert np.array_equal(pred, orc.predict(X, [(a[0], a[1], a[2])], 1))
    # its leaves are exactly the Newton steps of the rows they hold: update_tree recomputes them
    leaf, hess = orc.update_tree(X, g, h, a[1], a[2], 0.0, 1.0)
    used = a[4][:, 0] > 0
    assert np.allclose(leaf[used], a[0][used], rtol=1e-9, atol=1e-12)
    assert np.allclose(hess[used], a[4][used], rtol=1e-12)
