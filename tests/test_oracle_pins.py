"""Pins the CPU oracle against things that do not come from the oracle itself:
known answers printed by rocThrust's own headers, closed forms, Python
big-integer arithmetic, a brute-force numpy restatement, and the known-answer
cases of the reference's own tests (legateboost/test/models/test_tree.py)."""
import json
import os

import numpy as np
import pytest

import brute
import oracle_lib as orc

M = 2**31 - 1
A = 48271
HERE = os.path.dirname(os.path.abspath(__file__))


def kat():
    with open(os.path.join(HERE, "golden", "thrust_rng_kat.json")) as f:
        return json.load(f)


# ----------------------------------------------------------------------------- RNG


def test_minstd_closed_forms():
    # seed 42: first raw draw is 42*48271 mod m, first uniform is (x-1)/(m-1)
    x = orc.lib.orc_minstd_next(orc.lib.orc_minstd_seed(42))
    assert x == (42 * A) % M
    assert orc.lib.orc_uniform01(x) == (x - 1) / 2147483646.0
    assert abs(orc.lib.orc_uniform01(x) - 0.0009440728472024881) < 1e-18
    # seeding rule: 0 and multiples of m map to 1
    for s, want in [(0, 1), (M, 1), (2 * M, 1), (1, 1), (M + 5, 5), (2**32 - 1, (2**32 - 1) % M)]:
        assert orc.lib.orc_minstd_seed(s) == want


def test_minstd_discard_is_repeated_stepping():
    for s in [1, 42, 2147483646, 123456789]:
        x = orc.lib.orc_minstd_seed(s)
        y = x
        for z in range(0, 300):
            assert orc.lib.orc_minstd_discard(x, z) == y
            y = (y * A) % M
        assert orc.lib.orc_minstd_discard(x, 10**12) == (x * pow(A, 10**12, M)) % M


def test_thrust_known_answers_real_pairs():
    k = kat()
    for c in k["real_pairs"]:
        seed = int(c["seed"])
        x = orc.lib.orc_minstd_seed(seed & 0xFFFFFFFF)
        x = orc.lib.orc_minstd_next(x)
        assert orc.lib.orc_uniform01(x) == float.fromhex(c["u1"]), c
        x = orc.lib.orc_minstd_next(x)
        assert orc.lib.orc_uniform01(x) == float.fromhex(c["u2"]), c
    raw = k["raw"]
    x = orc.lib.orc_minstd_seed(42)
    for want in raw:
        x = orc.lib.orc_minstd_next(x)
        assert x == want


def test_thrust_known_answers_row_samples():
    for c in kat()["row_samples"]:
        got = orc.row_samples(c["seed"], c["rows"], len(c["out"]))
        assert got.tolist() == c["out"], c


def test_row_samples_in_range_and_formula():
    for seed, rows in [(7, 1), (7, 2), (99, 1000), (5, 10**7), (2**31 - 1, 3)]:
        got = orc.row_samples(seed, rows, 64)
        assert got.min() >= 0 and got.max() <= rows - 1
        s = seed % M or 1
        for i in range(64):
            x = (s * pow(A, i + 1, M)) % M
            assert got[i] == int(((x - 1) / 2147483646.0) * float(rows))


# ----------------------------------------------------------------------------- hash


def _sar(v, n):
    """arithmetic shift right on a 64-bit two's-complement value held as a Python int"""
    if v >= 2**63:
        v -= 2**64
    return (v >> n) & (2**64 - 1)


def py_hash(k):
    k &= 2**64 - 1
    k ^= _sar(k, 33)
    k = (k * 0xFF51AFD7ED558CCD) & (2**64 - 1)
    k ^= _sar(k, 33)
    k = (k * 0xC4CEB9FE1A85EC53) & (2**64 - 1)
    k ^= _sar(k, 33)
    return k - 2**64 if k >= 2**63 else k


def py_combine(seed, v):
    s = seed & (2**64 - 1)
    t = (py_hash(v) + 0x9E3779B9 + ((s << 6) & (2**64 - 1)) + _sar(s, 2)) & (2**64 - 1)
    r = s ^ t
    return r - 2**64 if r >= 2**63 else r


def fmix64_unsigned(k):
    k ^= k >> 33
    k = (k * 0xFF51AFD7ED558CCD) & (2**64 - 1)
    k ^= k >> 33
    k = (k * 0xC4CEB9FE1A85EC53) & (2**64 - 1)
    k ^= k >> 33
    return k


def test_hash_matches_bigint_restatement():
    rs = np.random.RandomState(0)
    vals = [0, 1, 2, -1, -2, 2**31 - 1, 2**31, 2**63 - 1, -(2**63), 10**7, 99999999] + [
        int(v) for v in rs.randint(-(2**62), 2**62, size=200)
    ]
    for v in vals:
        assert orc.lib.orc_hash(v) == py_hash(v), v
    assert orc.lib.orc_hash(0) == 0


def test_hash_equals_published_fmix64_when_no_sign_is_involved():
    # Where both intermediate products are non-negative as int64, the signed
    # variant must coincide with MurmurHash3's fmix64.
    found = 0
    for v in range(1, 4000):
        k = v ^ (v >> 33)
        k1 = (k * 0xFF51AFD7ED558CCD) & (2**64 - 1)
        if k1 >= 2**63:
            continue
        k1 ^= k1 >> 33
        k2 = (k1 * 0xC4CEB9FE1A85EC53) & (2**64 - 1)
        if k2 >= 2**63:
            continue
        found += 1
        want = fmix64_unsigned(v)
        want = want - 2**64 if want >= 2**63 else want
        assert orc.lib.orc_hash(v) == want
    assert found > 100
    # and it must differ from the unsigned one where the sign matters (v = 1)
    assert fmix64_unsigned(1) == 0xB456BCFC34C2CB2C
    assert orc.lib.orc_hash(1) != 0xB456BCFC34C2CB2C - 2**64


def test_hash_combine_matches_bigint_restatement():
    rs = np.random.RandomState(1)
    for _ in range(300):
        seed = int(rs.randint(0, 2**31))
        row = int(rs.randint(0, 2**40))
        k = int(rs.randint(0, 16))
        assert orc.lib.orc_hash_combine2(seed, row, k) == py_combine(py_combine(seed, row), k)
    # distinct (row, k) must give distinct streams for a fixed seed (spot check)
    seen = {orc.lib.orc_hash_combine2(5, r, k) for r in range(200) for k in range(4)}
    assert len(seen) == 800


# ----------------------------------------------------------------------------- quantiser


def test_abs_sum_order_definition():
    rs = np.random.RandomState(3)
    for n in [1, 2, 255, 256, 257, 4095, 4096, 4097, 3 * 4096 + 5, 70000]:
        g = rs.randn(n)
        h = rs.rand(n)
        got = orc.abs_sums(g, h)
        # independent restatement of the stated order with numpy reshapes
        def level(a):
            m = (len(a) + 4095) // 4096
            pad = np.zeros(m * 4096)
            pad[: len(a)] = a
            lanes = np.zeros((m, 256))
            p3 = pad.reshape(m, 16, 256)
            for j in range(16):
                lanes = lanes + p3[:, j, :]
            s = 128
            while s >= 1:
                lanes = lanes[:, :s] + lanes[:, s: 2 * s]
                s //= 2
            return lanes[:, 0]
        a, b = level(np.abs(g)), level(np.abs(h))
        while len(a) > 1:
            a, b = level(a), level(b)
        assert got[0] == a[0] and got[1] == b[0]
        assert np.isclose(got[0], np.abs(g).sum(), rtol=1e-12)


def test_scales():
    sc = orc.scales(np.array([4.0, 0.0]))
    assert sc[0] == (2**31 - 1) / 4.0 and sc[1] == 1.0 and sc[2] == 1.0 / sc[0] and sc[3] == 1.0


def test_quantise_invariants_and_determinism():
    rs = np.random.RandomState(4)
    n, k = 5000, 3
    g = rs.randn(n, k)
    h = rs.rand(n, k) + 1e-3
    sc = orc.scales(orc.abs_sums(g, h))
    q = orc.quantise_all(g, h, 1234, sc)
    q2 = orc.quantise_all(g, h, 1234, sc)
    assert (q == q2).all()
    sg, sh = g * sc[0], h * sc[1]
    assert ((q[..., 0] == np.floor(sg)) | (q[..., 0] == np.floor(sg) + 1)).all()
    assert ((q[..., 1] == np.floor(sh)) | (q[..., 1] == np.floor(sh) + 1)).all()
    assert (q[..., 1] >= 0).all()
    assert np.abs(q[..., 0]).sum() <= 2**31 - 1 + n * k
    # unbiased: mean rounding error close to 0
    assert abs((q[..., 0] - sg).mean()) < 0.05
    # the draw order is grad first, hess second, from the per-(row,k) seed
    r, kk = 17, 2
    seed = py_combine(py_combine(1234, r), kk)
    x = (seed & 0xFFFFFFFF) % M or 1
    x = (x * A) % M
    u1 = (x - 1) / 2147483646.0
    x = (x * A) % M
    u2 = (x - 1) / 2147483646.0
    assert q[r, kk, 0] == int(np.floor(sg[r, kk]) + (u1 < sg[r, kk] - np.floor(sg[r, kk])))
    assert q[r, kk, 1] == int(np.floor(sh[r, kk]) + (u2 < sh[r, kk] - np.floor(sh[r, kk])))
    # row_offset shifts the row that is hashed
    q3 = orc.quantise_all(g[10:20], h[10:20], 1234, sc, row_offset=10)
    assert (q3 == q[10:20]).all()


# ----------------------------------------------------------------------------- proposals


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_split_proposals_bruteforce(dtype):
    rs = np.random.RandomState(5)
    n, f, s = 500, 7, 64
    X = rs.randn(n, f).astype(dtype)
    X[:, 2] = rs.randint(0, 5, n)  # duplicates
    X[:, 3] = 1.5  # constant
    props, rp = orc.split_proposals(X, 77, s)
    rows = orc.row_samples(77, n, s)
    assert rp[0] == 0 and rp[-1] == len(props)
    for j in range(f):
        want = np.unique(X[rows, j]).astype(dtype)
        want[-1] = np.inf
        got = props[rp[j]: rp[j + 1]]
        assert got.dtype == dtype
        assert np.array_equal(got, want)
        assert (np.diff(got) > 0).all()
    assert rp[4] - rp[3] == 1 and np.isinf(props[rp[3]])


def test_split_proposals_negative_zero_and_non_local_rows():
    X = np.array([[0.0], [-0.0], [0.0], [1.0]], np.float32)
    props, rp = orc.split_proposals(X, 3, 32)
    assert len(props) == 2 and props[0] == 0.0 and np.isinf(props[1])
    assert np.signbit(props[0])  # -0.0 sorts first and is the one kept
    # a shard that holds only rows [2,4): other sampled rows contribute 0
    props2, rp2 = orc.split_proposals(X[2:], 3, 32, dataset_rows=4, row_offset=2)
    assert props2[0] == 0.0 and np.isinf(props2[-1])


# ----------------------------------------------------------------------------- full build vs brute force


def _rand_problem(seed, n, f, k, dtype=np.float32, lowcard=True):
    rs = np.random.RandomState(seed)
    X = rs.randn(n, f).astype(dtype)
    if lowcard and f > 2:
        X[:, 1] = rs.randint(0, 4, n)
    g = rs.randn(n, k)
    h = rs.rand(n, k) + 0.1
    return X, g, h


@pytest.mark.parametrize("n,f,k,depth,s,l1,l2,msg", [
    (300, 4, 1, 3, 16, 0.0, 1.0, 0.0),
    (1000, 6, 2, 4, 32, 0.0, 1.0, 0.0),
    (700, 3, 3, 5, 600, 0.5, 0.1, 0.01),
    (50, 2, 1, 6, 8, 0.0, 0.0, 0.0),
])
def test_build_tree_matches_bruteforce(n, f, k, depth, s, l1, l2, msg):
    X, g, h = _rand_problem(n + f, n, f, k)
    r = orc.build_tree(X, g, h, max_depth=depth, split_samples=s, seed=11, l1=l1, l2=l2, min_split_gain=msg)
    # quantised values and proposals are pinned separately; reuse them
    b = brute.build(X, r.quantised, r.proposals, r.row_pointers, r.scales, depth, l1, l2, msg)
    assert np.array_equal(r.feature, b["feature"])
    assert np.array_equal(r.split_value, b["split"])
    assert np.array_equal(r.gain, b["gain"])
    assert np.array_equal(r.leaf_value, b["leaf"])
    assert np.array_equal(r.node_sums, b["node_sums"])
    assert (r.feature != -1).sum() >= 1


def test_build_tree_with_feature_set_matches_bruteforce():
    X, g, h = _rand_problem(9, 800, 5, 1)
    fs = np.array([0, 1, 0, 1, 0], bool)
    r = orc.build_tree(X, g, h, max_depth=4, split_samples=32, seed=2, feature_set=fs)
    b = brute.build(X, r.quantised, r.proposals, r.row_pointers, r.scales, 4, 0.0, 1.0, 0.0, feature_set=fs)
    assert np.array_equal(r.feature, b["feature"])
    assert set(r.feature[r.feature >= 0]) <= {1, 3}


def test_histogram_invariants_and_bruteforce():
    X, g, h = _rand_problem(21, 2000, 5, 2)
    depth = 4
    r = orc.build_tree(X, g, h, max_depth=depth, split_samples=48, seed=9, want_levels=True)
    assert r.hist_node_begin == 0
    B = r.n_bins
    rp = r.row_pointers
    bins = brute.bins_of(X, r.proposals, rp)
    q = r.quantised
    for d in range(depth):
        pos = r.positions_per_level[d]
        for node in range(2**d - 1, 2 ** (d + 1) - 1):
            if r.node_sums[node, 0, 1] <= 0:
                continue
            rows = pos[pos[:, 0] == node, 1]
            for kk in range(2):
                H = r.histogram[node, kk]
                # last bin of each feature == node sum (hess > 0 so the write is never skipped there)
                for j in range(5):
                    assert np.array_equal(H[rp[j + 1] - 1], r.node_sums[node, kk])
                # brute force cumulative histogram; bins where the reference skips the
                # write (cumulative grad <= 0 and hess == 0) are excluded
                raw = np.zeros((B, 2), np.int64)
                for j in range(5):
                    np.add.at(raw[:, 0], bins[rows, j], q[rows, kk, 0])
                    np.add.at(raw[:, 1], bins[rows, j], q[rows, kk, 1])
                cum = np.concatenate([np.cumsum(raw[rp[j]: rp[j + 1]], axis=0) for j in range(5)])
                ok = (cum[:, 0] > 0) | (cum[:, 1] > 0)
                assert np.array_equal(H[ok], cum[ok])
            # children add up to the parent, exactly
            if r.feature[node] != -1 and 2 * node + 2 < r.histogram.shape[0]:
                lc, rc = 2 * node + 1, 2 * node + 2
                assert np.array_equal(r.node_sums[lc] + r.node_sums[rc], r.node_sums[node])
    # level statistics: all rows are instances at every level; built <= half below the root
    assert r.level_instances.tolist() == [2000] * depth
    assert r.level_built_instances[0] == 2000
    for d in range(1, depth):
        assert r.level_built_instances[d] <= 1000


def test_positions_are_a_stable_partition():
    X, g, h = _rand_problem(31, 3000, 4, 1)
    depth = 5
    r = orc.build_tree(X, g, h, max_depth=depth, split_samples=32, seed=1, want_levels=True)
    lv = r.positions_per_level
    assert np.array_equal(lv[0][:, 0], np.zeros(3000)) and np.array_equal(lv[0][:, 1], np.arange(3000))
    for d in range(depth - 1):
        cur = lv[d]
        node, row = cur[:, 0].astype(np.int64), cur[:, 1]
        valid = (node >= 0)
        feat = np.where(valid, r.feature[np.maximum(node, 0)], -1)
        alive = valid & (feat != -1)
        x = X[row, np.maximum(feat, 0)].astype(np.float64)
        new = np.where(alive, np.where(x <= r.split_value[np.maximum(node, 0)], 2 * node + 1, 2 * node + 2), -1)
        order = np.argsort(new, kind="stable")
        assert np.array_equal(lv[d + 1][:, 0], new[order])
        assert np.array_equal(lv[d + 1][:, 1], row[order])
    assert np.array_equal(r.positions, lv[depth - 1])


def test_batched_levels_give_the_same_tree():
    # a tiny histogram budget forces several node batches per level and a
    # re-allocated histogram (no subtraction at those levels)
    X, g, h = _rand_problem(41, 1500, 4, 2)
    a = orc.build_tree(X, g, h, max_depth=5, split_samples=16, seed=3)
    nb = a.n_bins
    for budget in [nb * 2 * 16 * 3, nb * 2 * 16 * 1, 1]:
        b = orc.build_tree(X, g, h, max_depth=5, split_samples=16, seed=3, hist_cache_bytes=budget)
        assert np.array_equal(a.feature, b.feature)
        assert np.array_equal(a.split_value, b.split_value)
        assert np.array_equal(a.gain, b.gain)
        assert np.array_equal(a.leaf_value, b.leaf_value)
        assert np.array_equal(a.positions, b.positions)
        assert b.hist_node_end - b.hist_node_begin <= max(1, budget // (nb * 2 * 16))


# ----------------------------------------------------------------------------- tie rule


@pytest.mark.parametrize("lo_value", [1.0, 470.0])
def test_gain_tie_rule(lo_value):
    # One feature whose proposals have empty bins between occupied ones:
    # cumulative sums are identical over runs of empty bins, so gains tie.
    n = 64
    X = np.zeros((n, 1), np.float32)
    X[: n // 2, 0] = lo_value
    X[n // 2:, 0] = 600.0
    # make proposals 1..600 exist by placing one row at each integer value first
    Xp = np.arange(1, 601, dtype=np.float32).reshape(-1, 1)
    Xall = np.concatenate([Xp, X])
    g = np.zeros((len(Xall), 1))
    h = np.full((len(Xall), 1), 1e-300)  # rows that only exist to create proposals quantise to 0
    g[600: 600 + n // 2] = -1.0
    g[600 + n // 2:] = 1.0
    h[600:] = 1.0
    r = orc.build_tree(Xall, g, h, max_depth=1, split_samples=2048, seed=0)
    b = brute.build(Xall, r.quantised, r.proposals, r.row_pointers, r.scales, 1, 0.0, 1.0, 0.0)
    assert r.feature[0] == 0
    assert r.split_value[0] == b["split"][0]
    # every threshold between the two groups separates them equally well: the
    # winner must be the one with the highest (bin mod 512), lowest bin inside it
    bin_idx = int(np.searchsorted(r.proposals, np.float32(r.split_value[0])))
    cum_h = np.cumsum(np.bincount(brute.bins_of(Xall, r.proposals, r.row_pointers)[:, 0],
                                  weights=r.quantised[:, 0, 1], minlength=r.n_bins))
    tied = np.nonzero(cum_h == cum_h[bin_idx])[0]
    assert len(tied) > 10
    res = tied % 512
    assert bin_idx == tied[res == res.max()].min()
    if lo_value > 1.0:
        # the tied run crosses bin 512, so the winner is bin 511 and not the last tied bin
        assert tied.min() < 511 < tied.max() and bin_idx == 511


# ----------------------------------------------------------------------------- reference known-answer tests


def _fit_predict(X, g, h, **kw):
    r = orc.build_tree(X, g, h, **kw)
    return r, orc.predict(X, [(r.leaf_value, r.feature, r.split_value)], g.shape[1])


def test_reference_test_basic():
    # legateboost/test/models/test_tree.py:11-21
    X = np.array([[0.0], [1.0]])
    g = np.array([[0.0], [-1.0]])
    h = np.array([[1.0], [1.0]])
    seed = np.random.RandomState(2).randint(0, 2**31)
    r, pred = _fit_predict(X, g, h, max_depth=1, split_samples=256, seed=seed, l2=0.0)
    assert np.allclose(pred, np.array([[0.0], [1.0]]))


def test_reference_l2_and_l1_regularization_closed_forms():
    # test_tree.py:64-78 and :160-184 with init=None, learning_rate=1: g = pred - y = -y, h = 1
    X = np.array([[0.0], [0.0]])
    y = np.array([500.0, 500.0])
    g = -y.reshape(-1, 1)
    h = np.ones((2, 1))
    r, pred = _fit_predict(X, g, h, max_depth=0, split_samples=256, seed=0, l2=10.0)
    assert np.isclose(pred[0, 0], y.sum() / (y.size + 10.0))
    leaf, hess = orc.update_tree(X, g, h, r.feature, r.split_value, 0.0, 10.0)
    assert np.isclose(leaf[0, 0], y.sum() / (y.size + 10.0))
    r, pred = _fit_predict(X, g, h, max_depth=0, split_samples=256, seed=0, l1=1.5, l2=0.0)
    assert np.isclose(pred[0, 0], (y.sum() - 1.5) / y.size)
    leaf, hess = orc.update_tree(X, g, h, r.feature, r.split_value, 1.5, 0.0)
    assert np.isclose(leaf[0, 0], (y.sum() - 1.5) / y.size)
    y = np.array([0.5, 0.5])
    r, pred = _fit_predict(X, -y.reshape(-1, 1), h, max_depth=0, split_samples=256, seed=0, l1=1.5, l2=0.0)
    assert np.isclose(pred[0, 0], 0.0)


def test_reference_min_split_gain():
    # test_tree.py:187-215
    rng = np.random.RandomState(0)
    X = rng.random_sample((100, 1))
    y = rng.random_sample(100)
    g, h = -y.reshape(-1, 1), np.ones((100, 1))
    a = orc.build_tree(X, g, h, max_depth=12, split_samples=256, seed=5, min_split_gain=0.0)
    b = orc.build_tree(X, g, h, max_depth=12, split_samples=256, seed=5, min_split_gain=0.03)
    assert (b.hessian > 0).sum() < (a.hessian > 0).sum()
    assert np.isclose(a.gain[0], b.gain[0] + 0.03)


def test_reference_improving_with_depth_and_sanity():
    # test_tree.py:24-45 and legateboost/testing/utils.py:22-39
    rs = np.random.RandomState(0)
    X = rs.random_sample((2000, 20))
    for k in (1, 5):
        g = rs.normal(size=(2000, k))
        h = rs.random_sample(g.shape) + 0.1
        y = -g / h
        losses = []
        for depth in range(0, 8):
            r, pred = _fit_predict(X, g, h, max_depth=depth, split_samples=256, seed=7)
            losses.append((((pred - y) ** 2 * h).sum(axis=0) / h.sum(axis=0)).mean())
            split_nodes = r.feature != -1
            assert (r.hessian[split_nodes] > 0).all() and (r.gain[split_nodes] > 0).all()
            is_leaf = (r.feature == -1) & (r.hessian[:, 0] > 0)
            assert np.isclose(r.hessian[is_leaf].sum(axis=0), r.hessian[0]).all()
        assert all(b <= a + 1e-12 for a, b in zip(losses, losses[1:]))
        assert losses[-1] < losses[0]


def test_max_depth_20_on_two_rows():
    # test_tree.py:48-61 (must neither blow up memory nor loop)
    X = np.random.RandomState(0).random_sample((2, 1))
    g = np.array([[-500.0], [-500.0]])
    h = np.ones((2, 1))
    r = orc.build_tree(X, g, h, max_depth=20, split_samples=256, seed=0, want_hist=False)
    assert r.feature.shape[0] == 2**21 - 1


# ----------------------------------------------------------------------------- predict / update


def test_predict_bruteforce_and_batch_additivity():
    rs = np.random.RandomState(8)
    X = rs.randn(500, 6).astype(np.float32)
    trees = []
    for t in range(3):
        g = rs.randn(500, 2)
        h = rs.rand(500, 2) + 0.5
        r = orc.build_tree(X, g, h, max_depth=4, split_samples=32, seed=t)
        trees.append((r.leaf_value, r.feature, r.split_value))

    def walk(tree, x):
        leaf, feat, split = tree
        pos = 0
        while feat[pos] != -1:
            pos = 2 * pos + 1 if float(x[feat[pos]]) <= split[pos] else 2 * pos + 2
        return leaf[pos]

    single = [orc.predict(X, [t], 2) for t in trees]
    for t, p in zip(trees, single):
        want = np.stack([walk(t, X[i]) for i in range(500)])
        assert np.array_equal(p, want)
    # test_model.py:8-21: batch == sum of singles (same addition order => exact)
    assert np.array_equal(orc.predict(X, trees, 2), (single[0] + single[1]) + single[2])


def test_update_after_fit_reproduces_fit():
    # test_estimator.py:60-65 at the task boundary: exact double sums vs quantised sums
    rs = np.random.RandomState(12)
    X = rs.randn(4000, 5).astype(np.float32)
    g = rs.randn(4000, 1)
    h = rs.rand(4000, 1) + 0.5
    r = orc.build_tree(X, g, h, max_depth=4, split_samples=64, seed=4)
    leaf, hess = orc.update_tree(X, g, h, r.feature, r.split_value, 0.0, 1.0)
    used = r.hessian[:, 0] > 0
    assert np.allclose(leaf[used], r.leaf_value[used], rtol=1e-4, atol=1e-6)
    assert np.allclose(hess[used], r.hessian[used], rtol=1e-5)
    assert (leaf[~used] == 0).all()


# ---- the boosting round's steps around the tree build ----------------------------------------


def test_reference_log_loss_known_answers():
    # legateboost/test/test_objective.py::test_log_loss gives gradient() probabilities; the raw
    # predictions that transform() maps to them are their logits / logarithms
    g, h = orc.weighted_gradient("log_loss", np.array([[1.0], [0.0]]), np.zeros((2, 1)))
    assert np.allclose(g, [[-0.5], [0.5]]) and np.allclose(h, [[0.25], [0.25]])
    prob = np.array([[0.3, 0.3, 0.4], [0.3, 0.4, 0.3], [0.4, 0.3, 0.3]])
    g, h = orc.weighted_gradient("log_loss", np.array([2.0, 1.0, 0.0]), np.log(prob) + 7.0)
    assert np.allclose(g, [[0.3, 0.3, -0.6], [0.3, -0.6, 0.3], [-0.6, 0.3, 0.3]])
    assert np.allclose(h, [[0.21, 0.21, 0.24], [0.21, 0.24, 0.21], [0.24, 0.21, 0.21]])


def test_weighted_gradient_against_the_reference_operator_sequence():
    # legateboost.py:205-211 spelt out with numpy, operator by operator
    rs = np.random.RandomState(11)
    n = 257
    w = rs.gamma(2.0, size=n)
    w[:5] = [0.0, 1e-12, 1.0, 3.0, 1e6]
    lr = 0.3
    for k in (1, 3):
        pred, y = rs.normal(size=(n, k)), rs.normal(size=(n, k))
        g, h = orc.weighted_gradient("squared_error", y, pred, w, lr)
        assert np.array_equal(g, (pred - y) * w[:, None] * lr)
        assert np.array_equal(h, np.maximum(np.ones((n, k)) * w[:, None], 1e-8))
        g, h = orc.weighted_gradient("squared_error", y, pred, None, lr)
        assert np.array_equal(g, (pred - y) * 1.0 * lr) and np.array_equal(h, np.ones((n, k)))
    pred, y = 4 * rs.normal(size=(n, 1)), rs.randint(0, 2, (n, 1)).astype(np.float64)
    p = 1.0 / (1.0 + np.exp(-pred))
    g, h = orc.weighted_gradient("log_loss", y, pred, w, lr)
    assert np.allclose(g, (p - y) * w[:, None] * lr, rtol=1e-13, atol=0)
    assert np.allclose(h, np.maximum(p * (1 - p) * w[:, None], 1e-8), rtol=1e-13, atol=0)
    assert h.min() == 1e-8  # the zero-weight rows sit on the floor
    k = 5
    pred, lab = 6 * rs.normal(size=(n, k)), rs.randint(0, k, n)
    pred[7] = [800.0, -800.0, 0.0, 799.0, 1.0]  # no overflow thanks to the row maximum
    e = np.exp(pred - pred.max(axis=1)[:, None])
    p = e / e.sum(axis=1)[:, None]
    gg = p.copy()
    gg[np.arange(n), lab] -= 1.0
    g, h = orc.weighted_gradient("log_loss", lab.astype(np.float64), pred, w, lr)
    assert np.allclose(g, gg * w[:, None] * lr, rtol=1e-12, atol=1e-300)
    assert np.allclose(h, np.maximum(p * (1 - p) * w[:, None], 1e-8), rtol=1e-12, atol=0)
    assert np.isfinite(g).all() and np.isfinite(h).all()
    # the class gradients of a row sum to zero, its hessians are those of a probability vector
    g1, h1 = orc.weighted_gradient("log_loss", lab.astype(np.float64), pred)
    assert np.abs(g1.sum(axis=1)).max() < 1e-15 and (h1 <= 0.25 + 1e-16).all()


def test_add_leaf_values_and_gather_rows_are_plain_indexing():
    rs = np.random.RandomState(5)
    leaf = rs.normal(size=(31, 3))
    row_leaf = rs.randint(0, 31, 500).astype(np.int32)
    pred = rs.normal(size=(500, 3))
    assert np.array_equal(orc.add_leaf_values(pred, leaf, row_leaf), pred + leaf[row_leaf])
    for dt in (np.float32, np.float64):
        X = rs.normal(size=(40, 7)).astype(dt)
        rows = np.array([100, 139, 99, 140, 120, 120, -1], np.int64)
        want = np.zeros((7, 7), dt)
        want[[0, 1, 4, 5]] = X[[0, 39, 20, 20]]
        assert np.array_equal(orc.gather_rows(X, rows, row_offset=100), want)


def test_row_leaf_update_equals_predict():
    # what the fused update relies on: leaf[row -> leaf] is PredictTask on the training rows
    rs = np.random.RandomState(2)
    X = rs.normal(size=(300, 6)).astype(np.float32)
    g, h = rs.normal(size=(300, 2)), np.ones((300, 2))
    t = orc.build_tree(X, g, h, max_depth=4, split_samples=16, seed=9)
    pr = orc.predict(X, [(t.leaf_value, t.feature, t.split_value)], 2)
    walk = np.zeros(300, np.int32)
    for r in range(300):
        nd = 0
        while t.feature[nd] != -1:
            nd = 2 * nd + 1 if X[r, t.feature[nd]] <= t.split_value[nd] else 2 * nd + 2
        walk[r] = nd
    assert np.array_equal(orc.add_leaf_values(np.zeros((300, 2)), t.leaf_value, walk), pr)


def test_the_four_stage_functions_chain_to_the_whole_build():
    """orc_histogram_level, orc_scan, orc_best_split and orc_update_positions are the loop body of
    orc_build_tree (pinned above by brute force); driven one by one from Python, with a histogram
    buffer that is re-allocated for the last level as GetHistogram (build_tree.cu:1191-1205) does,
    they must give the same tree, histograms and positions."""
    rs = np.random.RandomState(8)
    n, f, k, depth, s, seed = 4000, 6, 2, 4, 32, 5
    X = rs.normal(size=(n, f)).astype(np.float32)
    g = rs.normal(size=(n, k))
    h = np.abs(rs.normal(size=(n, k))) + 0.1
    props, rp = orc.split_proposals(X, seed, s)
    B = int(rp[-1])
    cache_nodes = 8  # levels 0..2 share a buffer of 7 nodes, level 3 (8 nodes) gets its own
    whole = orc.build_tree(X, g, h, max_depth=depth, split_samples=s, seed=seed, hist_cache_bytes=cache_nodes * k * B * 16)
    assert (whole.hist_node_begin, whole.hist_node_end) == (7, 15)
    sc = orc.scales(orc.abs_sums(g, h))
    q = orc.quantise_all(g, h, seed, sc)
    max_nodes = 2 ** (depth + 1) - 1
    sums = np.zeros((max_nodes, k, 2), np.int64)
    sums[0] = q.sum(axis=0)
    leaf = np.zeros((max_nodes, k))
    feature = -np.ones(max_nodes, np.int32)
    split = np.zeros(max_nodes)
    gain = np.zeros(max_nodes)
    pos = np.stack([np.zeros(n, np.int32), np.arange(n, dtype=np.int32)], axis=1).copy()
    hist_nodes = (0, 7)
    hist = np.zeros((7, k, B, 2), np.int64)
    for level in range(depth):
        batch = (2 ** level - 1, 2 ** (level + 1) - 1)
        if batch[1] > hist_nodes[1]:
            hist_nodes = batch
            hist = np.zeros((batch[1] - batch[0], k, B, 2), np.int64)
        assert np.array_equal(pos, whole.positions_per_level[level]) if whole.positions_per_level is not None else True
        orc.histogram_level(X, q, props, rp, pos, batch, sums, hist_nodes, hist)
        orc.scan(hist, hist_nodes, rp, sums, batch)
        orc.best_split(hist, hist_nodes, props, rp, sums, sc, batch, leaf, feature, split, gain)
        if level < depth - 1:
            orc.update_positions(X, pos, feature, split, max_nodes)
    assert np.array_equal(feature, whole.feature) and (feature != -1).sum() >= 8
    assert np.array_equal(split, whole.split_value) and np.array_equal(gain, whole.gain)
    assert np.array_equal(sums, whole.node_sums)
    assert np.array_equal(leaf[1:], whole.leaf_value[1:])
    assert np.array_equal(pos, whole.positions)
    assert np.array_equal(hist, whole.histogram)
    # a batch that is a part of a level adds the same bins as the level in one piece
    both = np.zeros((8, k, B, 2), np.int64)
    orc.histogram_level(X, q, props, rp, pos, (7, 11), sums, (7, 15), both)
    orc.histogram_level(X, q, props, rp, pos, (11, 15), sums, (7, 15), both)
    raw = np.zeros((8, k, B, 2), np.int64)
    orc.histogram_level(X, q, props, rp, pos, (7, 15), sums, (7, 15), raw)
    assert np.array_equal(both, raw)
    # every row of every output lands once per feature
    per_feature = np.add.reduceat(raw, rp[:-1], axis=2)  # [node][k][feature][2]
    for j in range(8):
        rows = pos[pos[:, 0] == 7 + j, 1]
        want = q[rows].sum(axis=0)  # [k][2]
        assert np.array_equal(per_feature[j], np.repeat(want[:, None, :], f, axis=1))
