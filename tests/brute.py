"""Independent brute-force restatement (numpy, boolean masks, no sorted
positions, no subtraction trick) of one tree build from already-quantised
gradients. Used to pin the oracle on small inputs."""
import numpy as np

EPS = 1e-5


def leaf_gain(G, H, l1, reg):
    z = np.where(G > l1, G - l1, np.where(G < -l1, G + l1, 0.0))
    return (z * z) / (H + reg)


def leaf_value(G, H, l1, l2):
    z = G - l1 if G > l1 else (G + l1 if G < -l1 else 0.0)
    return -z / (H + l2)


def bins_of(X, proposals, rp):
    n, f = X.shape
    out = np.empty((n, f), np.int64)
    for j in range(f):
        p = proposals[rp[j]:rp[j + 1]]
        out[:, j] = rp[j] + np.searchsorted(p, X[:, j], side="left")
    return out


def build(X, q, proposals, rp, scales, max_depth, l1, l2, msg, feature_set=None):
    """q: int64 [n,k,2]. Returns dict(feature, split, gain, leaf, node_sums, node_of_row)."""
    n, f = X.shape
    k = q.shape[1]
    B = len(proposals)
    max_nodes = 2 ** (max_depth + 1) - 1
    feature = -np.ones(max_nodes, np.int32)
    split = np.zeros(max_nodes)
    gain = np.zeros(max_nodes)
    leaf = np.zeros((max_nodes, k))
    sums = np.zeros((max_nodes, k, 2), np.int64)
    bins = bins_of(X, proposals, rp)
    feat_of_bin = np.searchsorted(rp, np.arange(B), side="right") - 1
    node_of_row = np.zeros(n, np.int64)
    sums[0] = q.sum(axis=0)
    inv_g, inv_h = scales[2], scales[3]
    for j in range(k):
        leaf[0, j] = leaf_value(sums[0, j, 0] * inv_g, sums[0, j, 1] * inv_h, l1, l2)
    reg = max(EPS, l2)
    for depth in range(max_depth):
        for node in range(2 ** depth - 1, 2 ** (depth + 1) - 1):
            if sums[node, 0, 1] <= 0:
                continue
            rows = np.nonzero(node_of_row == node)[0]
            hist = np.zeros((k, B, 2), np.int64)
            for j in range(f):
                for kk in range(k):
                    np.add.at(hist[kk, :, 0], bins[rows, j], q[rows, kk, 0])
                    np.add.at(hist[kk, :, 1], bins[rows, j], q[rows, kk, 1])
            cum = np.zeros_like(hist)
            for j in range(f):
                cum[:, rp[j]:rp[j + 1]] = np.cumsum(hist[:, rp[j]:rp[j + 1]], axis=1)
            tot = np.zeros(B)
            dead = np.zeros(B, bool)
            for kk in range(k):  # outputs added in order, like the reference's loop
                L = cum[kk]
                P = sums[node, kk]
                R = P[None, :] - L
                bad = (L[:, 1] <= 0) | (R[:, 1] <= 0)
                # the reference stops at the first bad output and zeroes the gain
                dead |= bad
                gk = 0.5 * (leaf_gain(L[:, 0] * inv_g, L[:, 1] * inv_h, l1, reg)
                            + leaf_gain(R[:, 0] * inv_g, R[:, 1] * inv_h, l1, reg)
                            - leaf_gain(P[0] * inv_g, P[1] * inv_h, l1, reg)) - msg
                with np.errstate(invalid="ignore"):
                    tot = tot + np.where(dead, 0.0, gk)
            tot = np.where(dead, 0.0, tot)
            if feature_set is not None:
                tot = np.where(np.asarray(feature_set, bool)[feat_of_bin], tot, -np.inf)
            cand = np.nonzero(tot > 0)[0]
            if len(cand) == 0:
                continue
            best = tot[cand].max()
            if not best > EPS:
                continue
            c = cand[tot[cand] == best]
            # tie rule: highest (bin mod 512); inside that residue class the lowest bin
            res = c % 512
            c = c[res == res.max()]
            b = c.min()
            feature[node] = feat_of_bin[b]
            split[node] = float(proposals[b])
            gain[node] = best
            lc, rc = 2 * node + 1, 2 * node + 2
            sums[lc] = cum[:, b]
            sums[rc] = sums[node] - cum[:, b]
            for kk in range(k):
                leaf[lc, kk] = leaf_value(sums[lc, kk, 0] * inv_g, sums[lc, kk, 1] * inv_h, l1, l2)
                leaf[rc, kk] = leaf_value(sums[rc, kk, 0] * inv_g, sums[rc, kk, 1] * inv_h, l1, l2)
            go_left = X[rows, feature[node]].astype(np.float64) <= split[node]
            node_of_row[rows] = np.where(go_left, lc, rc)
    return dict(feature=feature, split=split, gain=gain, leaf=leaf, node_sums=sums, node_of_row=node_of_row)
