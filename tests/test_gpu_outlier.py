"""One gradient far above the others: the packed 32-bit sub-histograms of the histogram kernel then
fill up after a tile or two, so a workgroup hands the bins of one node over in several parts. At
4,000,000 x 36 there are more parts in a launch than slots to park them in (the rest is added with
global atomics while the launch runs), and at the deep levels many nodes lie wholly inside one
workgroup's rows. The sums of such a node must come out whole whichever way its parts travelled:
checked bit for bit against the CPU oracle and through the exact integer identities of the
histograms."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(n, f, share):
    """X ~ N(0,1), squared-error-like gradients with one entry that holds `share` of the sum of |g|."""
    rs = np.random.RandomState(31)
    X = rs.normal(size=(n, f)).astype(np.float32)
    g = rs.normal(size=(n, 1)) * 0.1 + 0.05 * X[:, :1]
    g[n // 3, 0] = 0.0
    g[n // 3, 0] = np.abs(g).sum() * share / (1.0 - share)
    h = np.ones((n, 1))
    return X, g, h


def test_outlier_gradient_bit_exact_against_the_oracle():
    import gpu_util as gu

    n, f, depth = 4_000_000, 36, 10
    # a tile of the histogram kernel is 1364 rows here (three 16-byte lanes per row, four rows per
    # lane); with max |q| = 2^31 / 2000 one tile fits the packed sums and two do not
    X, g, h = _inputs(n, f, 1.0 / 2000.0)
    gr, cr = gu.both(X, g, h, max_depth=depth, split_samples=256, seed=77)
    q = np.abs(cr.quantised).max()
    assert 1364 * q <= 2**31 - 1 < 2 * 1364 * q
    gu.assert_tree_parity(gr, cr)
    assert (cr.feature != -1).sum() > 500
    # every scanned feature of every node that holds rows ends in the node's sums
    rp = cr.row_pointers
    last = torch.as_tensor(rp[1:] - 1, device=gr.histogram.device, dtype=torch.long)
    ends = gr.histogram[:, 0, last, :]
    sums = gr.node_sums[gr.hist_node_begin: gr.hist_node_end, 0, :]
    reached = sums[:, 1] > 0
    assert int(reached.sum()) > 500
    assert torch.equal(ends[reached], sums[reached].unsqueeze(1).expand(-1, f, -1))


def test_outlier_gradient_two_feature_groups():
    """The same at 100 features (two feature groups, tiles of 1024 rows), where the oracle would take
    minutes: the integer identities alone."""
    from lbtree import ops

    n, f, depth = 3_000_000, 100, 10
    X, g, h = _inputs(n, f, 1.0 / 1500.0)
    r = ops.build_tree(X, g, h, max_depth=depth, split_samples=256, seed=78, taps=True)
    torch.cuda.synchronize()
    q = int(r.quantised.abs().max())
    assert 1024 * q <= 2**31 - 1 < 2 * 1024 * q
    feature = r.feature.cpu().numpy()
    sums = r.node_sums.cpu().numpy()
    split = np.flatnonzero(feature >= 0)
    assert len(split) > 500
    assert np.array_equal(sums[2 * split + 1] + sums[2 * split + 2], sums[split])
    assert np.array_equal(r.quantised.to(torch.int64).sum(dim=0).cpu().numpy(), sums[0])
    rp = r.row_pointers.cpu().numpy()
    last = torch.as_tensor(rp[1:] - 1, device=X.device if isinstance(X, torch.Tensor) else r.histogram.device,
                           dtype=torch.long)
    ends = r.histogram[:, 0, last, :]
    node_sums = r.node_sums[r.hist_node_begin: r.hist_node_end, 0, :]
    reached = node_sums[:, 1] > 0
    assert torch.equal(ends[reached], node_sums[reached].unsqueeze(1).expand(-1, f, -1))
