"""Seeded synthetic inputs of the benchmark configurations. Large matrices are
generated on the device (torch is only the random source and the allocator)."""
import numpy as np
import torch


def config1(device="cuda"):
    """100000x32 f32 U[0,1); y = sum_j<4 sin(2 pi x_j) + N(0, 0.1^2); numpy RandomState(0)."""
    rs = np.random.RandomState(0)
    X = rs.random_sample((100000, 32)).astype(np.float32)
    y = np.sin(2 * np.pi * X[:, :4].astype(np.float64)).sum(axis=1) + rs.normal(0, 0.1, 100000)
    return X, y


def config2(n_rows=10_000_000, n_features=100, device="cuda", seed=0):
    """f32 matrix, first half of the columns U[0,1), second half N(0,1); y is a linear
    combination of 10 random columns plus a depth-3 interaction plus N(0, 0.5^2)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    half = n_features // 2
    X = torch.empty((n_rows, n_features), dtype=torch.float32, device=device)
    chunk = 1_000_000
    for lo in range(0, n_rows, chunk):
        hi = min(n_rows, lo + chunk)
        X[lo:hi, :half] = torch.rand((hi - lo, half), generator=gen, device=device)
        X[lo:hi, half:] = torch.randn((hi - lo, n_features - half), generator=gen, device=device)
    rs = np.random.RandomState(seed)
    idx = rs.choice(n_features, min(10, n_features), replace=False)
    w = rs.normal(size=len(idx))
    y = (X[:, torch.as_tensor(idx, device=device)].to(torch.float64) * torch.as_tensor(w, device=device)).sum(dim=1)
    a, b, c = 0, half, min(1, half - 1)
    inter = ((X[:, a] > 0.5) & (X[:, b] > 0.0) & (X[:, c] < 0.3)).to(torch.float64) * 2.0
    y = y + inter + 0.5 * torch.randn(n_rows, generator=gen, device=device, dtype=torch.float64)
    return X, y


def config3(n_rows=2_000_000, n_features=200, n_classes=8, device="cuda", seed=0):
    """f32 N(0,1) matrix; labels = argmax of 8 random projections + Gumbel noise."""
    gen = torch.Generator(device=device).manual_seed(seed)
    X = torch.randn((n_rows, n_features), generator=gen, device=device)
    P = torch.randn((n_features, n_classes), generator=gen, device=device)
    u = torch.rand((n_rows, n_classes), generator=gen, device=device).clamp_(1e-12, 1 - 1e-7)
    gumbel = -torch.log(-torch.log(u))
    y = torch.argmax(X @ P / np.sqrt(n_features) * 3.0 + gumbel, dim=1).to(torch.float64)
    return X, y


def config4(n_rows=1_000_000, n_features=50, device="cuda", seed=0):
    """lognormal(0,1.5) features, 30% of the columns integer with <= 16 levels;
    y piecewise constant in 6 features + N(0, 0.2^2)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    X = torch.exp(1.5 * torch.randn((n_rows, n_features), generator=gen, device=device))
    n_int = int(round(0.3 * n_features))
    X[:, :n_int] = torch.randint(0, 16, (n_rows, n_int), generator=gen, device=device).to(torch.float32)
    y = torch.zeros(n_rows, dtype=torch.float64, device=device)
    cols = [0, 1, n_int, n_int + 1, n_int + 2, n_features - 1]
    thr = [7.0, 3.0, 1.0, 2.5, 0.4, 1.0]
    for i, (cidx, t) in enumerate(zip(cols, thr)):
        y = y + (X[:, cidx] > t).to(torch.float64) * (1.0 + 0.5 * i)
    y = y + 0.2 * torch.randn(n_rows, generator=gen, device=device, dtype=torch.float64)
    return X, y


def config5_ensemble(n_trees=1000, depth=8, n_features=64, device="cuda", seed=0):
    """Complete depth-`depth` trees: split features U{0..n_features-1}, thresholds U[0,1),
    leaf values N(0, 0.01^2) f64. Returns a list of (leaf, feature, split) CUDA tensors."""
    rs = np.random.RandomState(seed)
    n_nodes = 2 ** (depth + 1) - 1
    n_internal = 2 ** depth - 1
    trees = []
    for _ in range(n_trees):
        feature = -np.ones(n_nodes, np.int32)
        feature[:n_internal] = rs.randint(0, n_features, n_internal)
        split = np.zeros(n_nodes)
        split[:n_internal] = rs.random_sample(n_internal)
        leaf = np.zeros((n_nodes, 1))
        leaf[n_internal:, 0] = rs.normal(0, 0.01, n_nodes - n_internal)
        trees.append((torch.from_numpy(leaf).to(device), torch.from_numpy(feature).to(device),
                      torch.from_numpy(split).to(device)))
    return trees


def config5_X(n_rows=20_000_000, n_features=64, device="cuda", seed=0):
    gen = torch.Generator(device=device).manual_seed(seed)
    return torch.rand((n_rows, n_features), generator=gen, device=device)
