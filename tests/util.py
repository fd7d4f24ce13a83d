"""Shared helpers for the parity tests: seeded inputs of the benchmark configurations
and small numpy restatements used to pin the oracle."""
import numpy as np
import torch


def uniform_cloud(gen, b, n, lo=-1.0, hi=1.0, dtype=torch.float32):
    return torch.rand(b, n, 3, generator=gen, dtype=dtype) * (hi - lo) + lo


def gaussian_mixture_cloud(gen, b, n, k=8, sigma=0.1):
    """Mixture of k isotropic Gaussians, centres uniform in [-1,1]^3 (FPS config)."""
    centres = torch.rand(b, k, 3, generator=gen) * 2 - 1
    comp = torch.randint(0, k, (b, n), generator=gen)
    pts = torch.gather(centres, 1, comp[:, :, None].expand(-1, -1, 3))
    return pts + sigma * torch.randn(b, n, 3, generator=gen)


def sphere_cloud(gen, b, n, noise=0.01):
    """Points on the unit sphere plus N(0, noise^2) (stress config)."""
    u = torch.randn(b, n, 3, generator=gen)
    return u / u.norm(dim=2, keepdim=True) + noise * torch.randn(b, n, 3, generator=gen)


def lattice_cloud(gen, b, n, steps=8, dtype=torch.float32):
    """Coordinates m/steps, m integer, steps a power of two: all differences, squares
    and three-term sums are exact in fp32, fused or not, and exact ties are frequent."""
    return (torch.randint(0, steps + 1, (b, n, 3), generator=gen).to(dtype)) / steps


def pairwise_d2_f64(a, b):
    """[B,N1,N2] squared distances in float64 (numpy), a:[B,N1,3], b:[B,N2,3]."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    diff = a[:, :, None, :] - b[:, None, :, :]
    return (diff * diff).sum(-1)


def ball_query_numpy(query, key, radius, k):
    """nonzero(d2 < r^2)[:k] + pad-with-first, the reference's test oracle
    (tests/ops/test_ball_query.py:15-40); rows without a hit stay -1. Arithmetic in
    the dtype of the inputs, un-fused."""
    b, n1, _ = query.shape
    out = np.full((b, n1, k), -1, np.int64)
    r = query.dtype.type(np.float32(radius))
    r2 = r * r
    for bi in range(b):
        for i in range(n1):
            d = key[bi] - query[bi, i][None, :]
            d2 = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
            hits = np.nonzero(d2 < r2)[0]
            if hits.size == 0:
                continue
            m = min(hits.size, k)
            out[bi, i, :m] = hits[:m]
            out[bi, i, m:] = hits[0]
    return out


def fps_numpy(points, k):
    """Running minimum + argmax, the reference's test oracle
    (tests/ops/test_sample_farthest_points.py:27-36)."""
    out = []
    for p in points:
        idx, cur, dist = [0], 0, None
        for _ in range(1, k):
            d = p - p[cur][None, :]
            d2 = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
            dist = d2 if dist is None else np.minimum(d2, dist)
            cur = int(np.argmax(dist))
            idx.append(cur)
        out.append(idx)
    return np.asarray(out, np.int64)


def sorted_pairs(dist, idx):
    """Rows of (distance, index) sorted by distance then index."""
    order = np.lexsort((idx, dist), axis=-1)
    return np.take_along_axis(dist, order, -1), np.take_along_axis(idx, order, -1)
