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


# ---- a MinK run worked out by hand ------------------------------------------------------
# mink.cuh:61-89 of the reference, k = 3, one query at the origin, keys on the x axis so
# that the squared distance of key j is MINK_X[j]**2 (all exact in binary):
#
#   j   x     d      what MinK::add does                              slots (d, j) afterwards
#   0   2     4      fill slot 0; first key: max = 4 in slot 0        (4,0)
#   1  -2     4      fill slot 1; 4 > 4 is false: max stays slot 0    (4,0) (4,1)
#   2   3     9      fill slot 2; 9 > 4: max = 9 in slot 2            (4,0) (4,1) (9,2)
#   3  -3     9      9 < 9 is false: rejected (a key equal to the     unchanged
#                    maximum never enters)
#   4   1     1      1 < 9: overwrite slot 2; rescan from max = 1:    (4,0) (4,1) (1,4)
#                    slot 0: 4 > 1 -> max 4, slot 0; slot 1: 4 > 4
#                    false -> of two equal maxima the LOWER slot is
#                    the next victim
#   5   2     4      4 < 4 is false: rejected                         unchanged
#   6   1.5   2.25   2.25 < 4: overwrite slot 0; rescan from 2.25:    (2.25,6) (4,1) (1,4)
#                    slot 1: 4 > 2.25 -> max 4, slot 1
#   7  -1.5   2.25   2.25 < 4: overwrite slot 1; rescan from 2.25:    (2.25,6) (2.25,7) (1,4)
#                    slot 0: 2.25 > 2.25 false -> the slot just
#                    written stays the victim although the lower
#                    slot 0 holds an equal key
#   8   0.5   0.25   0.25 < 2.25: overwrite slot 1 (not slot 0);      (2.25,6) (0.25,8) (1,4)
#                    rescan: slot 0: 2.25 > 0.25 -> max 2.25, slot 0
#   9   0     0      0 < 2.25: overwrite slot 0; rescan: slot 1:      (0,9) (0.25,8) (1,4)
#                    0.25 > 0 -> slot 1; slot 2: 1 > 0.25 -> slot 2
#
# MINK_STATES[m] is the (distance, index) row after the first m keys. Reading the rescan as
# '>=' changes the row at m = 8, starting the rescan from "no maximum" instead of the
# written slot changes it at m = 9, accepting a key equal to the maximum changes it at
# m = 4 and m = 6.
MINK_X = [2.0, -2.0, 3.0, -3.0, 1.0, 2.0, 1.5, -1.5, 0.5, 0.0]
MINK_STATES = {
    3: ([4.0, 4.0, 9.0], [0, 1, 2]),
    4: ([4.0, 4.0, 9.0], [0, 1, 2]),
    5: ([4.0, 4.0, 1.0], [0, 1, 4]),
    6: ([4.0, 4.0, 1.0], [0, 1, 4]),
    7: ([2.25, 4.0, 1.0], [6, 1, 4]),
    8: ([2.25, 2.25, 1.0], [6, 7, 4]),
    9: ([2.25, 0.25, 1.0], [6, 8, 4]),
    10: ([0.0, 0.25, 1.0], [9, 8, 4]),
}
MINK_NEAR = 2.0 ** -6  # |x| of the keys that pad the run to k > 3; its square is 2^-12


def mink_worked_example(m, k=3, dtype=np.float32):
    """Keys [1,k-3+m,3] and the expected (distance [k], index [k]) row for a query at the
    origin. For k > 3 the run above is preceded by k-3 keys at distance 2^-12: they fill
    slots 0..k-4 and, being smaller than every later maximum (the rescan's strict '>' never
    selects them while a larger key is stored), stay there, so the last three slots go
    through exactly the states of the table with every index shifted by k-3."""
    pad = k - 3
    xs = [MINK_NEAR if i % 2 == 0 else -MINK_NEAR for i in range(pad)] + MINK_X[:m]
    key = np.zeros((1, len(xs), 3), dtype)
    key[0, :, 0] = xs
    d, i = MINK_STATES[m]
    dist = np.asarray([MINK_NEAR ** 2] * pad + d, dtype)
    idx = np.asarray(list(range(pad)) + [j + pad for j in i], np.int64)
    return key, dist, idx
