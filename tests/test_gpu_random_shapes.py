"""Seeded random shapes and input kinds for every op against the oracle: sizes on either
side of the launch choices (1, 2, 63..65, 511..513, 1024, 2049, ... 20000 points), clouds
that are uniform, on a lattice (exact ties), on a sphere, clustered, scaled by 1e-8..1e8,
offset from the origin or on a line. Distances, indices and slot orders must be
bit-identical; fp32 scatters within 1e-5 relative / 1e-6 absolute of sums taken in double."""
import numpy as np
import pytest
import torch

import oracle
from util import gaussian_mixture_cloud, lattice_cloud, sphere_cloud, uniform_cloud

pytestmark = pytest.mark.gpu
SIZES = [1, 2, 3, 31, 64, 65, 200, 511, 512, 513, 1000, 1024, 1500, 2048, 2049, 3000, 4096, 5000,
         8192, 9000, 16384, 20000]


def _cloud(rng, g, b, n):
    kind = rng.choice(["uniform", "lattice", "sphere", "mixture", "scaled", "offset", "line"])
    if kind == "uniform":
        return uniform_cloud(g, b, n)
    if kind == "lattice":
        return lattice_cloud(g, b, n, int(rng.choice([2, 4, 8, 16])))
    if kind == "sphere":
        return sphere_cloud(g, b, n)
    if kind == "mixture":
        return gaussian_mixture_cloud(g, b, n)
    if kind == "scaled":
        return uniform_cloud(g, b, n) * float(10.0 ** rng.integers(-8, 9))
    if kind == "offset":
        return uniform_cloud(g, b, n) + float(rng.choice([10.0, 1000.0, -300.0]))
    t = torch.rand(b, n, 1, generator=g)
    return t * torch.tensor([1.0, 2.0, -0.5]) + 1e-3 * uniform_cloud(g, b, n)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_distance_ops_on_random_shapes(cuda, seed):
    from torkit3d_amd import _C

    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    done = 0
    while done < 60:
        op = rng.choice(["chamfer", "knn", "ball", "fps"])
        b, n1, n2 = int(rng.integers(1, 5)), int(rng.choice(SIZES)), int(rng.choice(SIZES))
        if b * n1 * n2 > 2e8:
            continue
        if op == "chamfer":
            a, c = _cloud(rng, g, b, n1), _cloud(rng, g, b, n2)
            got = _C.chamfer_distance_forward_cuda(a.to(cuda), c.to(cuda))
            want = oracle.chamfer_forward(a.numpy(), c.numpy())
            ok = all(np.array_equal(x.cpu().numpy(), y) for x, y in zip(got, want))
            case = (op, b, n1, n2)
        elif op == "knn":
            k = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 17, 20, 32, 40, 64, 100]))
            if k > n2:
                continue
            q, key = _cloud(rng, g, b, n1), _cloud(rng, g, b, n2)
            d, i = _C.knn_distance_cuda(q.to(cuda), key.to(cuda), k, 1)
            od, oi = oracle.knn(q.numpy(), key.numpy(), k)
            ok = np.array_equal(d.cpu().numpy(), od) and np.array_equal(i.cpu().numpy(), oi)
            case = (op, b, n1, n2, k)
        elif op == "ball":
            k = int(rng.choice([1, 4, 16, 32, 64, 100]))
            r = float(rng.choice([0.01, 0.1, 0.2, 0.5, 3.0]))
            key = _cloud(rng, g, b, n2)
            q = _cloud(rng, g, b, n1) if rng.random() < 0.5 else \
                key[:, torch.randint(0, n2, (n1,), generator=g)].contiguous()
            got = _C.ball_query_cuda(q.to(cuda), key.to(cuda), r, k).cpu().numpy()
            ok = np.array_equal(got, oracle.ball_query(q.numpy(), key.numpy(), r, k))
            case = (op, b, n1, n2, r, k)
        else:
            m = int(rng.integers(1, min(n1, 1500) + 1))
            pts = _cloud(rng, g, b, n1)
            got = _C.sample_farthest_points_cuda(pts.to(cuda), m).cpu().numpy()
            ok = np.array_equal(got, oracle.sample_farthest_points(pts.numpy(), m))
            case = (op, b, n1, m)
        assert ok, case
        done += 1


@pytest.mark.parametrize("seed", [21, 22])
def test_feature_ops_on_random_shapes(cuda, seed):
    from torkit3d_amd import _C

    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(40):
        b, c = int(rng.integers(1, 6)), int(rng.integers(1, 41))
        n1 = int(rng.choice([1, 2, 7, 64, 300, 1000, 2048, 2250, 2300, 4096, 4161, 5000, 9000,
                             16000, 16384, 16500, 20000]))
        n2 = int(rng.choice([1, 5, 63, 64, 65, 127, 129, 500, 1000, 3000, 8192, 20000]))
        weighted = bool(rng.integers(0, 2))
        k = 3 if weighted else int(rng.choice([1, 4, 16]))
        index = torch.randint(0, n1, (b, n2, k), generator=g)
        if rng.random() < 0.5:  # some indices outside the row: they contribute nothing
            out_of_row = torch.rand(b, n2, k, generator=g) < 0.05
            index[out_of_row] = -1 if rng.random() < 0.5 else n1 + 3
        feat = torch.randn(b, c, n1, generator=g)
        scale = float(10.0 ** rng.integers(-6, 7))
        shape = (b, c, n2) if weighted else (b, c, n2, k)
        go = torch.randn(*shape, generator=g) * scale
        if rng.random() < 0.3:  # a term far above the others in one row
            flat = go.view(b, c, -1)
            flat[rng.integers(0, b), rng.integers(0, c), rng.integers(0, flat.shape[2])] = 1e4 * scale
        case = (b, c, n1, n2, k, weighted, scale)
        if weighted:
            w = torch.rand(b, n2, k, generator=g)
            out = _C.interpolate_forward_cuda(feat.to(cuda), index.to(cuda), w.to(cuda))
            want = oracle.interpolate_forward(feat.numpy(), index.numpy(), w.numpy())
            gin = _C.interpolate_backward_cuda(go.to(cuda), index.to(cuda), w.to(cuda), n1)
            gw = oracle.interpolate_backward(go.numpy(), index.numpy(), w.numpy(), n1, wide=True)
        else:
            out = _C.group_points_forward_cuda(feat.to(cuda), index.to(cuda))
            want = oracle.group_forward(feat.numpy(), index.numpy())
            gin = _C.group_points_backward_cuda(go.to(cuda), index.to(cuda), n1)
            gw = oracle.group_backward(go.numpy(), index.numpy(), n1, wide=True)
        assert np.array_equal(out.cpu().numpy(), want), case
        # a row is resolved to 2^-38 of its largest term; where few jobs make the kernel split
        # the points, partial sums (each rounded to fp32) meet in float atomics: a few units
        # in the last place of the sum of the terms' magnitudes
        rowmax = np.abs(go.view(b, c, -1).numpy()).max(axis=2, keepdims=True)
        tol = 1e-5 * np.abs(gw) + 1e-6 * scale + rowmax * 2.0 ** -38
        if b * ((c + 3) // 4) < 128:
            if weighted:
                mag = oracle.interpolate_backward(go.abs().numpy(), index.numpy(), w.numpy(), n1, wide=True)
            else:
                mag = oracle.group_backward(go.abs().numpy(), index.numpy(), n1, wide=True)
            tol = tol + mag * 2.0 ** -21
        assert (np.abs(gin.cpu().numpy() - gw) <= tol).all(), case
