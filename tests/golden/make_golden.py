"""Generate ``tests/golden/tk3d_small.npz``: small known-answer vectors for all six ops.

The expected outputs come from the pure-Python restatement below, which shares no
code with ``oracle/`` or with the HIP kernels. fp32 arithmetic is emulated exactly
with rationals: every operation is evaluated in exact arithmetic and rounded once
to the nearest float32 (ties to even), so a fused multiply-add is a single
rounding of a*b+c, exactly as the hardware instruction. This pins the canonical
distance  fma(dz,dz, fma(dy,dy, dx*dx))  (the value the reference kernels produce,
e.g. torkit3d/csrc/cuda/chamfer_distance_kernel.cu:65-71 under nvcc's default
contraction) independently of any compiler's contraction settings.

The reference ships no fixtures of its own; the one literal example it holds (the
commented pair of clouds in tests/ops/test_chamfer_distance.py:42-43) is included
as case "chamfer_known".

Run:  python tests/golden/make_golden.py
"""
import os
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


# ---- exact float32 arithmetic ---------------------------------------------------

def round_f32(x):
    """Nearest float32 (ties to even) of an exact rational."""
    x = Fraction(x)
    if x == 0:
        return np.float32(0.0)
    sign = -1 if x < 0 else 1
    x = abs(x)
    # exponent e with 2^e <= x < 2^(e+1)
    e = x.numerator.bit_length() - x.denominator.bit_length()
    if Fraction(2) ** e > x:
        e -= 1
    elif Fraction(2) ** (e + 1) <= x:
        e += 1
    q = max(e - 23, -149)  # quantum exponent (subnormals bottom out at 2^-149)
    scaled = x / (Fraction(2) ** q)
    m = scaled.numerator // scaled.denominator
    rem = scaled - m
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (m & 1)):
        m += 1
    val = Fraction(m) * (Fraction(2) ** q)
    if val >= Fraction(2) ** 128:
        return np.float32(sign * np.inf)
    return np.float32(sign * float(val))  # exact: val has <= 24 significant bits


def F(v):
    return Fraction(float(v))


def sub32(a, b):
    return round_f32(F(a) - F(b))


def mul32(a, b):
    return round_f32(F(a) * F(b))


def add32(a, b):
    return round_f32(F(a) + F(b))


def fma32(a, b, c):
    return round_f32(F(a) * F(b) + F(c))


def dist2(key, query):
    dx, dy, dz = (sub32(key[i], query[i]) for i in range(3))
    d = mul32(dx, dx)
    d = fma32(dy, dy, d)
    d = fma32(dz, dz, d)
    return d


# ---- the six ops, literally ----------------------------------------------------------

def chamfer_one_direction(xyz1, xyz2):
    """chamfer_distance_kernel.cu:42-43,60-78: ascending scan, strict '<'."""
    b, n1, _ = xyz1.shape
    dist = np.zeros((b, n1), np.float32)
    idx = np.zeros((b, n1), np.int64)
    for bi in range(b):
        for i in range(n1):
            best, best_j = np.float32(np.inf), -1
            for j in range(xyz2.shape[1]):
                d = dist2(xyz2[bi, j], xyz1[bi, i])
                if d < best:
                    best, best_j = d, j
            dist[bi, i], idx[bi, i] = best, best_j
    return dist, idx


def chamfer_backward(gd1, gd2, xyz1, xyz2, idx1, idx2):
    """chamfer_distance_kernel.cu:184-196, both passes, adding in ascending order."""
    gx1 = np.zeros(xyz1.shape, np.float32)
    gx2 = np.zeros(xyz2.shape, np.float32)

    def one_pass(ga, gb, gd, idx, xa, xb):
        for bi in range(xa.shape[0]):
            for i in range(xa.shape[1]):
                j = idx[bi, i]
                g = mul32(gd[bi, i], np.float32(2))
                for d in range(3):
                    v = mul32(g, sub32(xa[bi, i, d], xb[bi, j, d]))
                    ga[bi, i, d] = add32(ga[bi, i, d], v)
                    gb[bi, j, d] = add32(gb[bi, j, d], -v)

    one_pass(gx1, gx2, gd1, idx1, xyz1, xyz2)
    one_pass(gx2, gx1, gd2, idx2, xyz2, xyz1)
    return gx1, gx2


def knn_mink(query, key, k):
    """MinK::add, mink.cuh:61-89, driven by knn_distance_kernel.cu:62-83."""
    b, n1, _ = query.shape
    dist = np.zeros((b, n1, k), np.float32)
    idx = np.zeros((b, n1, k), np.int64)
    for bi in range(b):
        for i in range(n1):
            keys, vals, max_key, max_idx = [], [], None, 0
            for j in range(key.shape[1]):
                d = dist2(key[bi, j], query[bi, i])
                if len(keys) < k:
                    if len(keys) == 0 or d > max_key:
                        max_key, max_idx = d, len(keys)
                    keys.append(d)
                    vals.append(j)
                elif d < max_key:
                    keys[max_idx], vals[max_idx] = d, j
                    max_key = d
                    for s in range(k):
                        if keys[s] > max_key:
                            max_key, max_idx = keys[s], s
            dist[bi, i], idx[bi, i] = keys, vals
    return dist, idx


def ball_query(query, key, radius, k):
    """ball_query_kernel.cu:26,66-101,123."""
    r = np.float32(radius)
    r2 = mul32(r, r)
    b, n1, _ = query.shape
    out = np.full((b, n1, k), -1, np.int64)
    for bi in range(b):
        for i in range(n1):
            cnt = 0
            for j in range(key.shape[1]):
                d = dist2(key[bi, j], query[bi, i])
                if cnt < k and d < r2:
                    out[bi, i, cnt] = j
                    cnt += 1
            if cnt < k:
                out[bi, i, cnt:] = out[bi, i, 0]
    return out


def fps_block_size(n):
    bs = 1
    while bs < n and bs < 512:
        bs *= 2
    return max(bs, 32)


def fps(points, k):
    """sample_farthest_points_kernel.cu:27-102: per-thread scan + shared-memory tree."""
    b, n, _ = points.shape
    bs = fps_block_size(n)
    out = np.zeros((b, k), np.int64)
    for bi in range(b):
        p = points[bi]
        md = [np.float32(-1)] * n
        sel = 0
        for it in range(1, k):
            sd, si = [np.float32(0)] * bs, [sel] * bs
            for tid in range(bs):
                for j in range(tid, n, bs):
                    d = dist2(p[j], p[sel])
                    if md[j] > d or md[j] < 0:
                        md[j] = d
                    if md[j] > sd[tid]:
                        sd[tid], si[tid] = md[j], j
            s = bs // 2
            while s > 0:
                for tid in range(s):
                    if sd[tid] < sd[tid + s]:
                        sd[tid], si[tid] = sd[tid + s], si[tid + s]
                s //= 2
            sel = si[0]
            out[bi, it] = sel
    return out


def group_forward(inp, index):
    b, c, _ = inp.shape
    _, n2, k = index.shape
    out = np.zeros((b, c, n2, k), np.float32)
    for bi in range(b):
        for ci in range(c):
            for m in range(n2):
                for s in range(k):
                    out[bi, ci, m, s] = inp[bi, ci, index[bi, m, s]]
    return out


def group_backward(gout, index, n1):
    b, c, n2, k = gout.shape
    gin = np.zeros((b, c, n1), np.float32)
    for bi in range(b):
        for ci in range(c):
            for m in range(n2):
                for s in range(k):
                    j = index[bi, m, s]
                    gin[bi, ci, j] = add32(gin[bi, ci, j], gout[bi, ci, m, s])
    return gin


def interpolate_forward(inp, index, weight):
    """interpolate_kernel.cu:31-45 with fused multiply-adds."""
    b, c, _ = inp.shape
    _, n2, k = index.shape
    out = np.zeros((b, c, n2), np.float32)
    for bi in range(b):
        for ci in range(c):
            for n in range(n2):
                acc = np.float32(0)
                for i in range(k):
                    acc = fma32(inp[bi, ci, index[bi, n, i]], weight[bi, n, i], acc)
                out[bi, ci, n] = acc
    return out


def interpolate_backward(gout, index, weight, n1):
    b, c, n2 = gout.shape
    k = index.shape[2]
    gin = np.zeros((b, c, n1), np.float32)
    for bi in range(b):
        for ci in range(c):
            for n in range(n2):
                for i in range(k):
                    j = index[bi, n, i]
                    gin[bi, ci, j] = add32(gin[bi, ci, j], mul32(gout[bi, ci, n], weight[bi, n, i]))
    return gin


# ---- cases -------------------------------------------------------------------------------

def lattice(rng, shape, steps=8):
    """Coordinates k/steps: differences, squares and sums are exact, ties abound."""
    return (rng.integers(0, steps + 1, size=shape) / steps).astype(np.float32)


def main():
    rng = np.random.default_rng(20240607)
    out = {}

    # chamfer: random, lattice (ties), and the reference's literal example
    a = (rng.random((2, 24, 3)) * 2 - 1).astype(np.float32)
    b = (rng.random((2, 19, 3)) * 2 - 1).astype(np.float32)
    d1, i1 = chamfer_one_direction(a, b)
    d2, i2 = chamfer_one_direction(b, a)
    g1 = rng.standard_normal((2, 24)).astype(np.float32)
    g2 = rng.standard_normal((2, 19)).astype(np.float32)
    gx1, gx2 = chamfer_backward(g1, g2, a, b, i1, i2)
    out.update(chamfer_rand_xyz1=a, chamfer_rand_xyz2=b, chamfer_rand_dist1=d1,
               chamfer_rand_idx1=i1, chamfer_rand_dist2=d2, chamfer_rand_idx2=i2,
               chamfer_rand_gd1=g1, chamfer_rand_gd2=g2, chamfer_rand_gx1=gx1,
               chamfer_rand_gx2=gx2)
    a = lattice(rng, (2, 20, 3), 4)
    b = lattice(rng, (2, 30, 3), 4)
    d1, i1 = chamfer_one_direction(a, b)
    d2, i2 = chamfer_one_direction(b, a)
    out.update(chamfer_lat_xyz1=a, chamfer_lat_xyz2=b, chamfer_lat_dist1=d1,
               chamfer_lat_idx1=i1, chamfer_lat_dist2=d2, chamfer_lat_idx2=i2)
    a = np.array([[[0, 0, 1], [1, 0, 0]]], np.float32)
    b = np.array([[[0, 0, 1.1], [1.2, 0, 0]]], np.float32)
    d1, i1 = chamfer_one_direction(a, b)
    d2, i2 = chamfer_one_direction(b, a)
    out.update(chamfer_known_xyz1=a, chamfer_known_xyz2=b, chamfer_known_dist1=d1,
               chamfer_known_idx1=i1, chamfer_known_dist2=d2, chamfer_known_idx2=i2)

    # knn: random k=3 and k=5, lattice k=4 (ties at the k-th boundary)
    q = rng.standard_normal((2, 9, 3)).astype(np.float32)
    key = rng.standard_normal((2, 21, 3)).astype(np.float32)
    for k in (3, 5):
        d, i = knn_mink(q, key, k)
        out["knn_rand_k%d_dist" % k], out["knn_rand_k%d_idx" % k] = d, i
    out.update(knn_rand_query=q, knn_rand_key=key)
    q, key = lattice(rng, (1, 10, 3), 3), lattice(rng, (1, 25, 3), 3)
    d, i = knn_mink(q, key, 4)
    out.update(knn_lat_query=q, knn_lat_key=key, knn_lat_k4_dist=d, knn_lat_k4_idx=i)

    # ball query: queries drawn from the keys; one far-away query with no hit
    key = rng.random((2, 40, 3)).astype(np.float32)
    q = key[:, rng.permutation(40)[:7]].copy()
    q[1, 3] = 50.0
    out.update(ball_key=key, ball_query=q, ball_radius=np.float32(0.35),
               ball_idx_k8=ball_query(q, key, 0.35, 8),
               ball_idx_k3=ball_query(q, key, 0.35, 3))
    key = lattice(rng, (1, 30, 3), 4)
    q = key[:, :6].copy()
    out.update(ball_lat_key=key, ball_lat_query=q, ball_lat_radius=np.float32(0.5),
               ball_lat_idx_k6=ball_query(q, key, 0.5, 6))

    # fps: random, lattice (ties for the maximum), duplicates
    p = rng.random((2, 45, 3)).astype(np.float32)
    out.update(fps_rand_points=p, fps_rand_idx=fps(p, 20))
    p = lattice(rng, (2, 70, 3), 2)
    out.update(fps_lat_points=p, fps_lat_idx=fps(p, 40))
    p = np.repeat(rng.random((1, 5, 3)).astype(np.float32), 8, axis=1)
    out.update(fps_dup_points=p, fps_dup_idx=fps(p, 12))

    # group / interpolate
    f = rng.standard_normal((2, 3, 11)).astype(np.float32)
    idx = rng.integers(0, 11, (2, 5, 4)).astype(np.int64)
    go = rng.standard_normal((2, 3, 5, 4)).astype(np.float32)
    out.update(group_input=f, group_index=idx, group_output=group_forward(f, idx),
               group_grad_output=go, group_grad_input=group_backward(go, idx, 11))
    idx = rng.integers(0, 11, (2, 6, 3)).astype(np.int64)
    w = rng.random((2, 6, 3)).astype(np.float32)
    go = rng.standard_normal((2, 3, 6)).astype(np.float32)
    out.update(interp_input=f, interp_index=idx, interp_weight=w,
               interp_output=interpolate_forward(f, idx, w), interp_grad_output=go,
               interp_grad_input=interpolate_backward(go, idx, w, 11))

    path = os.path.join(HERE, "tk3d_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, "with", len(out), "arrays")


if __name__ == "__main__":
    main()
