"""Pins the CPU oracle for the distance ops (chamfer, knn, ball query, fps).

Checks, per op: the committed golden vectors (made by an independent exact-arithmetic
Python restatement), library routines / brute force in numpy and torch, closed
forms, and tie behaviour on lattice inputs where fp32 arithmetic is exact.
"""
import numpy as np
import pytest
import torch

import oracle
from util import (ball_query_numpy, fps_numpy, lattice_cloud, pairwise_d2_f64, sorted_pairs,
                  uniform_cloud)


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ---- golden vectors ---------------------------------------------------------------

@pytest.mark.parametrize("case", ["rand", "lat", "known"])
def test_chamfer_forward_golden(golden, case):
    out = oracle.chamfer_forward(golden[f"chamfer_{case}_xyz1"], golden[f"chamfer_{case}_xyz2"])
    for name, got in zip(("dist1", "idx1", "dist2", "idx2"), out):
        np.testing.assert_array_equal(got, golden[f"chamfer_{case}_{name}"], err_msg=name)


def test_chamfer_known_answer(golden):
    # The literal example in the reference's tests/ops/test_chamfer_distance.py:42-43.
    np.testing.assert_allclose(golden["chamfer_known_dist1"], [[0.01, 0.04]], rtol=1e-5)
    np.testing.assert_array_equal(golden["chamfer_known_idx1"], [[0, 1]])
    np.testing.assert_array_equal(golden["chamfer_known_idx2"], [[0, 1]])


def test_chamfer_backward_golden(golden):
    g = golden
    gx1, gx2 = oracle.chamfer_backward(g["chamfer_rand_gd1"], g["chamfer_rand_gd2"],
                                       g["chamfer_rand_xyz1"], g["chamfer_rand_xyz2"],
                                       g["chamfer_rand_idx1"], g["chamfer_rand_idx2"])
    np.testing.assert_array_equal(gx1, g["chamfer_rand_gx1"])
    np.testing.assert_array_equal(gx2, g["chamfer_rand_gx2"])


def test_knn_golden(golden):
    for k in (3, 5):
        d, i = oracle.knn(golden["knn_rand_query"], golden["knn_rand_key"], k)
        np.testing.assert_array_equal(d, golden[f"knn_rand_k{k}_dist"])
        np.testing.assert_array_equal(i, golden[f"knn_rand_k{k}_idx"])
    d, i = oracle.knn(golden["knn_lat_query"], golden["knn_lat_key"], 4)
    np.testing.assert_array_equal(d, golden["knn_lat_k4_dist"])
    np.testing.assert_array_equal(i, golden["knn_lat_k4_idx"])


def test_ball_query_golden(golden):
    r = float(golden["ball_radius"])
    for k in (8, 3):
        got = oracle.ball_query(golden["ball_query"], golden["ball_key"], r, k)
        np.testing.assert_array_equal(got, golden[f"ball_idx_k{k}"])
    assert (golden["ball_idx_k8"][1, 3] == -1).all()  # the far-away query has no hit
    got = oracle.ball_query(golden["ball_lat_query"], golden["ball_lat_key"],
                            float(golden["ball_lat_radius"]), 6)
    np.testing.assert_array_equal(got, golden["ball_lat_idx_k6"])


@pytest.mark.parametrize("case,k", [("rand", 20), ("lat", 40), ("dup", 12)])
def test_fps_golden(golden, case, k):
    got = oracle.sample_farthest_points(golden[f"fps_{case}_points"], k)
    np.testing.assert_array_equal(got, golden[f"fps_{case}_idx"])


# ---- chamfer ------------------------------------------------------------------------

@pytest.mark.parametrize("b,n1,n2", [(2, 1024, 1024), (3, 257, 300), (1, 5, 1)])
def test_chamfer_matches_bruteforce_fp64(b, n1, n2):
    # fp64 random data has no near-ties, so argmin must agree with numpy exactly.
    g = gen(11)
    a = uniform_cloud(g, b, n1, dtype=torch.float64).numpy()
    c = uniform_cloud(g, b, n2, dtype=torch.float64).numpy()
    d1, i1, d2, i2 = oracle.chamfer_forward(a, c)
    D = pairwise_d2_f64(a, c)
    np.testing.assert_array_equal(i1, D.argmin(2))
    np.testing.assert_array_equal(i2, D.argmin(1))
    np.testing.assert_allclose(d1, D.min(2), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(d2, D.min(1), rtol=1e-12, atol=1e-15)


def test_chamfer_fp32_against_torch_bruteforce():
    # The reference's own oracle: torch brute force (tests/ops/test_chamfer_distance.py:8-31),
    # distances atol 1e-6, indices exact except where fused/un-fused rounding meets a
    # near-tie; every such disagreement must be a <= 1 ulp tie.
    g = gen(1)
    a, c = uniform_cloud(g, 2, 1024), uniform_cloud(g, 2, 1024)
    diff = a[:, :, None, :] - c[:, None, :, :]
    D = (diff ** 2).sum(-1)
    td1, ti1 = D.min(2)
    td2, ti2 = D.min(1)
    d1, i1, d2, i2 = oracle.chamfer_forward(a.numpy(), c.numpy())
    np.testing.assert_allclose(d1, td1.numpy(), atol=1e-6, rtol=1e-5)
    np.testing.assert_allclose(d2, td2.numpy(), atol=1e-6, rtol=1e-5)
    for mine, theirs, dist in ((i1, ti1.numpy(), D.numpy()), (i2, ti2.numpy(), D.numpy().transpose(0, 2, 1))):
        bad = np.argwhere(mine != theirs)
        assert len(bad) <= 2
        for bi, qi in bad:
            x, y = dist[bi, qi, mine[bi, qi]], dist[bi, qi, theirs[bi, qi]]
            assert abs(x - y) <= 2 * np.spacing(np.float32(max(x, y)))


def test_chamfer_unfused_variant_equals_numpy_fp32():
    # The un-fused variant of the oracle is plain fp32 numpy arithmetic.
    g = gen(2)
    a, c = uniform_cloud(g, 2, 300).numpy(), uniform_cloud(g, 2, 200).numpy()
    d1, i1, d2, i2 = oracle.chamfer_forward(a, c, fused=False)
    diff = a[:, :, None, :] - c[:, None, :, :]
    D = (diff[..., 0] * diff[..., 0] + diff[..., 1] * diff[..., 1]) + diff[..., 2] * diff[..., 2]
    np.testing.assert_array_equal(d1, D.min(2))
    np.testing.assert_array_equal(i1, D.argmin(2))
    np.testing.assert_array_equal(d2, D.min(1))
    np.testing.assert_array_equal(i2, D.argmin(1))


def test_chamfer_lattice_ties_pick_lowest_index():
    # On a lattice fused and un-fused arithmetic are both exact, ties are common and
    # numpy's argmin (first minimum) is the reference's strict-'<' rule.
    g = gen(3)
    a, c = lattice_cloud(g, 3, 200, 4).numpy(), lattice_cloud(g, 3, 150, 4).numpy()
    d1, i1, d2, i2 = oracle.chamfer_forward(a, c)
    D = pairwise_d2_f64(a, c)
    assert (np.sum(D == D.min(2, keepdims=True), axis=2) > 1).any()  # ties really occur
    np.testing.assert_array_equal(i1, D.argmin(2))
    np.testing.assert_array_equal(i2, D.argmin(1))
    np.testing.assert_array_equal(d1, D.min(2).astype(np.float32))


def test_chamfer_identical_clouds_and_swap():
    g = gen(4)
    a = uniform_cloud(g, 2, 333).numpy()
    d1, i1, d2, i2 = oracle.chamfer_forward(a, a)
    assert (d1 == 0).all() and (d2 == 0).all()
    np.testing.assert_array_equal(i1, np.tile(np.arange(333), (2, 1)))
    c = uniform_cloud(g, 2, 100).numpy()
    x = oracle.chamfer_forward(a, c)
    y = oracle.chamfer_forward(c, a)
    for u, v in zip(x, (y[2], y[3], y[0], y[1])):
        np.testing.assert_array_equal(u, v)


def test_chamfer_empty_and_nan():
    a = np.zeros((2, 4, 3), np.float32)
    e = np.zeros((2, 0, 3), np.float32)
    d1, i1, d2, i2 = oracle.chamfer_forward(a, e)
    assert np.isinf(d1).all() and (i1 == -1).all() and d2.shape == (2, 0)
    c = np.full((2, 3, 3), np.nan, np.float32)
    d1, i1, _, _ = oracle.chamfer_forward(a, c)
    assert np.isinf(d1).all() and (i1 == -1).all()  # NaN is never selected


def test_chamfer_backward_matches_autograd():
    g = gen(5)
    a = uniform_cloud(g, 2, 64, dtype=torch.float64).requires_grad_()
    c = uniform_cloud(g, 2, 80, dtype=torch.float64).requires_grad_()
    gd1 = torch.randn(2, 64, generator=g, dtype=torch.float64)
    gd2 = torch.randn(2, 80, generator=g, dtype=torch.float64)
    D = ((a[:, :, None, :] - c[:, None, :, :]) ** 2).sum(-1)
    (D.min(2).values * gd1).sum().add((D.min(1).values * gd2).sum()).backward()
    _, i1, _, i2 = oracle.chamfer_forward(a.detach().numpy(), c.detach().numpy())
    gx1, gx2 = oracle.chamfer_backward(gd1.numpy(), gd2.numpy(), a.detach().numpy(),
                                       c.detach().numpy(), i1, i2)
    np.testing.assert_allclose(gx1, a.grad.numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(gx2, c.grad.numpy(), rtol=1e-12, atol=1e-14)


# ---- knn ------------------------------------------------------------------------------

@pytest.mark.parametrize("b,n1,n2,k", [(1, 512, 1024, 3), (2, 512, 1024, 32), (3, 511, 1025, 31),
                                        (2, 64, 200, 64)])
def test_knn_matches_cdist_topk_fp64(b, n1, n2, k):
    # The reference checks against torch.cdist + topk in fp64
    # (tests/ops/test_knn_distance.py:20-32): sqrt distances, sorted, exact indices.
    g = gen(0)
    q = torch.randn(b, n1, 3, generator=g, dtype=torch.float64)
    key = torch.randn(b, n2, 3, generator=g, dtype=torch.float64)
    d, i = oracle.knn(q.numpy(), key.numpy(), k)
    sd, si = sorted_pairs(d, i)
    td, ti = torch.topk(torch.cdist(q, key), k, dim=2, largest=False, sorted=True)
    np.testing.assert_array_equal(si, ti.numpy())
    np.testing.assert_allclose(np.sqrt(sd), td.numpy(), atol=5e-5, rtol=1e-4)


def test_knn_k1_is_chamfer_argmin_and_kN_is_permutation():
    g = gen(6)
    q, key = uniform_cloud(g, 2, 200).numpy(), uniform_cloud(g, 2, 77).numpy()
    d, i = oracle.knn(q, key, 1)
    cd, ci, _, _ = oracle.chamfer_forward(q, key)
    np.testing.assert_array_equal(d[..., 0], cd)
    np.testing.assert_array_equal(i[..., 0], ci)
    d, i = oracle.knn(q, key, 77)
    np.testing.assert_array_equal(np.sort(i, axis=2), np.tile(np.arange(77), (2, 200, 1)))
    # while filling, MinK stores keys in arrival order
    np.testing.assert_array_equal(i, np.tile(np.arange(77), (2, 200, 1)))


def test_knn_lattice_ties_keep_k_smallest_distances():
    # Lattice data: several keys tie at the k-th distance. Which of the tied keys
    # survive depends on MinK's eviction order (the first slot holding the maximum is
    # overwritten, mink.cuh:74-88, which can evict an earlier key and keep a later one
    # of equal distance), so only the distances are determined: they are the k
    # smallest, every index is distinct and carries its own distance, and any key
    # strictly closer than the k-th distance is present. The exact slot contents are
    # pinned by the golden vectors (case knn_lat).
    g = gen(7)
    q, key = lattice_cloud(g, 2, 50, 4).numpy(), lattice_cloud(g, 2, 120, 4).numpy()
    k = 6
    d, i = oracle.knn(q, key, k)
    D = pairwise_d2_f64(q, key)
    np.testing.assert_array_equal(np.sort(d, axis=2),
                                  np.sort(D, axis=2)[:, :, :k].astype(np.float32))
    np.testing.assert_array_equal(np.take_along_axis(D, i, 2).astype(np.float32), d)
    assert all(len(set(row)) == k for row in i.reshape(-1, k))
    kth = np.sort(D, axis=2)[:, :, k - 1]
    for b in range(2):
        for n in range(50):
            closer = set(np.nonzero(D[b, n] < kth[b, n])[0])
            assert closer <= set(i[b, n])


# ---- ball query ---------------------------------------------------------------------------

@pytest.mark.parametrize("b,n1,n2,r,k", [(2, 64, 128, 0.1, 32), (3, 65, 129, 0.1, 32),
                                          (3, 65, 129, 10.0, 32), (4, 128, 256, 0.5, 64)])
def test_ball_query_matches_numpy_fp64(b, n1, n2, r, k):
    # Shapes and construction of the reference's test (tests/ops/test_ball_query.py:6-60):
    # fp64 keys ~ N(0,1), queries a random subset of the keys.
    rng = np.random.RandomState(0)
    key = rng.randn(b, n2, 3)
    query = np.stack([p[rng.choice(n2, n1, replace=False)] for p in key])
    got = oracle.ball_query(query, key, r, k)
    np.testing.assert_array_equal(got, ball_query_numpy(query, key, r, k))
    if r == 10.0:
        np.testing.assert_array_equal(got, np.tile(np.arange(k), (b, n1, 1)))


def test_ball_query_fp32_lattice_and_no_hit_rows():
    g = gen(8)
    key = lattice_cloud(g, 2, 300, 8).numpy()
    query = np.concatenate([key[:, :40], np.full((2, 2, 3), 9.0, np.float32)], axis=1)
    got = oracle.ball_query(query, key, 0.25, 16)  # 0.25^2 is exact: '<' is strict on ties
    np.testing.assert_array_equal(got, ball_query_numpy(query, key, 0.25, 16))
    assert (got[:, 40:] == -1).all()
    D = pairwise_d2_f64(query, key)
    assert (D[:, :40] == 0.0625).any()  # points exactly on the sphere exist and are excluded


def test_ball_query_radius_is_rounded_to_float_first():
    # radius arrives as a C float (ball_query.h:9): r2 = fl32(r)*fl32(r) also for fp64 data.
    key = np.array([[[0.0, 0.0, 0.0], [0.1, 0.0, 0.0]]], np.float64)
    query = key[:, :1].copy()
    r32 = float(np.float32(0.1))
    assert r32 > 0.1  # fl32(0.1) is above 0.1, so the point at distance 0.1 is inside
    got = oracle.ball_query(query, key, 0.1, 2)
    np.testing.assert_array_equal(got, [[[0, 1]]])


# ---- farthest point sampling ------------------------------------------------------------------

@pytest.mark.parametrize("b,n,k", [(1, 31, 2), (2, 1024, 128), (3, 1025, 129), (16, 1024, 512)])
def test_fps_matches_numpy_fp64(b, n, k):
    # The reference's test: fp64 uniform points, numpy running-min/argmax oracle
    # (tests/ops/test_sample_farthest_points.py:41-62).
    rng = np.random.RandomState(0)
    pts = rng.rand(b, n, 3)
    want = fps_numpy(pts, k)
    np.testing.assert_array_equal(oracle.sample_farthest_points(pts, k), want)
    np.testing.assert_array_equal(oracle.sample_farthest_points(pts, k, "lowest"), want)


def test_fps_fp32_both_rules_agree_without_ties():
    g = gen(2)
    pts = uniform_cloud(g, 4, 4096).numpy()
    a = oracle.sample_farthest_points(pts, 256)
    b = oracle.sample_farthest_points(pts, 256, "lowest")
    np.testing.assert_array_equal(a, b)


def test_fps_full_sample_is_permutation_and_gaps_shrink():
    g = gen(9)
    pts = uniform_cloud(g, 2, 300).numpy()
    idx = oracle.sample_farthest_points(pts, 300)
    np.testing.assert_array_equal(np.sort(idx, axis=1), np.tile(np.arange(300), (2, 1)))
    # distance of each pick to the set before it never increases
    for b in range(2):
        p = pts[b].astype(np.float64)
        gaps = [((p[idx[b, :t]] - p[idx[b, t]]) ** 2).sum(1).min() for t in range(1, 300)]
        assert all(x >= y - 1e-12 for x, y in zip(gaps, gaps[1:]))


def test_fps_line_closed_form():
    # Points 0..16 on a line, start at 0: farthest is 16, then the midpoint 8; the
    # next two picks are the quarter points 4 and 12 in tie order.
    pts = np.zeros((1, 17, 3), np.float32)
    pts[0, :, 0] = np.arange(17)
    low = oracle.sample_farthest_points(pts, 5, "lowest")[0]
    np.testing.assert_array_equal(low, [0, 16, 8, 4, 12])
    ref = oracle.sample_farthest_points(pts, 5)[0]
    assert list(ref[:3]) == [0, 16, 8] and sorted(ref[3:]) == [4, 12]
    # Reference tie order for 17 points in a 32-thread block: candidates 4 and 12 sit in
    # threads 4 (00100b) and 12 (01100b); the tree prefers the smaller bit-reversed
    # thread id: rev5(4)=4 < rev5(12)=6.
    np.testing.assert_array_equal(ref, [0, 16, 8, 4, 12])


def test_fps_reference_tie_rule_differs_from_lowest_index():
    # 64 points, block of 64 threads (one point per thread). Put ties at points 1 and 2:
    # rev6(1)=32 > rev6(2)=16, so the reference's tree picks 2 where numpy picks 1.
    pts = np.zeros((1, 64, 3), np.float32)
    pts[0, 1] = [1, 0, 0]
    pts[0, 2] = [0, 1, 0]
    assert oracle.sample_farthest_points(pts, 2)[0, 1] == 2
    assert oracle.sample_farthest_points(pts, 2, "lowest")[0, 1] == 1


def test_fps_all_duplicates_repeat_previous_choice():
    pts = np.ones((2, 40, 3), np.float32)
    np.testing.assert_array_equal(oracle.sample_farthest_points(pts, 10), np.zeros((2, 10)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("k", [3, 4, 5, 8, 16, 33])
def test_knn_slot_order_of_the_hand_worked_mink_run(k, dtype):
    # expected rows are literals derived by hand from mink.cuh:61-89 (tests/util.py)
    from util import MINK_STATES, mink_worked_example

    for m in sorted(MINK_STATES):
        key, dist, idx = mink_worked_example(m, k, dtype)
        query = np.zeros((1, 2, 3), dtype)
        query[0, 1, 1] = 100.0  # a second query far away: same order, other distances
        got_d, got_i = oracle.knn(query, key, k)
        np.testing.assert_array_equal(got_d[0, 0], dist, err_msg="m=%d" % m)
        np.testing.assert_array_equal(got_i[0, 0], idx, err_msg="m=%d" % m)
        np.testing.assert_array_equal(got_i[0, 1], idx, err_msg="m=%d far" % m)


def test_chamfer_backward_wide_sums_in_double():
    # fp32 terms exactly as the reference's threads form them, summed in float64 by numpy
    g = gen(31)
    b, n1, n2 = 3, 400, 90
    a, c = uniform_cloud(g, b, n1).numpy(), uniform_cloud(g, b, n2).numpy()
    gd1 = torch.randn(b, n1, generator=g).numpy()
    gd2 = torch.randn(b, n2, generator=g).numpy()
    _, i1, _, i2 = oracle.chamfer_forward(a, c)
    i1[0, 5] = -1          # skipped entries
    i2[1, 7] = n1
    acc1 = np.zeros((b, n1, 3)), np.zeros((b, n2, 3))

    def one_pass(own, other, gd, idx, x, y):
        for bi in range(b):
            ok = (idx[bi] >= 0) & (idx[bi] < y.shape[1])
            j = idx[bi][ok]
            v = (gd[bi][ok] * np.float32(2))[:, None] * (x[bi][ok] - y[bi][j])
            assert v.dtype == np.float32
            own[bi][ok] += v.astype(np.float64)
            np.add.at(other[bi], j, -v.astype(np.float64))

    one_pass(acc1[0], acc1[1], gd1, i1, a, c)
    one_pass(acc1[1], acc1[0], gd2, i2, c, a)
    gx1, gx2 = oracle.chamfer_backward(gd1, gd2, a, c, i1, i2, wide=True)
    np.testing.assert_array_equal(gx1, acc1[0].astype(np.float32))
    np.testing.assert_array_equal(gx2, acc1[1].astype(np.float32))
    # and it stays within rounding of the sequential fp32 sum
    sx1, sx2 = oracle.chamfer_backward(gd1, gd2, a, c, i1, i2)
    np.testing.assert_allclose(gx2, sx2, rtol=1e-4, atol=1e-4)
    assert not np.array_equal(gx2, sx2)
