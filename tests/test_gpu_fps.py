"""Farthest point sampling on the GPU: indices bit-identical to the oracle (which
replays the reference kernel's threads, including its tie order)."""
import numpy as np
import pytest
import torch

import oracle
from util import fps_numpy, gaussian_mixture_cloud, lattice_cloud

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def run(points, k, cuda, transpose=False):
    from torkit3d_amd.ops.sample_farthest_points import sample_farthest_points

    return sample_farthest_points(points.to(cuda), k, transpose=transpose).cpu().numpy()


@pytest.mark.parametrize("b,n,k,transpose", [(1, 31, 2, True), (2, 1024, 128, True),
                                              (3, 1025, 129, False), (3, 1025, 129, True),
                                              (16, 1024, 512, False), (32, 1024, 512, True),
                                              (32, 8192, 2048, False)])
def test_reference_cases_fp64(cuda, b, n, k, transpose):
    # tests/ops/test_sample_farthest_points.py:41-62: fp64 uniform points vs numpy
    np.random.seed(0)
    pts = np.random.rand(b, n, 3)
    want = oracle.sample_farthest_points(pts, k)
    if b * n * k <= 3 * 1025 * 129:
        np.testing.assert_array_equal(want, fps_numpy(pts, k))
    t = torch.from_numpy(pts)
    if transpose:
        t = t.transpose(1, 2).contiguous()
    np.testing.assert_array_equal(run(t, k, cuda, transpose), want)


def test_sampling_config_fp32(cuda):
    # benchmark config 2: B=16, N=4096 from a mixture of 8 Gaussians, 1024 samples
    pts = gaussian_mixture_cloud(gen(2), 16, 4096)
    got = run(pts, 1024, cuda)
    np.testing.assert_array_equal(got, oracle.sample_farthest_points(pts.numpy(), 1024))
    assert (got[:, 0] == 0).all()
    assert all(len(set(row)) == 1024 for row in got)


def test_set_abstraction_chain_fp32(cuda):
    # benchmark config 5: B=8, 16384 -> 4096 -> 1024 -> 256, each level on the previous picks
    from torkit3d_amd import _C

    g = gen(5)
    xyz = torch.rand(8, 16384, 3, generator=g)
    cur_gpu, cur_cpu = xyz.to(cuda), xyz.numpy()
    for k in (4096, 1024, 256):
        got = _C.sample_farthest_points_cuda(cur_gpu, k)
        want = oracle.sample_farthest_points(cur_cpu, k)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
        cur_gpu = torch.gather(cur_gpu, 1, got[:, :, None].expand(-1, -1, 3)).contiguous()
        cur_cpu = np.take_along_axis(cur_cpu, want[:, :, None], 1)


@pytest.mark.parametrize("n", [1, 2, 31, 33, 64, 65, 255, 257, 511, 513, 1000, 2049, 4097,
                                8191, 12000, 16384])
def test_every_launch_shape_fp32(cuda, n):
    pts = torch.rand(2, n, 3, generator=gen(n))
    k = min(n, 70)
    np.testing.assert_array_equal(run(pts, k, cuda), oracle.sample_farthest_points(pts.numpy(), k))


@pytest.mark.parametrize("n,dtype", [(16385, torch.float32), (20000, torch.float32),
                                      (8193, torch.float64)])
def test_workspace_path_for_large_clouds(cuda, n, dtype):
    pts = torch.rand(2, n, 3, generator=gen(n), dtype=dtype)
    np.testing.assert_array_equal(run(pts, 40, cuda), oracle.sample_farthest_points(pts.numpy(), 40))


@pytest.mark.parametrize("n", [64, 70, 600, 3000, 17000])
def test_ties_follow_the_reference_tree_order(cuda, n):
    # lattice clouds tie for the maximum all the time; the oracle replays the reference's
    # per-thread scan and tree, which is not lowest-index order
    pts = lattice_cloud(gen(n), 3, n, 2)
    k = min(n, 60)
    want = oracle.sample_farthest_points(pts.numpy(), k)
    np.testing.assert_array_equal(run(pts, k, cuda), want)
    if n == 600:
        assert not np.array_equal(want, oracle.sample_farthest_points(pts.numpy(), k, "lowest"))


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 64, 333])
def test_every_sample_count_ends_on_the_right_step(cuda, k):
    # the fp32 kernel takes several selection steps per exchange between its waves; the
    # last exchange must stop exactly at num_samples
    pts = torch.rand(3, 2000, 3, generator=gen(50 + k))
    guard = torch.full((3, k + 8), -7, dtype=torch.int64, device=cuda)
    from torkit3d_amd import _C

    got = _C.sample_farthest_points_cuda(pts.to(cuda), k)
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.sample_farthest_points(pts.numpy(), k))
    assert int(guard.min()) == -7


@pytest.mark.parametrize("kind", ["clusters", "two_far_copies", "lattice_fine", "half_duplicates",
                                  "line", "shell"])
def test_multi_step_selection_on_adversarial_clouds(cuda, kind):
    # clouds on which the candidates of different waves are close to each other, tie, or
    # sit in the same wave: the shortcut must refuse exactly the steps it cannot prove
    g = gen(60)
    n = 4096
    if kind == "clusters":      # 64 tight clusters: after 64 picks every candidate is tiny
        centres = torch.rand(2, 64, 3, generator=g)
        pts = centres[:, torch.randint(0, 64, (n,), generator=g)] + 1e-3 * torch.randn(2, n, 3, generator=g)
    elif kind == "two_far_copies":  # every point twice: each maximum is held by two points
        half = torch.rand(2, n // 2, 3, generator=g)
        pts = torch.cat([half, half + torch.tensor([4.0, 0.0, 0.0])], dim=1)
        pts = torch.cat([pts[:, ::2], pts[:, 1::2]], dim=1)
    elif kind == "lattice_fine":
        pts = lattice_cloud(g, 2, n, 3)
    elif kind == "half_duplicates":
        half = torch.rand(2, n // 2, 3, generator=g)
        pts = torch.cat([half, half], dim=1)
    elif kind == "line":         # points on a line: neighbours of a pick are the next picks
        pts = torch.zeros(2, n, 3)
        pts[:, :, 0] = torch.rand(2, n, generator=g)
    else:                        # thin shell
        u = torch.randn(2, n, 3, generator=g)
        pts = u / u.norm(dim=2, keepdim=True)
    k = 1500
    np.testing.assert_array_equal(run(pts, k, cuda), oracle.sample_farthest_points(pts.numpy(), k))


def test_duplicates_and_full_sample(cuda):
    ones = torch.ones(2, 500, 3)
    np.testing.assert_array_equal(run(ones, 20, cuda), np.zeros((2, 20), np.int64))
    pts = torch.rand(2, 700, 3, generator=gen(1))
    got = run(pts, 700, cuda)
    np.testing.assert_array_equal(np.sort(got, axis=1), np.tile(np.arange(700), (2, 1)))
    np.testing.assert_array_equal(got, oracle.sample_farthest_points(pts.numpy(), 700))


def test_errors(cuda):
    from torkit3d_amd import _C

    pts = torch.zeros(2, 8, 3, device=cuda)
    with pytest.raises(RuntimeError):
        _C.sample_farthest_points_cuda(pts, 0)
    with pytest.raises(RuntimeError):
        _C.sample_farthest_points_cuda(pts, 9)
    with pytest.raises(RuntimeError):
        _C.sample_farthest_points_cuda(torch.zeros(2, 8, 4, device=cuda), 2)


# ---- clouds beyond one workgroup's registers: one launch per step, many workgroups ----

@pytest.mark.parametrize("b,n,k,dtype,transpose", [
    (1, 20000, 300, torch.float32, False), (3, 65536 + 3, 120, torch.float32, True),
    (2, 40000, 64, torch.float64, False), (5, 16385, 33, torch.float32, True),
    (1, 8200, 500, torch.float64, True), (2, 17000, 17000 // 40, torch.float32, False)])
def test_wide_path_shapes_layouts_and_types(cuda, b, n, k, dtype, transpose):
    pts = torch.rand(b, n, 3, generator=gen(n + k), dtype=dtype)
    want = oracle.sample_farthest_points(pts.numpy(), k)
    dev = pts.transpose(1, 2).contiguous() if transpose else pts
    np.testing.assert_array_equal(run(dev, k, cuda, transpose), want)


@pytest.mark.parametrize("n", [17000, 70001])
def test_wide_path_ties_follow_the_reference_tree_order(cuda, n):
    pts = lattice_cloud(gen(n), 2, n, 3)
    want = oracle.sample_farthest_points(pts.numpy(), 80)
    np.testing.assert_array_equal(run(pts, 80, cuda), want)
    assert not np.array_equal(want, oracle.sample_farthest_points(pts.numpy(), 80, "lowest"))


def test_wide_path_duplicates_repeat_the_previous_choice(cuda):
    # 5 distinct positions: from the sixth sample on nothing lies away from the chosen set
    base = torch.rand(1, 5, 3, generator=gen(5))
    pts = base[:, torch.randint(0, 5, (30000,), generator=gen(6))]
    want = oracle.sample_farthest_points(pts.numpy(), 12)
    np.testing.assert_array_equal(run(pts, 12, cuda), want)
    assert len(set(want[0, 5:].tolist())) == 1


def test_wide_path_with_coordinates(cuda):
    from torkit3d_amd.ops.sample_farthest_points import sample_farthest_points_gather

    pts = torch.rand(2, 3, 30000, generator=gen(7)).to(cuda)
    idx, xyz = sample_farthest_points_gather(pts, 50, transpose=True)
    want = oracle.sample_farthest_points(pts.transpose(1, 2).contiguous().cpu().numpy(), 50)
    np.testing.assert_array_equal(idx.cpu().numpy(), want)
    assert torch.equal(xyz, torch.gather(pts, 2, idx[:, None, :].expand(-1, 3, -1)))


# ---- non-finite coordinates: the reference's "unset" minima take the first distance as
# it comes, so a point with a NaN coordinate is never selected and the others are sampled
# as if it were absent; a NaN in point 0 leaves nothing to select ----

@pytest.mark.parametrize("n,dtype", [(300, torch.float32), (5000, torch.float32),
                                      (5000, torch.float64), (30000, torch.float32)])
def test_points_with_nan_are_never_selected(cuda, n, dtype):
    pts = torch.rand(3, n, 3, generator=gen(n), dtype=dtype)
    pts[0, 7, 1] = float("nan")
    pts[0, n // 2] = float("nan")
    pts[1, n - 1, 0] = float("nan")
    pts[2, 0, 2] = float("nan")        # point 0 itself: every distance is NaN
    k = 40
    want = oracle.sample_farthest_points(pts.numpy(), k)
    got = run(pts, k, cuda)
    np.testing.assert_array_equal(got, want)
    assert 7 not in got[0] and n // 2 not in got[0] and n - 1 not in got[1]
    assert (got[2] == 0).all()


def test_points_at_infinity(cuda):
    pts = torch.rand(2, 2000, 3, generator=gen(9))
    pts[0, 100, 0] = float("inf")
    pts[1, 5] = float("-inf")
    pts[1, 900, 2] = float("inf")
    want = oracle.sample_farthest_points(pts.numpy(), 30)
    np.testing.assert_array_equal(run(pts, 30, cuda), want)


# ---- 4097 to 16384 points, 256 samples or more: the kernel that lays the points out by
# region (Morton order), skips the blocks a new centre cannot reach and accepts from sixteen
# candidates per exchange. The lane order is no longer the reference's priority order there,
# so ties are resolved explicitly. 4097..8192 points run it with 8 points per lane, more with
# 16. ----

def _region_cloud(kind, g, b, n):
    if kind == "uniform":
        return torch.rand(b, n, 3, generator=g)
    if kind == "mixture":
        return gaussian_mixture_cloud(g, b, n)
    if kind == "lattice":            # ties for the maximum at almost every step
        return lattice_cloud(g, b, n, 3)
    if kind == "coarse_lattice":     # 27 positions: after 27 picks nothing lies away
        return lattice_cloud(g, b, n, 2)
    if kind == "two_far_copies":     # every maximum is held by two points, in different regions
        half = torch.rand(b, n // 2, 3, generator=g)
        pts = torch.cat([half, half + torch.tensor([4.0, 0.0, 0.0])], dim=1)
        return torch.cat([pts[:, ::2], pts[:, 1::2]], dim=1).contiguous()
    if kind == "half_duplicates":    # every point twice at the same place
        half = torch.rand(b, n // 2, 3, generator=g)
        return torch.cat([half, half], dim=1)
    if kind == "line":               # degenerate boxes
        pts = torch.zeros(b, n, 3)
        pts[:, :, 0] = torch.rand(b, n, generator=g)
        return pts
    if kind == "shell":
        u = torch.randn(b, n, 3, generator=g)
        return u / u.norm(dim=2, keepdim=True)
    if kind == "clusters":
        centres = torch.rand(b, 64, 3, generator=g)
        return centres[:, torch.randint(0, 64, (n,), generator=g)] + 1e-3 * torch.randn(b, n, 3, generator=g)
    if kind == "far_from_origin":    # coarse float grid: many exact ties, huge offsets
        return torch.rand(b, n, 3, generator=g) + 4096.0
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["uniform", "mixture", "lattice", "coarse_lattice", "two_far_copies",
                                  "half_duplicates", "line", "shell", "clusters", "far_from_origin"])
def test_region_kernel_on_adversarial_clouds(cuda, kind):
    g = gen(70)
    pts = _region_cloud(kind, g, 2, 12000 if kind in ("uniform", "lattice") else 16384)
    k = 2100
    np.testing.assert_array_equal(run(pts, k, cuda), oracle.sample_farthest_points(pts.numpy(), k))
    # and with 8 points per lane
    pts = _region_cloud(kind, g, 2, 6000 if kind in ("uniform", "lattice") else 8192)
    k = 700
    np.testing.assert_array_equal(run(pts, k, cuda), oracle.sample_farthest_points(pts.numpy(), k))
    # and with 4 (2049 to 4096 points)
    pts = _region_cloud(kind, g, 2, 2700 if kind in ("uniform", "lattice") else 4096)
    k = 600
    np.testing.assert_array_equal(run(pts, k, cuda), oracle.sample_farthest_points(pts.numpy(), k))


@pytest.mark.parametrize("n,k,transpose", [(8193, 2048, False), (16384, 16384, False),
                                           (10000, 2049, True), (16383, 4096, True),
                                           (4097, 256, False), (8192, 8192, False),
                                           (5000, 300, True), (16384, 256, True),
                                           (8193, 257, False), (2049, 256, False),
                                           (4096, 4096, False), (3072, 256, True),
                                           (3073, 512, True), (2500, 2500, False)])
def test_region_kernel_shapes_and_layouts(cuda, n, k, transpose):
    pts = torch.rand(2, n, 3, generator=gen(n + k))
    want = oracle.sample_farthest_points(pts.numpy(), k)
    dev = pts.transpose(1, 2).contiguous() if transpose else pts
    np.testing.assert_array_equal(run(dev, k, cuda, transpose), want)


@pytest.mark.parametrize("n,k,transpose", [(4096, 1024, False), (3000, 512, True), (2049, 2049, False)])
def test_clouds_in_sampling_order_between_2049_and_4096_points(cuda, n, k, transpose):
    # A cloud that is itself a farthest point sample in sampling order (the next level of a
    # PointNet++ encoder): its point 1 is the point farthest from point 0, by which the region
    # kernel recognises it and leaves it to the multi-step kernel launched behind it. The
    # answer is the first k indices in order. Then a cloud in random order whose point 1
    # happens to be the farthest from point 0: it takes the same route and must come out right
    # as well, and one with a NaN in that place.
    big = torch.rand(2, 3 * n, 3, generator=gen(n + k))
    first = oracle.sample_farthest_points(big.numpy(), n)
    pts = torch.gather(big, 1, torch.from_numpy(first)[:, :, None].expand(-1, -1, 3)).contiguous()
    want = oracle.sample_farthest_points(pts.numpy(), k)
    np.testing.assert_array_equal(want, np.tile(np.arange(k), (2, 1)))
    dev = pts.transpose(1, 2).contiguous() if transpose else pts
    np.testing.assert_array_equal(run(dev, k, cuda, transpose), want)
    rnd = torch.rand(2, n, 3, generator=gen(n))
    rnd[:, 0] = 0.0
    rnd[:, 1] = 5.0                      # farther from point 0 than anything in the unit cube
    dev = rnd.transpose(1, 2).contiguous() if transpose else rnd
    np.testing.assert_array_equal(run(dev, k, cuda, transpose),
                                  oracle.sample_farthest_points(rnd.numpy(), k))
    rnd[0, 1, 2] = float("nan")
    dev = rnd.transpose(1, 2).contiguous() if transpose else rnd
    np.testing.assert_array_equal(run(dev, k, cuda, transpose),
                                  oracle.sample_farthest_points(rnd.numpy(), k))


@pytest.mark.parametrize("n", [9000, 5000, 3000])
def test_region_kernel_with_non_finite_points(cuda, n):
    pts = torch.rand(3, n, 3, generator=gen(71))
    pts[0, 7, 1] = float("nan")
    pts[0, n // 2] = float("nan")
    pts[1, 100, 0] = float("inf")
    pts[2, 0, 2] = float("nan")        # point 0 itself: every distance is NaN
    k = 2048 if n == 9000 else 400
    want = oracle.sample_farthest_points(pts.numpy(), k)
    np.testing.assert_array_equal(run(pts, k, cuda), want)


@pytest.mark.parametrize("b,n,k", [(16, 8192, 2048), (4, 10000, 512)])
def test_shapes_the_reference_author_profiled(cuda, b, n, k):
    # tests/ops/test_sample_farthest_points.py:74-76 (profile runs, no recorded result)
    pts = torch.rand(b, n, 3, generator=gen(8))
    np.testing.assert_array_equal(run(pts, k, cuda), oracle.sample_farthest_points(pts.numpy(), k))
