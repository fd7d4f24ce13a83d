"""Group points and feature interpolation on the GPU. Forward results are
bit-identical to the oracle; fp32 backward within 1e-5 relative / 1e-6 absolute of the
oracle's sums taken in double and rounded once (the kernels sum in 64-bit fixed point,
the reference's atomics in an order that changes from run to run)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-5, 1e-6


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("b,c,n1,n2,k", [(2, 3, 512, 128, 32), (5, 64, 513, 129, 33),
                                          (32, 32, 1024, 512, 64), (16, 3, 8192, 2048, 32)])
def test_group_reference_cases(cuda, b, c, n1, n2, k):
    # tests/ops/test_group_points.py:15-45: fp32, torch.gather oracle, ones upstream
    from torkit3d_amd.ops.group_points import group_points

    torch.manual_seed(0)
    feat = torch.randn(b, c, n1).to(cuda).requires_grad_()
    index = torch.randint(0, n1, (b, n2, k)).to(cuda)
    want = feat.unsqueeze(2).expand(b, c, n2, n1).gather(3, index.unsqueeze(1).expand(b, c, n2, k))
    got = group_points(feat, index)
    assert torch.equal(got, want)
    got.backward(torch.ones_like(got))
    mine = feat.grad.clone()
    feat.grad = None
    want.backward(torch.ones_like(want))
    torch.testing.assert_close(mine, feat.grad, rtol=RTOL, atol=1e-6)


def test_group_config_fp32(cuda):
    # benchmark config 3: features (16,64,4096) gathered to (16,64,1024,32)
    from torkit3d_amd import _C

    g = gen(3)
    feat = torch.randn(16, 64, 4096, generator=g)
    index = torch.randint(0, 4096, (16, 1024, 32), generator=g)
    out = _C.group_points_forward_cuda(feat.to(cuda), index.to(cuda))
    np.testing.assert_array_equal(out.cpu().numpy(), oracle.group_forward(feat.numpy(), index.numpy()))
    go = torch.randn(16, 64, 1024, 32, generator=g)
    gin = _C.group_points_backward_cuda(go.to(cuda), index.to(cuda), 4096)
    np.testing.assert_allclose(gin.cpu().numpy(),
                               oracle.group_backward(go.numpy(), index.numpy(), 4096, wide=True),
                               rtol=RTOL, atol=ATOL)


def _ball_query_indices(xyz, num_centres, radius, k, cuda):
    """FPS centres of `xyz` [B,N,3] and their ball-query neighbours, checked against the
    oracle on the way: the index pattern the benchmark configurations name (runs of the
    first hit where a ball holds fewer than k points, clustered destinations)."""
    from torkit3d_amd import _C

    fps = _C.sample_farthest_points_cuda(xyz.to(cuda), num_centres)
    ofps = oracle.sample_farthest_points(xyz.numpy(), num_centres)
    np.testing.assert_array_equal(fps.cpu().numpy(), ofps)
    centres = torch.gather(xyz, 1, torch.from_numpy(ofps)[:, :, None].expand(-1, -1, 3))
    index = _C.ball_query_cuda(centres.to(cuda), xyz.to(cuda), radius, k)
    np.testing.assert_array_equal(index.cpu().numpy(),
                                  oracle.ball_query(centres.numpy(), xyz.numpy(), radius, k))
    return centres, index


def _check_group_forward_backward(feat, index, go, cuda):
    from torkit3d_amd import _C

    n1 = feat.shape[2]
    oidx = index.cpu().numpy()
    out = _C.group_points_forward_cuda(feat.to(cuda), index)
    np.testing.assert_array_equal(out.cpu().numpy(), oracle.group_forward(feat.numpy(), oidx))
    gin = _C.group_points_backward_cuda(go.to(cuda), index, n1)
    np.testing.assert_allclose(gin.cpu().numpy(),
                               oracle.group_backward(go.numpy(), oidx, n1, wide=True),
                               rtol=RTOL, atol=ATOL)


def test_group_config_with_ball_query_indices(cuda):
    # benchmark config 3 as stated: 1024 FPS centres of 4096 uniform points, r = 0.2,
    # 32 neighbours padded with the first hit, features (16,64,4096), forward + backward
    g = gen(3)
    xyz = torch.rand(16, 4096, 3, generator=g)
    _, index = _ball_query_indices(xyz, 1024, 0.2, 32, cuda)
    padded = (index[:, :, 1:] == index[:, :, :1]).any(-1).float().mean()
    assert float(padded) > 0.002  # corner centres do not fill their ball
    feat = torch.randn(16, 64, 4096, generator=g)
    go = torch.randn(16, 64, 1024, 32, generator=g)
    _check_group_forward_backward(feat, index, go, cuda)


def test_group_stress_chain_with_ball_query_indices(cuda):
    # benchmark config 5: B=8, FPS 16384 -> 4096 -> 1024 -> 256, ball query radii
    # 0.1 / 0.2 / 0.4 with 32 / 32 / 64 neighbours, features of 32 / 64 / 128 channels
    g = gen(5)
    xyz = torch.rand(8, 16384, 3, generator=g)
    for num_centres, radius, k, channels in ((4096, 0.1, 32, 32), (1024, 0.2, 32, 64),
                                             (256, 0.4, 64, 128)):
        centres, index = _ball_query_indices(xyz, num_centres, radius, k, cuda)
        feat = torch.randn(8, channels, xyz.shape[1], generator=g)
        go = torch.randn(8, channels, num_centres, k, generator=g)
        _check_group_forward_backward(feat, index, go, cuda)
        xyz = centres


def test_scatter_onto_one_destination_and_empty_balls(cuda):
    # the extremes of the ball-query pattern: every slot of every row names the same point
    # (4096 x 32 terms meet in one sum), and rows without a hit (-1) contribute nothing
    from torkit3d_amd import _C

    g = gen(24)
    index = torch.full((2, 4096, 32), 77, dtype=torch.int64)
    index[1, ::3] = -1
    go = torch.randn(2, 8, 4096, 32, generator=g)
    gin = _C.group_points_backward_cuda(go.to(cuda), index.to(cuda), 512).cpu().numpy()
    want = oracle.group_backward(go.numpy(), index.numpy(), 512, wide=True)
    np.testing.assert_allclose(gin, want, rtol=RTOL, atol=ATOL)
    assert np.count_nonzero(gin) == 16


@pytest.mark.parametrize("b,c,n1,n2,k,dtype", [
    (8, 32, 16384, 4096, 32, torch.float32),   # config 5 level 1: a 64 KiB row per channel
    (8, 64, 4096, 1024, 32, torch.float32),    # config 5 level 2
    (8, 128, 1024, 256, 64, torch.float32),    # config 5 level 3
    (2, 4, 20000, 300, 8, torch.float32),      # rows too long for LDS: global atomics
    (1, 3, 700, 1000, 16, torch.float32),      # few rows: the point range is split
    (2, 5, 100, 7, 3, torch.float64), (3, 2, 9000, 50, 5, torch.float64),
    (1, 1, 1, 1, 1, torch.float32), (2, 3, 10, 0, 4, torch.float32)])
def test_group_shapes_and_paths(cuda, b, c, n1, n2, k, dtype):
    from torkit3d_amd import _C

    g = gen(n1)
    feat = torch.randn(b, c, n1, generator=g, dtype=dtype)
    index = torch.randint(0, n1, (b, n2, k), generator=g)
    out = _C.group_points_forward_cuda(feat.to(cuda), index.to(cuda))
    np.testing.assert_array_equal(out.cpu().numpy(), oracle.group_forward(feat.numpy(), index.numpy()))
    go = torch.randn(b, c, n2, k, generator=g, dtype=dtype)
    gin = _C.group_points_backward_cuda(go.to(cuda), index.to(cuda), n1)
    tol = dict(rtol=RTOL, atol=ATOL) if dtype == torch.float32 else dict(rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gin.cpu().numpy(),
                               oracle.group_backward(go.numpy(), index.numpy(), n1, wide=True), **tol)


def test_group_non_contiguous_inputs_and_out_of_range(cuda):
    from torkit3d_amd import _C

    g = gen(1)
    feat = torch.randn(2, 40, 6, generator=g).to(cuda).transpose(1, 2)  # [2,6,40] strided
    index = torch.randint(0, 40, (2, 5, 3), generator=g).to(cuda)
    out = _C.group_points_forward_cuda(feat, index)
    np.testing.assert_array_equal(out.cpu().numpy(),
                                  oracle.group_forward(feat.contiguous().cpu().numpy(), index.cpu().numpy()))
    # ball_query marks rows without a hit with -1: those gather 0 instead of faulting
    index[0, 0, :] = -1
    index[1, 1, 0] = 40
    out = _C.group_points_forward_cuda(feat, index)
    assert float(out[0, :, 0, :].abs().max()) == 0 and float(out[1, :, 1, 0].abs().max()) == 0


@pytest.mark.parametrize("b,c,n1,n2", [(2, 64, 128, 512), (3, 65, 129, 513), (32, 64, 256, 1024),
                                        (32, 64, 2048, 8192)])
def test_interpolate_reference_cases_fp64(cuda, b, c, n1, n2):
    # tests/ops/test_interpolate_feature.py:25-67: fp64, k=3, gather*weight oracle
    from torkit3d_amd.ops.interpolate_feature import interpolate_feature

    torch.manual_seed(0)
    feat = torch.randn(b, c, n1, dtype=torch.float64).to(cuda).requires_grad_()
    index = torch.randint(0, n1, (b, n2, 3)).to(cuda)
    weight = torch.rand(b, n2, 3, dtype=torch.float64).to(cuda)
    weight = weight / weight.sum(2, keepdim=True)
    grouped = feat.unsqueeze(2).expand(b, c, n2, n1).gather(3, index.unsqueeze(1).expand(b, c, n2, 3))
    want = (grouped * weight.unsqueeze(1)).sum(-1)
    got = interpolate_feature(feat, index, weight)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-13)
    go = torch.randn(b, c, n2, dtype=torch.float64, device=cuda)
    got.backward(go)
    mine = feat.grad.clone()
    feat.grad = None
    want.backward(go)
    torch.testing.assert_close(mine, feat.grad, rtol=1e-11, atol=1e-12)


def test_interpolation_config_fp32(cuda):
    # benchmark config 4: knn(3) -> inverse squared distance weights -> interpolate
    # features (32,128,2048) onto 8192 queries, forward and backward
    from torkit3d_amd import _C
    from torkit3d_amd.ops.interpolate_feature import three_nn_weights
    from util import uniform_cloud

    g = gen(4)
    q, key = uniform_cloud(g, 32, 8192), uniform_cloud(g, 32, 2048)
    feat = torch.randn(32, 128, 2048, generator=g)
    d2, idx = _C.knn_distance_cuda(q.to(cuda), key.to(cuda), 3, 1)
    w = three_nn_weights(d2)
    od2, oidx = oracle.knn(q.numpy(), key.numpy(), 3)
    ow = oracle.three_nn_weights(od2)
    np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=RTOL, atol=1e-6)
    out = _C.interpolate_forward_cuda(feat.to(cuda), idx, w)
    want = oracle.interpolate_forward(feat.numpy(), idx.cpu().numpy(), w.cpu().numpy())
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    go = torch.randn(32, 128, 8192, generator=g)
    gin = _C.interpolate_backward_cuda(go.to(cuda), idx, w, 2048)
    ogin = oracle.interpolate_backward(go.numpy(), idx.cpu().numpy(), w.cpu().numpy(), 2048,
                                       wide=True)
    np.testing.assert_allclose(gin.cpu().numpy(), ogin, rtol=RTOL, atol=ATOL)


def test_interpolate_only_k3_through_the_reference_interface(cuda):
    from torkit3d_amd import _C

    feat = torch.zeros(1, 2, 5, device=cuda)
    idx = torch.zeros(1, 4, 2, dtype=torch.int64, device=cuda)
    w = torch.zeros(1, 4, 2, device=cuda)
    with pytest.raises(RuntimeError):
        _C.interpolate_forward_cuda(feat, idx, w)
    with pytest.raises(RuntimeError, match="Only support k=3"):
        _C.interpolate_backward_cuda(torch.zeros(1, 2, 4, device=cuda), idx, w, 5)


def test_fp32_backward_is_bit_reproducible(cuda):
    # fp32 scatters accumulate in 64-bit fixed point: integer adds commute, so repeated
    # calls give identical bits (the reference's float atomics do not)
    from torkit3d_amd import _C

    g = gen(21)
    index = torch.randint(0, 2048, (8, 4096, 3), generator=g).to(cuda)
    weight = torch.rand(8, 4096, 3, generator=g).to(cuda)
    go = torch.randn(8, 64, 4096, generator=g).to(cuda)
    first = _C.interpolate_backward_cuda(go, index, weight, 2048)
    gindex = torch.randint(0, 4096, (8, 1024, 32), generator=g).to(cuda)
    ggo = torch.randn(8, 32, 1024, 32, generator=g).to(cuda)
    gfirst = _C.group_points_backward_cuda(ggo, gindex, 4096)
    a = torch.randn(4, 5000, 3, generator=g).to(cuda)
    c = torch.randn(4, 3000, 3, generator=g).to(cuda)
    _, i1, _, i2 = _C.chamfer_distance_forward_cuda(a, c)
    gd1 = torch.randn(4, 5000, generator=g).to(cuda)
    gd2 = torch.randn(4, 3000, generator=g).to(cuda)
    cfirst = _C.chamfer_distance_backward_cuda(gd1, gd2, a, c, i1, i2)
    for _ in range(3):
        assert torch.equal(_C.interpolate_backward_cuda(go, index, weight, 2048), first)
        assert torch.equal(_C.group_points_backward_cuda(ggo, gindex, 4096), gfirst)
        again = _C.chamfer_distance_backward_cuda(gd1, gd2, a, c, i1, i2)
        assert torch.equal(again[0], cfirst[0]) and torch.equal(again[1], cfirst[1])


@pytest.mark.parametrize("where", [100, 200, 2500, 4095])
def test_scatter_outlier_missed_by_the_magnitude_sample(cuda, where):
    # The fixed-point scale comes from a 1-in-8 sample of the gradient; a term far above
    # the sampled maximum must send the workgroup through its exact second pass.
    from torkit3d_amd import _C

    g = gen(22)
    index = torch.randint(0, 512, (2, 4096, 3), generator=g)
    weight = torch.rand(2, 4096, 3, generator=g)
    go = torch.randn(2, 16, 4096, generator=g)
    go[1, 5, where] = 3.0e7  # 2^25 times a typical term
    got = _C.interpolate_backward_cuda(go.to(cuda), index.to(cuda), weight.to(cuda), 512)
    want = oracle.interpolate_backward(go.numpy(), index.numpy(), weight.numpy(), 512, wide=True)
    got = got.cpu().numpy()
    # the row with the outlier is resolved to 2^-40 of its largest term per sum, every
    # other row to the usual tolerance
    np.testing.assert_allclose(got[1, 5], want[1, 5], rtol=RTOL, atol=3.0e7 * 2.0 ** -40)
    got[1, 5] = want[1, 5]
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    gidx = torch.randint(0, 512, (2, 1024, 4), generator=g)
    ggo = torch.randn(2, 16, 1024, 4, generator=g)
    ggo.view(2, 16, -1)[0, 3, where] = -1.0e8
    got = _C.group_points_backward_cuda(ggo.to(cuda), gidx.to(cuda), 512).cpu().numpy()
    want = oracle.group_backward(ggo.numpy(), gidx.numpy(), 512, wide=True)
    np.testing.assert_allclose(got[0, 3], want[0, 3], rtol=RTOL, atol=1.0e8 * 2.0 ** -40)
    got[0, 3] = want[0, 3]
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_scatter_non_finite_gradients_follow_float_arithmetic(cuda):
    # inf and NaN have no fixed-point image: such a row falls back to float atomics and
    # must give what float addition gives (inf stays inf, inf - inf and NaN give NaN)
    from torkit3d_amd import _C

    g = gen(23)
    index = torch.randint(0, 256, (2, 2048, 3), generator=g)
    weight = torch.rand(2, 2048, 3, generator=g) + 0.1
    go = torch.randn(2, 8, 2048, generator=g)
    go[0, 1, 7] = float("inf")
    go[0, 2, 9] = float("nan")
    go[1, 3, 11] = float("inf")
    go[1, 3, 12] = -float("inf")
    index[1, 12] = index[1, 11]  # +inf and -inf meet in the same rows
    got = _C.interpolate_backward_cuda(go.to(cuda), index.to(cuda), weight.to(cuda), 256).cpu().numpy()
    want = oracle.interpolate_backward(go.numpy(), index.numpy(), weight.numpy(), 256)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isposinf(got), np.isposinf(want))
    assert np.array_equal(np.isneginf(got), np.isneginf(want))
    finite = np.isfinite(want)
    assert np.isnan(want).any() and np.isinf(want).any()
    wide = oracle.interpolate_backward(go.numpy(), index.numpy(), weight.numpy(), 256, wide=True)
    np.testing.assert_allclose(got[finite], wide[finite], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("n1", [16385, 40000, 262144, 300000])
def test_backward_into_rows_longer_than_lds(cuda, n1):
    """Destination rows beyond 16384 points are accumulated in windows (up to 16 of
    them) or, longer still, with global atomics; integer-valued gradients and weights of
    k/4 make every sum exact, so both must equal torch's scatter_add bit for bit."""
    from torkit3d_amd import _C

    g = torch.Generator().manual_seed(n1)
    b, c, n2, k = 2, 5, 3000, 7
    index = torch.randint(0, n1, (b, n2, k), generator=g).to(cuda)
    index[0, :50] = n1 - 1                      # the last destination, many times
    index[1, :50, 0] = 16384                    # first point of the second window
    grad = torch.randint(-3, 4, (b, c, n2, k), generator=g).float().to(cuda)
    got = _C.group_points_backward_cuda(grad, index, n1)
    want = torch.zeros(b, c, n1, device=cuda).scatter_add_(
        2, index.view(b, 1, -1).expand(b, c, -1), grad.view(b, c, -1))
    assert torch.equal(got, want)

    index3 = torch.randint(0, n1, (b, n2, 3), generator=g).to(cuda)
    weight = (torch.randint(0, 5, (b, n2, 3), generator=g).float() / 4).to(cuda)
    grad3 = torch.randint(-2, 3, (b, c, n2), generator=g).float().to(cuda)
    got = _C.interpolate_backward_cuda(grad3, index3, weight, n1)
    want = torch.zeros(b, c, n1, device=cuda)
    for i in range(3):
        want.scatter_add_(2, index3[:, None, :, i].expand(b, c, n2), grad3 * weight[:, None, :, i])
    assert torch.equal(got, want)


@pytest.mark.parametrize("n1", [16385, 32768, 32769])
def test_forward_from_rows_longer_than_64_kib(cuda, n1):
    """Rows up to 128 KiB are staged one at a time, longer ones read through the cache;
    both must equal torch.gather (weights k/4 keep the interpolation sums exact)."""
    from torkit3d_amd import _C

    g = torch.Generator().manual_seed(n1)
    feat = torch.randint(-8, 9, (2, 6, n1), generator=g).float().to(cuda)
    index = torch.randint(0, n1, (2, 3000, 5), generator=g).to(cuda)
    index[0, 0] = n1 - 1
    want = torch.gather(feat, 2, index.view(2, 1, -1).expand(2, 6, -1)).view(2, 6, 3000, 5)
    assert torch.equal(_C.group_points_forward_cuda(feat, index), want)
    index3 = torch.randint(0, n1, (2, 3000, 3), generator=g).to(cuda)
    weight = (torch.randint(0, 5, (2, 3000, 3), generator=g).float() / 4).to(cuda)
    want = torch.zeros(2, 6, 3000, device=cuda)
    for i in range(3):
        want += torch.gather(feat, 2, index3[:, None, :, i].expand(2, 6, 3000)) * weight[:, None, :, i]
    assert torch.equal(_C.interpolate_forward_cuda(feat, index3, weight), want)


@pytest.mark.parametrize("b,c,n1,n2", [
    (40, 64, 300, 1000),    # 640 jobs of 4 rows: workgroups take a second job
    (3, 7, 2000, 777),      # a channel group of 3 at the tail, points not a multiple of 64
    (1, 4, 300, 100000),    # one job per batch: the points are split and merged with atomics
    (2, 5, 5000, 3000),     # rows of 40 KB: one workgroup of 1024 lanes per CU, 2 rows each
    (2, 3, 16000, 500),     # one row fills the LDS
    (1, 1, 1, 1), (2, 2, 5, 63), (1, 130, 64, 65)])
def test_whole_row_scatter_shapes_retries_and_bad_indices(cuda, b, c, n1, n2):
    """The whole-row fp32 scatter: shapes on either side of its launch choices, indices
    outside the row (they contribute nothing), gradients far above the sampled magnitude
    in some rows (those rows are repeated with exact bounds, in a workgroup's first job and
    in a later one) and a NaN and an inf in others (those rows are summed in floating
    point), for interpolation (3 weighted neighbours) and grouping (flattened [n2, 4])."""
    from torkit3d_amd import _C

    g = gen(b * 1000 + c)
    # few jobs: the points are split, and the partial sums (each rounded to fp32) meet in
    # float atomics, a few units in the last place of sums of a thousand terms
    atol = 2e-5 if n2 >= 100000 else ATOL
    for k, weighted in ((3, True), (4, False)):
        index = torch.randint(0, n1, (b, n2, k), generator=g)
        bad = torch.rand(b, n2, k, generator=g) < 0.02
        index[bad] = torch.where(torch.rand(int(bad.sum()), generator=g) < 0.5, -1, n1 + 5)
        go = torch.randn(b, c, n2, generator=g) if weighted else torch.randn(b, c, n2, k, generator=g)
        flat = go.view(b, c, -1)
        big = [(0, 0), (b - 1, c - 1), (b // 2, c // 2), (b - 1, 0)]
        for n, (bi, ci) in enumerate(big):
            flat[bi, ci, (97 * (n + 1)) % flat.shape[2]] = 3.0e7 * (n + 1)
        odd = []
        if b * c > 8:
            odd = [(0, c - 1, float("nan")), (b - 1, c // 3, float("inf"))]
            for bi, ci, v in odd:
                flat[bi, ci, flat.shape[2] // 2] = v
        if weighted:
            weight = torch.rand(b, n2, k, generator=g) + 0.05
            got = _C.interpolate_backward_cuda(go.to(cuda), index.to(cuda), weight.to(cuda), n1)
            want = oracle.interpolate_backward(go.numpy(), index.numpy(), weight.numpy(), n1, wide=True)
        else:
            got = _C.group_points_backward_cuda(go.to(cuda), index.to(cuda), n1)
            want = oracle.group_backward(go.numpy(), index.numpy(), n1, wide=True)
        got = got.cpu().numpy()
        for bi, ci, _ in odd:
            assert np.array_equal(np.isnan(got[bi, ci]), np.isnan(want[bi, ci]))
            assert np.array_equal(np.isposinf(got[bi, ci]), np.isposinf(want[bi, ci]))
            keep = np.isfinite(want[bi, ci])
            np.testing.assert_allclose(got[bi, ci][keep], want[bi, ci][keep], rtol=RTOL, atol=atol)
            got[bi, ci] = want[bi, ci]
        for bi, ci in big:
            if (bi, ci) in [(o[0], o[1]) for o in odd]:
                continue
            # a row is resolved to 2^-40 of its largest term per sum
            top = float(np.abs(flat[bi, ci].numpy()).max()) * (1.05 if weighted else 1.0)
            np.testing.assert_allclose(got[bi, ci], want[bi, ci], rtol=RTOL, atol=top * 2.0 ** -40 + atol)
            got[bi, ci] = want[bi, ci]
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=atol)
