"""Entry points that fuse what the reference does in Python around its ops (layout
copies, coordinate gathers, concatenation, weight arithmetic): each must equal the
unfused composition of the ops already checked against the oracle."""
import numpy as np
import pytest
import torch

import oracle
from util import uniform_cloud

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("b,n,k", [(3, 1000, 200), (2, 4096, 1024), (2, 37, 37), (1, 20000, 300)])
def test_fps_either_layout_with_coordinates(cuda, dtype, b, n, k):
    from torkit3d_amd import _C
    from torkit3d_amd.ops.sample_farthest_points import (sample_farthest_points,
                                                          sample_farthest_points_gather)

    pts = uniform_cloud(gen(n), b, n).to(dtype)
    want = oracle.sample_farthest_points(pts.numpy(), k)
    bnc = pts.to(cuda)
    bcn = bnc.transpose(1, 2).contiguous()
    assert np.array_equal(_C.sample_farthest_points_cuda(bnc, k).cpu().numpy(), want)
    assert np.array_equal(sample_farthest_points(bcn, k, transpose=True).cpu().numpy(), want)
    idx, xyz = sample_farthest_points_gather(bnc, k)
    assert np.array_equal(idx.cpu().numpy(), want)
    assert torch.equal(xyz, torch.gather(bnc, 1, idx[:, :, None].expand(-1, -1, 3)))
    idx, xyz = sample_farthest_points_gather(bcn, k, transpose=True)
    assert np.array_equal(idx.cpu().numpy(), want)
    assert torch.equal(xyz, torch.gather(bcn, 2, idx[:, None, :].expand(-1, 3, -1)))


def test_fps_gather_on_duplicates_repeats_the_first_point(cuda):
    from torkit3d_amd.ops.sample_farthest_points import sample_farthest_points_gather

    pts = torch.full((2, 50, 3), 0.25, device=cuda)
    idx, xyz = sample_farthest_points_gather(pts, 7)
    assert int(idx.abs().sum()) == 0 and torch.equal(xyz, pts[:, :7])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("b,n1,n2,r,k", [(2, 300, 1000, 0.2, 16), (1, 70, 257, 0.5, 64),
                                         (3, 128, 4096, 0.1, 32), (2, 5, 3, 10.0, 4)])
def test_ball_query_channels_first(cuda, dtype, b, n1, n2, r, k):
    from torkit3d_amd.ops.ball_query import ball_query

    q, key = uniform_cloud(gen(1), b, n1).to(dtype), uniform_cloud(gen(2), b, n2).to(dtype)
    want = oracle.ball_query(q.numpy(), key.numpy(), r, k)
    got = ball_query(q.to(cuda).transpose(1, 2).contiguous(),
                     key.to(cuda).transpose(1, 2).contiguous(), r, k)  # transpose=True default
    assert np.array_equal(got.cpu().numpy(), want)
    got = ball_query(q.to(cuda), key.to(cuda), r, k, transpose=False)
    assert np.array_equal(got.cpu().numpy(), want)


def unfused_group(feature, xyz, centre, index):
    from torkit3d_amd.ops.group_points import group_points

    nbr_xyz = group_points(xyz, index) - centre.unsqueeze(-1)
    if feature is None:
        return nbr_xyz
    return torch.cat([group_points(feature, index), nbr_xyz], dim=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("b,c,n1,n2,k", [(2, 16, 500, 100, 8), (16, 64, 4096, 1024, 32),
                                         (1, 0, 300, 64, 5), (2, 5, 20000, 77, 3)])
def test_group_points_with_xyz(cuda, dtype, b, c, n1, n2, k):
    from torkit3d_amd.ops.group_points import group_points_with_xyz

    g = gen(c + k)
    feature = torch.randn(b, c, n1, generator=g, dtype=dtype).to(cuda) if c else None
    xyz = torch.rand(b, 3, n1, generator=g, dtype=dtype).to(cuda)
    centre = torch.rand(b, 3, n2, generator=g, dtype=dtype).to(cuda)
    index = torch.randint(0, n1, (b, n2, k), generator=g).to(cuda)
    upstream = torch.randn(b, c + 3, n2, k, generator=g, dtype=dtype).to(cuda)

    leaves = [t.clone().requires_grad_(True) if t is not None else None
              for t in (feature, xyz, centre)]
    out = group_points_with_xyz(leaves[0], leaves[1], leaves[2], index)
    ref_leaves = [t.clone().requires_grad_(True) if t is not None else None
                  for t in (feature, xyz, centre)]
    ref = unfused_group(ref_leaves[0], ref_leaves[1], ref_leaves[2], index)
    assert torch.equal(out, ref)  # copies and one subtraction: bit-identical

    out.backward(upstream)
    # Yardstick for the gradients: the same composition on float64 copies, moved with
    # torch.gather (sums in double, rounded once for the fp32 comparison).
    wide = [t.double().clone().requires_grad_(True) if t is not None else None
            for t in (feature, xyz, centre)]
    flat = index.view(b, 1, n2 * k)
    parts = [torch.gather(wide[1], 2, flat.expand(-1, 3, -1)).view(b, 3, n2, k)
             - wide[2].unsqueeze(-1)]
    if c:
        parts.insert(0, torch.gather(wide[0], 2, flat.expand(-1, c, -1)).view(b, c, n2, k))
    torch.cat(parts, dim=1).backward(upstream.double())
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-12, atol=1e-12)
    for got, want in zip(leaves, wide):
        if got is not None:
            torch.testing.assert_close(got.grad, want.grad.to(dtype), **tol)


def test_group_points_with_xyz_skips_unwanted_gradients(cuda):
    from torkit3d_amd.ops.group_points import group_points_with_xyz

    g = gen(3)
    feature = torch.randn(2, 8, 100, generator=g).to(cuda).requires_grad_(True)
    xyz = torch.rand(2, 3, 100, generator=g).to(cuda)
    centre = torch.rand(2, 3, 10, generator=g).to(cuda)
    index = torch.randint(0, 100, (2, 10, 4), generator=g).to(cuda)
    group_points_with_xyz(feature, xyz, centre, index).sum().backward()
    counts = torch.zeros(2, 100, device=cuda).scatter_add_(
        1, index.reshape(2, -1), torch.ones(2, 40, device=cuda))
    assert torch.equal(feature.grad, counts[:, None, :].expand(-1, 8, -1))
    assert xyz.grad is None and centre.grad is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("b,n1,n2", [(2, 1000, 300), (32, 8192, 2048), (1, 10, 3),
                                     (2, 3000, 4100), (1, 16384, 1024)])
def test_three_nn_matches_knn_and_the_weight_recipe(cuda, dtype, b, n1, n2):
    from torkit3d_amd import _C
    from torkit3d_amd.ops.interpolate_feature import three_nn_interpolation

    q, key = uniform_cloud(gen(4), b, n1).to(dtype), uniform_cloud(gen(5), b, n2).to(dtype)
    qd, kd = q.to(cuda), key.to(cuda)
    want_d, want_i = _C.knn_distance_cuda(qd, kd, 3, 1)
    want_w = oracle.three_nn_weights(want_d.cpu().numpy())
    for transpose in (False, True):
        a, c = (qd.transpose(1, 2).contiguous(), kd.transpose(1, 2).contiguous()) \
            if transpose else (qd, kd)
        d, i, w = three_nn_interpolation(a, c, transpose)
        assert torch.equal(d, want_d) and torch.equal(i, want_i)
        # weights: within 2 ulp of the numpy restatement of pointnet2.py:128-130
        rtol = 3e-7 if dtype == torch.float32 else 5e-16
        np.testing.assert_allclose(w.cpu().numpy(), want_w, rtol=rtol, atol=0)
        np.testing.assert_allclose(w.sum(-1).cpu().numpy(), 1.0, rtol=1e-6)


def test_three_nn_weight_at_zero_distance_uses_eps(cuda):
    from torkit3d_amd.ops.interpolate_feature import three_nn_interpolation

    key = torch.tensor([[[0.0, 0, 0], [1, 0, 0], [0, 1, 0], [5, 5, 5]]], device=cuda)
    d, i, w = three_nn_interpolation(key[:, :1], key, False)
    assert float(d[0, 0, 0]) == 0.0 and int(i[0, 0, 0]) == 0
    want = oracle.three_nn_weights(d.cpu().numpy())
    np.testing.assert_allclose(w.cpu().numpy(), want, rtol=3e-7)
    assert float(w[0, 0, 0]) > 0.999999


def reference_set_abstraction(layer, in_xyz, out_xyz, in_feature):
    """SetAbstraction.forward as the reference writes it (pointnet2.py:42-62)."""
    from torkit3d_amd.ops.ball_query import ball_query

    index = ball_query(out_xyz, in_xyz, layer.query_neighbor.radius,
                       layer.query_neighbor.max_neighbors)
    grouped = unfused_group(in_feature, in_xyz, out_xyz, index)
    return torch.max(layer.mlp(grouped), dim=3)[0]


def reference_feature_propagation(layer, in_xyz, in_feature, out_xyz, out_feature,
                                  fused_weights=False):
    """FeaturePropagation.forward from unfused ops (pointnet2.py:100-105, :125-133).
    ``fused_weights``: take the weights from the fused 3-NN call (they differ from the
    torch recipe by up to 2 ulp, checked on its own), so that the rest of the layer sees
    identical input."""
    from torkit3d_amd.ops.interpolate_feature import (interpolate_feature,
                                                      three_nn_interpolation, three_nn_weights)
    from torkit3d_amd.ops.knn_points import knn_points

    with torch.no_grad():
        distance, index = knn_points(out_xyz, in_xyz, 3, transpose=True)
        weight = three_nn_weights(distance)
        if fused_weights:
            fd, fi, weight = three_nn_interpolation(out_xyz, in_xyz, True)
            assert torch.equal(fd, distance) and torch.equal(fi, index)
    feature = interpolate_feature(in_feature, index, weight)
    if out_feature is not None:
        feature = torch.cat([feature, out_feature], dim=1)
    return layer.mlp(feature)


def test_pointnet2_layers_equal_their_unfused_form(cuda):
    from torkit3d_amd.layers.pointnet2 import BallQuery, FeaturePropagation, SetAbstraction
    from torkit3d_amd.ops.sample_farthest_points import sample_farthest_points_gather

    torch.manual_seed(0)
    g = gen(6)
    xyz = torch.rand(4, 3, 2048, generator=g).to(cuda)
    feature = torch.randn(4, 16, 2048, generator=g).to(cuda)
    _, centres = sample_farthest_points_gather(xyz, 512, transpose=True)

    sa = SetAbstraction(16, [32, 64], BallQuery(0.2, 16), use_xyz=True).to(cuda)
    f1 = feature.clone().requires_grad_(True)
    f2 = feature.clone().requires_grad_(True)
    out = sa(xyz, centres, f1)
    ref = reference_set_abstraction(sa, xyz, centres, f2)
    assert out.shape == (4, 64, 512)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
    out.square().sum().backward()
    ref.square().sum().backward()
    torch.testing.assert_close(f1.grad, f2.grad, rtol=1e-5, atol=1e-6)

    fp = FeaturePropagation(64 + 16, [32]).to(cuda)
    coarse = out.detach()
    c1 = coarse.clone().requires_grad_(True)
    c2 = coarse.clone().requires_grad_(True)
    up = fp(centres, c1, xyz, feature)
    ref = reference_feature_propagation(fp, centres, c2, xyz, feature)
    assert up.shape == (4, 32, 2048)
    torch.testing.assert_close(up, ref, rtol=1e-5, atol=1e-5)
    # Gradients: a 2-ulp difference in the weights is amplified by the batch statistics of
    # the MLP, so the unfused form is given the fused call's weights; what is left to
    # differ is the interpolation's forward and backward, and those must agree.
    ref = reference_feature_propagation(fp, centres, c2, xyz, feature, fused_weights=True)
    torch.testing.assert_close(up, ref, rtol=1e-6, atol=1e-6)
    up.square().sum().backward()
    ref.square().sum().backward()
    torch.testing.assert_close(c1.grad, c2.grad, rtol=1e-5, atol=1e-6)


def test_errors(cuda):
    from torkit3d_amd import _fused

    x = torch.zeros(2, 3, 8, device=cuda)
    with pytest.raises(RuntimeError):
        _fused.ball_query_bcn(x.transpose(1, 2).contiguous(), x, 0.1, 4)  # not [B,3,N]
    with pytest.raises(RuntimeError):
        _fused.three_nn(x[:, :, :2].contiguous(), x[:, :, :2].contiguous(), True)  # N2 < 3
    with pytest.raises(RuntimeError):
        _fused.sample_farthest_points_gather(x, 9, True)
    with pytest.raises(RuntimeError):
        _fused.group_points_concat_forward(None, x, x, torch.zeros(2, 8, 2, device=cuda))


def test_edge_features_match_the_gather_form(cuda):
    # torkit3d/ops/edge_conv.py: the group_points form must equal the torch.gather form
    from torkit3d_amd.ops.edge_conv import (EdgeConvBlock, get_edge_feature_builtin,
                                            get_edge_feature_custom)
    from torkit3d_amd.ops.knn_points import knn_points

    g = gen(8)
    feat = torch.randn(2, 6, 500, generator=g).to(cuda)
    xyz = torch.rand(2, 500, 3, generator=g).to(cuda)
    _, idx = knn_points(xyz, xyz, 8)
    f1 = feat.clone().requires_grad_(True)
    f2 = feat.clone().requires_grad_(True)
    a = get_edge_feature_custom(f1, f1, idx)
    b = get_edge_feature_builtin(f2, f2, idx)
    assert a.shape == (2, 12, 500, 8) and torch.equal(a, b)
    assert torch.equal(get_edge_feature_custom(feat, feat, idx, include_query=False), b[:, :6])
    up = torch.randn(2, 12, 500, 8, generator=g).to(cuda)
    a.backward(up)
    f3 = feat.double().clone().requires_grad_(True)
    get_edge_feature_builtin(f3, f3, idx).backward(up.double())  # torch.gather, sums in double
    torch.testing.assert_close(f1.grad, f3.grad.float(), rtol=1e-5, atol=1e-6)
    torch.manual_seed(0)
    block = EdgeConvBlock(6, [16, 32], checkpoint=True).to(cuda)
    out = block(f1, f1, idx)
    assert out.shape == (2, 32, 500)
    out.sum().backward()
