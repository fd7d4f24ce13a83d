"""The Python layer keeps the reference's API: module paths, function names,
argument names, defaults, and host-side error behaviour (checked on CPU tensors)."""
import inspect

import pytest
import torch

import torkit3d_amd
from torkit3d_amd import _C
from torkit3d_amd.ops import (ball_query, chamfer_distance, group_points, interpolate_feature,
                              knn_points, native, sample_farthest_points)


def params(fn):
    return [(p.name, p.default) for p in inspect.signature(fn).parameters.values()]


E = inspect.Parameter.empty


def test_signatures_match_the_reference():
    # torkit3d/ops/chamfer_distance.py:32,62; knn_points.py:16-24; ball_query.py:17-19;
    # sample_farthest_points.py:17; group_points.py:22; interpolate_feature.py:27-29;
    # native.py:4-10
    assert params(chamfer_distance.chamfer_distance) == [
        ("xyz1", E), ("xyz2", E), ("transpose", False), ("sqrt", False), ("eps", 1e-12)]
    assert params(chamfer_distance.nn_distance) == [("xyz1", E), ("xyz2", E), ("transpose", False)]
    assert params(knn_points.knn_points) == [
        ("query", E), ("key", E), ("k", E), ("sorted", False), ("sqrt_distance", False),
        ("transpose", False), ("version", 1)]
    assert params(ball_query.ball_query) == [
        ("query", E), ("key", E), ("radius", E), ("max_neighbors", E), ("transpose", True)]
    assert params(sample_farthest_points.sample_farthest_points) == [
        ("points", E), ("num_samples", E), ("transpose", False)]
    assert params(group_points.group_points) == [("points", E), ("index", E)]
    assert params(interpolate_feature.interpolate_feature) == [
        ("feature", E), ("index", E), ("weight", E)]
    assert params(native.knn) == [
        ("query", E), ("key", E), ("k", E), ("sorted", False), ("transpose", False)]


def test_autograd_function_classes_exist():
    for mod, name in ((chamfer_distance, "ChamferDistanceFunction"),
                      (knn_points, "KNNDistanceFunction"), (ball_query, "BallQueryFunction"),
                      (sample_farthest_points, "SampleFarthestPointsFunction"),
                      (group_points, "GroupPointsFunction"),
                      (interpolate_feature, "InterpolateFeature")):
        assert issubclass(getattr(mod, name), torch.autograd.Function)


def test_extension_module_exports_the_nine_symbols():
    # torkit3d/csrc/torkit3d.cpp:13-21
    want = {"sample_farthest_points_cuda", "ball_query_cuda", "group_points_forward_cuda",
            "group_points_backward_cuda", "interpolate_forward_cuda", "interpolate_backward_cuda",
            "knn_distance_cuda", "chamfer_distance_forward_cuda", "chamfer_distance_backward_cuda"}
    assert want == set(_C.__all__)
    for name in want:
        assert callable(getattr(_C, name))


def test_aliases():
    assert torkit3d_amd.knn_distance is knn_points.knn_points
    assert torkit3d_amd.farthest_point_sample is sample_farthest_points.sample_farthest_points
    assert torkit3d_amd.gather_points is group_points.group_points
    assert torkit3d_amd.three_interpolate is interpolate_feature.interpolate_feature


def test_cpu_tensors_are_rejected_like_the_reference():
    x = torch.zeros(1, 4, 3)
    idx = torch.zeros(1, 4, 3, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.knn_distance_cuda(x, x, 2, 1)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.sample_farthest_points_cuda(x, 2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.ball_query_cuda(x, x, 0.1, 2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.group_points_forward_cuda(x, idx)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.interpolate_forward_cuda(x, idx, x)
    with pytest.raises(AssertionError, match="Only support cuda"):
        chamfer_distance.chamfer_distance(x, x)  # torkit3d/ops/chamfer_distance.py:15


def test_native_knn_runs_on_cpu():
    g = torch.Generator().manual_seed(0)
    q, key = torch.randn(2, 10, 3, generator=g), torch.randn(2, 30, 3, generator=g)
    d, i = native.knn(q, key, 4, sorted=True)
    want = torch.cdist(q, key).sort(dim=2)
    assert torch.equal(i, want.indices[:, :, :4]) and torch.allclose(d, want.values[:, :, :4])
    d2, i2 = native.knn(q.transpose(1, 2), key.transpose(1, 2), 4, sorted=True, transpose=True)
    assert torch.equal(i, i2)


def test_three_nn_weights_matches_reference_recipe():
    d2 = torch.tensor([[[0.0, 1.0, 4.0]]])
    w = interpolate_feature.three_nn_weights(d2)
    inv = 1.0 / torch.clamp(d2, min=1e-10)
    assert torch.equal(w, inv / inv.sum(2, keepdim=True))


def test_layers_keep_the_reference_constructors():
    # torkit3d/layers/pointnet2.py:16, :72, :91, :109 and the sub-module names its
    # checkpoints are keyed by (torkit3d/nn/modules/conv.py:18-23)
    from torkit3d_amd.layers import pointnet2

    assert params(pointnet2.SetAbstraction.__init__)[1:] == [
        ("in_channels", E), ("mlp_channels", E), ("query_neighbor", E), ("use_xyz", E)]
    assert params(pointnet2.BallQuery.__init__)[1:] == [("radius", E), ("max_neighbors", E)]
    assert params(pointnet2.FeaturePropagation.__init__)[1:] == [
        ("in_channels", E), ("mlp_channels", E)]
    assert params(pointnet2.FeatureInterpolator.__init__)[1:] == [
        ("num_neighbors", 3), ("eps", 1e-10)]
    assert params(pointnet2.SetAbstraction.forward)[1:] == [
        ("in_xyz", E), ("out_xyz", E), ("in_feature", E)]
    assert params(pointnet2.FeaturePropagation.forward)[1:] == [
        ("in_xyz", E), ("in_feature", E), ("out_xyz", E), ("out_feature", None)]
    sa = pointnet2.SetAbstraction(4, [8, 16], pointnet2.BallQuery(0.2, 8), True)
    assert sorted(sa.state_dict()) == sorted(
        ["mlp.%d.%s" % (i, k) for i in range(2) for k in (
            "conv.weight", "bn.weight", "bn.bias", "bn.running_mean", "bn.running_var",
            "bn.num_batches_tracked")])
    assert sa.mlp[0].conv.in_channels == 7 and sa.out_channels == 16
    fp = pointnet2.FeaturePropagation(10, [6])
    assert "mlp.0.conv.weight" in fp.state_dict() and fp.mlp[0].conv.kernel_size == (1,)


def test_batch_index_select_is_a_batched_gather():
    from torkit3d_amd.nn import batch_index_select

    x = torch.arange(2 * 3 * 5.0).reshape(2, 3, 5)
    idx = torch.tensor([[4, 0], [1, 1]])
    out = batch_index_select(x, idx, dim=2)
    assert out.shape == (2, 3, 2)
    assert torch.equal(out[0], x[0][:, [4, 0]]) and torch.equal(out[1], x[1][:, [1, 1]])
    assert torch.equal(batch_index_select(x, torch.tensor([2, 0]), dim=1),
                       torch.stack([x[0, 2], x[1, 0]]))


def test_fused_entry_points_reject_cpu_tensors():
    from torkit3d_amd import _fused

    x = torch.zeros(1, 3, 8)
    idx = torch.zeros(1, 8, 2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _fused.ball_query_bcn(x, x, 0.1, 2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _fused.sample_farthest_points_gather(x, 2, True)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _fused.three_nn(x, x, True)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _fused.group_points_concat_forward(None, x, x, idx)


def test_edge_conv_module_keeps_the_reference_api():
    # torkit3d/ops/edge_conv.py:17, :48-50, :73-75, :96-97
    from torkit3d_amd.ops import edge_conv

    assert params(edge_conv.EdgeConvBlock.__init__)[1:] == [
        ("in_channels", E), ("conv_channels", E), ("checkpoint", False)]
    want = [("query_feature", E), ("key_feature", E), ("key_ind", E), ("include_query", True)]
    assert params(edge_conv.get_edge_feature_builtin) == want
    assert params(edge_conv.get_edge_feature_custom) == want
    assert edge_conv.get_edge_feature is edge_conv.get_edge_feature_custom
    block = edge_conv.EdgeConvBlock(3, [8])
    assert "convs.0.conv.weight" in block.state_dict() and block.convs[0].conv.in_channels == 6
    q = torch.randn(1, 3, 5)
    idx = torch.tensor([[[0, 1], [1, 2], [2, 3], [3, 4], [4, 0]]])
    edge = edge_conv.get_edge_feature_builtin(q, q, idx)
    assert edge.shape == (1, 6, 5, 2)
    assert torch.equal(edge[0, :3, 0, 1], q[0, :, 1] - q[0, :, 0])
    assert torch.equal(edge[0, 3:, 2, 0], q[0, :, 2])


def test_model_zoo_keeps_the_reference_constructors_and_parameter_names():
    # torkit3d/models/classification/pointnet.py:17-22, dgcnn.py:19-27, pointnet2.py:20-29,
    # torkit3d/models/segmentation/pointnet2.py:19-26
    from torkit3d_amd.models.classification.dgcnn import DGCNN
    from torkit3d_amd.models.classification.pointnet import PointNet
    from torkit3d_amd.models.classification.pointnet2 import PN2SSG as PN2Cls
    from torkit3d_amd.models.segmentation.pointnet2 import PN2SSG as PN2Seg

    assert params(PointNet.__init__)[1:] == [
        ("in_channels", 3), ("local_channels", (64, 64, 64, 128, 1024)),
        ("global_channels", (512, 256))]
    assert params(DGCNN.__init__)[1:] == [
        ("in_channels", 3), ("edge_conv_channels", (64, 64, 64, 128)),
        ("local_channels", (1024,)), ("global_channels", (512, 256)), ("k", 20),
        ("feature_knn", False)]
    assert params(PN2Cls.__init__)[1:] == [
        ("in_channels", 0), ("sa_channels", ((64, 64, 128), (128, 128, 256))),
        ("num_samples", (512, 128)), ("radius_list", (0.2, 0.4)), ("num_neighbors", (32, 64)),
        ("local_channels", (256, 512, 1024)), ("use_xyz", True)]
    assert params(PN2Seg.__init__)[1:] == [
        ("in_channels", 0), ("num_samples", (2048, 512, 128, 32)),
        ("radius_list", (0.1, 0.2, 0.4, 0.8)), ("max_neighbors", 32), ("use_xyz", True)]
    assert params(PointNet.forward)[1:] == [("points", E), ("points_feature", None),
                                            ("points_mask", None)]
    assert params(DGCNN.forward)[1:] == [("points", E), ("points_feature", None),
                                         ("knn_ind", None)]

    def conv_bn_weights(cin, widths):
        total = 0
        for w in widths:
            total += cin * w + 2 * w  # bias-free 1x1 conv or linear, batch norm scale + shift
            cin = w
        return total

    net = PointNet(6)
    assert net.out_channels == 256
    assert sum(p.numel() for p in net.parameters()) == (
        conv_bn_weights(6, (64, 64, 64, 128, 1024)) + conv_bn_weights(1024, (512, 256)))
    keys = set(net.state_dict())
    assert {"mlp_local.4.conv.weight", "mlp_local.0.bn.running_var",
            "mlp_global.1.fc.weight", "mlp_global.1.bn.bias"} <= keys
    assert not any(k.endswith("conv.bias") or k.endswith("fc.bias") for k in keys)
    assert all(m.momentum == 0.01 for m in net.modules()
               if isinstance(m, (torch.nn.BatchNorm1d, torch.nn.BatchNorm2d)))

    net = DGCNN(3)
    assert net.out_channels == 256 and net.k == 20
    assert sum(p.numel() for p in net.parameters()) == (
        conv_bn_weights(6, (64,)) + conv_bn_weights(128, (64,)) + conv_bn_weights(128, (64,))
        + conv_bn_weights(128, (128,)) + conv_bn_weights(320, (1024,))
        + conv_bn_weights(1024, (512, 256)))
    assert {"edge_convs.3.convs.0.conv.weight", "mlp_local.0.conv.weight",
            "mlp_global.0.fc.weight"} <= set(net.state_dict())
    assert DGCNN(3, edge_conv_channels=(8, (8, 16))).edge_convs[1].convs[1].conv.out_channels == 16

    net = PN2Cls(0)
    assert net.out_channels == 1024
    assert sum(p.numel() for p in net.parameters()) == (
        conv_bn_weights(3, (64, 64, 128)) + conv_bn_weights(131, (128, 128, 256))
        + conv_bn_weights(256, (256, 512, 1024)))
    assert net.sa_layers[1].query_neighbor.radius == 0.4
    assert net.sa_layers[1].query_neighbor.max_neighbors == 64
    assert PN2Cls(5, use_xyz=False, sa_channels=((8,), (8,)), local_channels=(8,)
                  ).sa_layers[0].mlp[0].conv.in_channels == 5

    net = PN2Seg(4)
    assert net.out_channels == 132 and net.in_channels == 4
    assert sum(p.numel() for p in net.parameters()) == (
        conv_bn_weights(7, (32, 32, 64)) + conv_bn_weights(67, (64, 64, 128))
        + conv_bn_weights(131, (128, 128, 256)) + conv_bn_weights(259, (256, 256, 512))
        + conv_bn_weights(768, (256, 256)) + conv_bn_weights(384, (256, 256))
        + conv_bn_weights(320, (256, 128)) + conv_bn_weights(132, (128, 128, 128)))
    assert {"sa_layers.3.mlp.2.conv.weight", "fp_layers.3.mlp.2.bn.weight",
            "fp_layers.0.mlp.0.conv.weight"} <= set(net.state_dict())
    assert [l.query_neighbor.radius for l in net.sa_layers] == [0.1, 0.2, 0.4, 0.8]


def test_pointnet_runs_on_cpu_with_feature_and_mask():
    from torkit3d_amd.models.classification.pointnet import PointNet

    torch.manual_seed(0)
    net = PointNet(5, local_channels=(8, 16), global_channels=(4,)).eval()
    points, feature = torch.randn(3, 3, 20), torch.randn(3, 2, 20)
    mask = torch.ones(3, 20, dtype=torch.bool)
    mask[:, 10:] = False
    out = net(points, feature, mask)
    assert out["feature"].shape == (3, 4) and out["max_indices"].shape == (3, 16)
    # Masked points contribute zeros, which post-ReLU features can only tie, never beat.
    short = net(points[..., :10], feature[..., :10])
    torch.testing.assert_close(out["feature"], short["feature"])


def test_other_spellings_of_the_ops():
    # knn_distance (the compiled op's name), farthest_point_sample, three_interpolate and
    # gather_points name the same functions, in the op modules and at the package root
    import torkit3d_amd
    from torkit3d_amd.ops import group_points, interpolate_feature, knn_points, sample_farthest_points

    assert knn_points.knn_distance is knn_points.knn_points
    assert sample_farthest_points.farthest_point_sample is sample_farthest_points.sample_farthest_points
    assert interpolate_feature.three_interpolate is interpolate_feature.interpolate_feature
    assert group_points.gather_points is group_points.group_points
    assert torkit3d_amd.knn_distance is knn_points.knn_points
    assert torkit3d_amd.farthest_point_sample is sample_farthest_points.sample_farthest_points
