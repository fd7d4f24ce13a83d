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
