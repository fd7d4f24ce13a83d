"""Weighted feature interpolation (API of torkit3d/ops/interpolate_feature.py)."""
import torch

from .. import _C, _fused


class InterpolateFeature(torch.autograd.Function):
    """forward(feature, index, weight) -> interpolated; backward ->
    (grad_feature, None, None) (torkit3d/ops/interpolate_feature.py:6-24)."""

    @staticmethod
    def forward(ctx, feature, index, weight):
        ctx.save_for_backward(index, weight)
        ctx.n1 = feature.size(2)
        return _C.interpolate_forward_cuda(
            feature.contiguous(), index.contiguous(), weight.contiguous())

    @staticmethod
    def backward(ctx, *grad_out):
        index, weight = ctx.saved_tensors
        grad_input = _C.interpolate_backward_cuda(
            grad_out[0].contiguous(), index.contiguous(), weight.contiguous(), ctx.n1)
        return grad_input, None, None


def interpolate_feature(feature, index, weight):
    """feature [B, C, N1], index [B, N2, K], weight [B, N2, K] -> [B, C, N2] with
    out[b, c, n] = sum_i feature[b, c, index[b, n, i]] * weight[b, n, i]."""
    return InterpolateFeature.apply(feature, index, weight)


def three_nn_weights(distance, eps=1e-10):
    """Normalised inverse-squared-distance weights used by the reference's
    FeatureInterpolator (torkit3d/layers/pointnet2.py:128-130): ``distance`` is the
    squared distance returned by ``knn_points``."""
    inv_distance = 1.0 / torch.clamp(distance, min=eps)
    return inv_distance / torch.sum(inv_distance, dim=2, keepdim=True)


def three_nn_interpolation(query_xyz, key_xyz, transpose=False, eps=1e-10):
    """Index and weight of the reference's FeatureInterpolator in one kernel:
    ``knn_points(query, key, 3)`` followed by ``three_nn_weights``
    (torkit3d/layers/pointnet2.py:125-130).

    Args:
        query_xyz: [B, N1, 3] ([B, 3, N1] if ``transpose``); key_xyz likewise.

    Returns:
        distance [B, N1, 3] (squared, MinK slot order), index [B, N1, 3] int64,
        weight [B, N1, 3]. Not differentiable, as in the reference (``no_grad``).
    """
    with torch.no_grad():
        return _fused.three_nn(query_xyz.contiguous(), key_xyz.contiguous(), bool(transpose), eps)

three_interpolate = interpolate_feature  # the spelling common elsewhere
