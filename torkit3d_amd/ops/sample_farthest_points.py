"""Farthest point sampling (API of torkit3d/ops/sample_farthest_points.py)."""
import torch

from .. import _C


class SampleFarthestPointsFunction(torch.autograd.Function):
    """Not differentiable (torkit3d/ops/sample_farthest_points.py:6-14)."""

    @staticmethod
    def forward(ctx, points, num_samples):
        index = _C.sample_farthest_points_cuda(points, num_samples)
        ctx.mark_non_differentiable(index)
        return index

    @staticmethod
    def backward(ctx, *grad_outputs):
        return (None,) * 2


def sample_farthest_points(points, num_samples, transpose=False):
    """Indices of ``num_samples`` farthest points per cloud, starting from point 0.

    Args:
        points: [B, N, 3] ([B, 3, N] if ``transpose``).

    Returns:
        index [B, num_samples] int64.
    """
    if transpose:
        points = points.transpose(1, 2)
    points = points.contiguous()
    return SampleFarthestPointsFunction.apply(points, num_samples)
