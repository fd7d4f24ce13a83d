"""K nearest neighbours with distances (API of torkit3d/ops/knn_points.py)."""
import torch

from .. import _C


class KNNDistanceFunction(torch.autograd.Function):
    """Not differentiable; backward returns None for every input
    (torkit3d/ops/knn_points.py:6-13)."""

    @staticmethod
    def forward(ctx, query_xyz, key_xyz, k, version):
        distance, index = _C.knn_distance_cuda(query_xyz, key_xyz, k, version)
        ctx.mark_non_differentiable(distance, index)
        return distance, index

    @staticmethod
    def backward(ctx, *grad_outputs):
        return (None,) * 4


def knn_points(query, key, k, sorted=False, sqrt_distance=False, transpose=False, version=1):
    """For each query point, its k nearest key points.

    Args:
        query: [B, N1, 3] ([B, 3, N1] if ``transpose``).
        key: [B, N2, 3] ([B, 3, N2] if ``transpose``).
        k: neighbours per query, k <= N2.
        sorted: sort each row by ascending distance.
        sqrt_distance: return Euclidean rather than squared distances.
        transpose: inputs are channel-first.
        version: kernel selector of the reference (0 or 1); results are identical.

    Returns:
        (distance [B, N1, k], index [B, N1, k]) - distance first, as the reference's
        code returns them (torkit3d/ops/knn_points.py:45-51).
    """
    if transpose:
        query, key = query.transpose(1, 2), key.transpose(1, 2)
    query, key = query.contiguous(), key.contiguous()
    distance, index = KNNDistanceFunction.apply(query, key, k, version)
    if sorted:
        distance, order = torch.sort(distance, dim=2)
        index = torch.gather(index, 2, order)
    if sqrt_distance:
        distance = torch.sqrt(distance)
    return distance, index
