"""Chamfer / nearest-neighbour distance (API of torkit3d/ops/chamfer_distance.py)."""
import torch

from .. import _C
from ._common import on_gpu, rows_of_points, with_batch_dim


def safe_sqrt(x, eps=1e-12):
    """sqrt(max(x, eps)) (torkit3d/ops/chamfer_distance.py:6-7)."""
    return torch.clamp(x, eps).sqrt()


class ChamferDistanceFunction(torch.autograd.Function):
    """forward(xyz1, xyz2) -> (dist1, dist2); backward(grad_dist1, grad_dist2) ->
    (grad_xyz1, grad_xyz2) (torkit3d/ops/chamfer_distance.py:10-29). The matches found
    by the forward kernel are kept for the backward kernel, which needs nothing else."""

    @staticmethod
    def forward(ctx, xyz1, xyz2):
        clouds = on_gpu(xyz1, xyz2)
        dist1, idx1, dist2, idx2 = _C.chamfer_distance_forward_cuda(*clouds)
        ctx.save_for_backward(*clouds, idx1, idx2)
        ctx.mark_non_differentiable(idx1, idx2)
        return dist1, dist2

    @staticmethod
    def backward(ctx, grad_dist1, grad_dist2):
        grads = on_gpu(grad_dist1, grad_dist2)
        return tuple(_C.chamfer_distance_backward_cuda(*grads, *ctx.saved_tensors))


def chamfer_distance(xyz1, xyz2, transpose=False, sqrt=False, eps=1e-12):
    """Squared nearest-neighbour distances in both directions, differentiable.

    Args:
        xyz1: (b, n1, 3), or (n1, 3); (b, 3, n1) if ``transpose``.
        xyz2: (b, n2, 3) likewise.
        transpose: inputs are channel-first.
        sqrt: return sqrt(clamp(dist, eps)) instead of squared distances.
        eps: floor used by ``sqrt``.

    Returns:
        dist1 (b, n1), dist2 (b, n2).
    """
    clouds = [rows_of_points(with_batch_dim(c), transpose) for c in (xyz1, xyz2)]
    dists = ChamferDistanceFunction.apply(*clouds)
    return tuple(safe_sqrt(d, eps) for d in dists) if sqrt else dists


def nn_distance(xyz1, xyz2, transpose=False):
    """Inference form: [dist1, idx1, dist2, idx2], no autograd node
    (torkit3d/ops/chamfer_distance.py:62-71)."""
    clouds = [rows_of_points(with_batch_dim(c), transpose) for c in (xyz1, xyz2)]
    if transpose:
        clouds = [c.contiguous() for c in clouds]
    return _C.chamfer_distance_forward_cuda(*clouds)
