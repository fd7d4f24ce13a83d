"""Chamfer / nearest-neighbour distance (API of torkit3d/ops/chamfer_distance.py)."""
import torch

from .. import _C, _fused
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


class ChamferDistanceChannelsFirstFunction(torch.autograd.Function):
    """The same on [B,3,N] clouds: the forward kernels read them in place (the reference
    copies both to [B,N,3] first, torkit3d/ops/chamfer_distance.py:52-55). The backward
    kernel works on [B,N,3], so the copies are made there, only when gradients are asked for."""

    @staticmethod
    def forward(ctx, xyz1, xyz2):
        clouds = on_gpu(xyz1, xyz2)
        dist1, idx1, dist2, idx2 = _fused.chamfer_forward_bcn(*clouds)
        ctx.save_for_backward(*clouds, idx1, idx2)
        ctx.mark_non_differentiable(idx1, idx2)
        return dist1, dist2

    @staticmethod
    def backward(ctx, grad_dist1, grad_dist2):
        xyz1, xyz2, idx1, idx2 = ctx.saved_tensors
        grads = on_gpu(grad_dist1, grad_dist2)
        g1, g2 = _C.chamfer_distance_backward_cuda(
            *grads, xyz1.transpose(1, 2).contiguous(), xyz2.transpose(1, 2).contiguous(), idx1, idx2)
        return g1.transpose(1, 2), g2.transpose(1, 2)


def _channels_first_in_place(transpose, clouds):
    return transpose and all(c.dim() == 3 and c.is_contiguous() and c.is_cuda for c in clouds)


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
    if _channels_first_in_place(transpose, (xyz1, xyz2)):
        dists = ChamferDistanceChannelsFirstFunction.apply(xyz1, xyz2)
    else:
        clouds = [rows_of_points(with_batch_dim(c), transpose) for c in (xyz1, xyz2)]
        dists = ChamferDistanceFunction.apply(*clouds)
    return tuple(safe_sqrt(d, eps) for d in dists) if sqrt else dists


def nn_distance(xyz1, xyz2, transpose=False):
    """Inference form: [dist1, idx1, dist2, idx2], no autograd node
    (torkit3d/ops/chamfer_distance.py:62-71)."""
    if _channels_first_in_place(transpose, (xyz1, xyz2)):
        return _fused.chamfer_forward_bcn(xyz1, xyz2)
    clouds = [rows_of_points(with_batch_dim(c), transpose) for c in (xyz1, xyz2)]
    if transpose:
        clouds = [c.contiguous() for c in clouds]
    return _C.chamfer_distance_forward_cuda(*clouds)
