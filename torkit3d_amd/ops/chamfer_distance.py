"""Chamfer / nearest-neighbour distance (API of torkit3d/ops/chamfer_distance.py)."""
import torch

from .. import _C


def safe_sqrt(x, eps=1e-12):
    """sqrt(max(x, eps)) (torkit3d/ops/chamfer_distance.py:6-7)."""
    return torch.sqrt(torch.clamp(x, eps))


class ChamferDistanceFunction(torch.autograd.Function):
    """forward(xyz1, xyz2) -> (dist1, dist2); backward(grad_dist1, grad_dist2) ->
    (grad_xyz1, grad_xyz2) (torkit3d/ops/chamfer_distance.py:10-29)."""

    @staticmethod
    def forward(ctx, xyz1, xyz2):
        xyz1, xyz2 = xyz1.contiguous(), xyz2.contiguous()
        assert xyz1.is_cuda and xyz2.is_cuda, "Only support cuda currently."
        dist1, idx1, dist2, idx2 = _C.chamfer_distance_forward_cuda(xyz1, xyz2)
        ctx.save_for_backward(xyz1, xyz2, idx1, idx2)
        ctx.mark_non_differentiable(idx1, idx2)
        return dist1, dist2

    @staticmethod
    def backward(ctx, grad_dist1, grad_dist2):
        xyz1, xyz2, idx1, idx2 = ctx.saved_tensors
        grad_dist1, grad_dist2 = grad_dist1.contiguous(), grad_dist2.contiguous()
        assert grad_dist1.is_cuda and grad_dist2.is_cuda, "Only support cuda currently."
        grad_xyz1, grad_xyz2 = _C.chamfer_distance_backward_cuda(
            grad_dist1, grad_dist2, xyz1, xyz2, idx1, idx2)
        return grad_xyz1, grad_xyz2


def _batched(xyz):
    return xyz.unsqueeze(0) if xyz.dim() == 2 else xyz


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
    xyz1, xyz2 = _batched(xyz1), _batched(xyz2)
    if transpose:
        xyz1, xyz2 = xyz1.transpose(1, 2), xyz2.transpose(1, 2)
    dist1, dist2 = ChamferDistanceFunction.apply(xyz1, xyz2)
    if sqrt:
        dist1, dist2 = safe_sqrt(dist1, eps), safe_sqrt(dist2, eps)
    return dist1, dist2


def nn_distance(xyz1, xyz2, transpose=False):
    """Inference form: [dist1, idx1, dist2, idx2], no autograd node
    (torkit3d/ops/chamfer_distance.py:62-71)."""
    xyz1, xyz2 = _batched(xyz1), _batched(xyz2)
    if transpose:
        xyz1 = xyz1.transpose(1, 2).contiguous()
        xyz2 = xyz2.transpose(1, 2).contiguous()
    return _C.chamfer_distance_forward_cuda(xyz1, xyz2)
