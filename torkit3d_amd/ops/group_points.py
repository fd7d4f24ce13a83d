"""Group (gather) point features by neighbour index (API of torkit3d/ops/group_points.py)."""
import torch

from .. import _C


class GroupPointsFunction(torch.autograd.Function):
    """forward(points, index) -> grouped; backward -> (grad_points, None)
    (torkit3d/ops/group_points.py:6-19)."""

    @staticmethod
    def forward(ctx, points, index):
        ctx.save_for_backward(index)
        ctx.num_points = points.size(2)
        return _C.group_points_forward_cuda(points.contiguous(), index.contiguous())

    @staticmethod
    def backward(ctx, *grad_output):
        (index,) = ctx.saved_tensors
        grad_input = _C.group_points_backward_cuda(
            grad_output[0].contiguous(), index.contiguous(), ctx.num_points)
        return grad_input, None


def group_points(points, index):
    """points [B, C, N1], index [B, N2, K] -> [B, C, N2, K] with
    out[b, c, m, s] = points[b, c, index[b, m, s]]."""
    return GroupPointsFunction.apply(points, index)
