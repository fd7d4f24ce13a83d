"""Group (gather) point features by neighbour index (API of torkit3d/ops/group_points.py)."""
import torch

from .. import _C, _fused


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


class GroupPointsWithXYZFunction(torch.autograd.Function):
    """forward(feature or None, xyz, centre, index) -> [B, C+3, N2, K];
    backward -> (grad_feature, grad_xyz, grad_centre, None)."""

    @staticmethod
    def forward(ctx, feature, xyz, centre, index):
        ctx.save_for_backward(index)
        ctx.num_points = xyz.size(2)
        ctx.has_feature = feature is not None
        return _fused.group_points_concat_forward(
            feature.contiguous() if feature is not None else None, xyz.contiguous(),
            centre.contiguous(), index.contiguous())

    @staticmethod
    def backward(ctx, *grad_output):
        (index,) = ctx.saved_tensors
        need_feature = ctx.has_feature and ctx.needs_input_grad[0]
        need_xyz, need_centre = ctx.needs_input_grad[1], ctx.needs_input_grad[2]
        grad = grad_output[0].contiguous()
        grad_feature, grad_xyz = _fused.group_points_concat_backward(
            grad, index.contiguous(), ctx.num_points, need_feature, need_xyz)
        grad_centre = -grad[:, grad.size(1) - 3:].sum(dim=3) if need_centre else None
        return grad_feature, grad_xyz, grad_centre, None


def group_points_with_xyz(feature, xyz, centre, index):
    """The grouping step of the reference's SetAbstraction with ``use_xyz``
    (torkit3d/layers/pointnet2.py:46-58) as one op: equal to
    ``torch.cat([group_points(feature, index), group_points(xyz, index) -
    centre.unsqueeze(-1)], dim=1)``, written once.

    Args:
        feature: [B, C, N1] or None; xyz: [B, 3, N1]; centre: [B, 3, N2];
        index: [B, N2, K] int64.
    """
    return GroupPointsWithXYZFunction.apply(feature, xyz, centre, index)

gather_points = group_points  # the spelling common elsewhere
