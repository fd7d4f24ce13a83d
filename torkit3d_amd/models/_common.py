"""Pieces shared by the models."""
import torch
from torch import nn

from ..nn import batch_index_select
from ..ops.sample_farthest_points import sample_farthest_points, sample_farthest_points_gather


def zero_biases(model, bn_momentum=None):
    """Zero the bias of every convolution / linear layer; optionally set the momentum of
    every batch norm (the models' ``reset_parameters``)."""
    for module in model.modules():
        if isinstance(module, (nn.Linear, nn.Conv1d, nn.Conv2d)) and module.bias is not None:
            nn.init.zeros_(module.bias)
        if bn_momentum is not None and isinstance(module, (nn.BatchNorm1d, nn.BatchNorm2d)):
            module.momentum = bn_momentum


def farthest_points_xyz(points, num_samples):
    """points [B, 3, N] -> coordinates [B, 3, num_samples] of the farthest point sample.

    One kernel emits the indices and the coordinates; the reference runs the sampler
    on a transposed copy and then ``batch_index_select`` (models/segmentation/
    pointnet2.py:89-90). A cloud that needs gradients takes that two-step route, since
    the gather is the differentiable part."""
    if points.requires_grad and torch.is_grad_enabled():
        index = sample_farthest_points(points, num_samples, True)
        return batch_index_select(points, index, dim=2)
    _, xyz = sample_farthest_points_gather(points, num_samples, True)
    return xyz
