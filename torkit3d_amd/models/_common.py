"""Pieces shared by the models."""
import torch
from torch import nn

from ..layers.pointnet2 import BallQuery, SetAbstraction
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


def set_abstraction_levels(in_channels, mlp_channels, radii, neighbors, use_xyz):
    """One ``SetAbstraction`` per level, each fed by the previous level's features."""
    levels = nn.ModuleList()
    for channels, radius, count in zip(mlp_channels, radii, neighbors):
        levels.append(SetAbstraction(in_channels=in_channels, mlp_channels=channels,
                                     query_neighbor=BallQuery(radius=radius, max_neighbors=count),
                                     use_xyz=use_xyz))
        in_channels = channels[-1]
    return levels


def descend(levels, num_samples, points, feature):
    """Runs the levels on prefixes of one farthest point sample (a prefix of a farthest
    point sample is the sample of that size, which is why the reference samples once).

    Returns the coordinates and features of every level, the input cloud first."""
    sampled = farthest_points_xyz(points, num_samples[0])
    xyz, features = [points], [feature]
    for level, count in zip(levels, num_samples):
        xyz.append(sampled[..., :count])
        features.append(level(xyz[-2], xyz[-1], features[-1]))
    return xyz, features
