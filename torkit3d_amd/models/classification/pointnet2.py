"""PointNet++ (single-scale grouping) for classification
(torkit3d/models/classification/pointnet2.py)."""
import torch
from torch import nn

from ...nn import mlp1d_bn_relu
from .._common import descend, set_abstraction_levels, zero_biases

__all__ = ["PN2SSG"]


class PN2SSG(nn.Module):
    """Set abstraction levels on prefixes of one farthest point sample, a shared MLP
    and max pooling. The defaults are the reference's (ModelNet40)."""

    def __init__(self, in_channels=0, sa_channels=((64, 64, 128), (128, 128, 256)),
                 num_samples=(512, 128), radius_list=(0.2, 0.4), num_neighbors=(32, 64),
                 local_channels=(256, 512, 1024), use_xyz=True):
        super().__init__()
        assert len(sa_channels) == len(num_samples) == len(radius_list) == len(num_neighbors)
        self.in_channels = in_channels
        self.out_channels = local_channels[-1]
        self.sa_channels = sa_channels
        self.num_samples = num_samples
        self.radius_list = radius_list
        self.num_neighbors = num_neighbors
        self.use_xyz = use_xyz
        self.sa_layers = set_abstraction_levels(in_channels, sa_channels, radius_list,
                                                num_neighbors, use_xyz)
        self.mlp_local = mlp1d_bn_relu(sa_channels[-1][-1], local_channels)
        self.reset_parameters()

    def forward(self, points, points_feature=None):
        """points [B,3,N], points_feature [B,C,N] or None
        -> {"feature": [B, out_channels], "max_indices": [B, out_channels]}."""
        _, features = descend(self.sa_layers, self.num_samples, points, points_feature)
        pooled, max_indices = torch.max(self.mlp_local(features[-1]), 2)
        return {"feature": pooled, "max_indices": max_indices}

    def reset_parameters(self):
        zero_biases(self)
