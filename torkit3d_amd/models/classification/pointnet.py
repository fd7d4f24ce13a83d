"""PointNet for classification (torkit3d/models/classification/pointnet.py)."""
import torch
from torch import nn

from ...nn import mlp1d_bn_relu, mlp_bn_relu
from .._common import zero_biases

__all__ = ["PointNet"]


class PointNet(nn.Module):
    """Shared per-point MLP, max pooling over the points, MLP on the pooled vector.
    No op of this package is involved; the model is here so that code importing the
    reference's zoo finds it."""

    def __init__(self, in_channels=3, local_channels=(64, 64, 64, 128, 1024),
                 global_channels=(512, 256)):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = (tuple(local_channels) + tuple(global_channels))[-1]
        self.mlp_local = mlp1d_bn_relu(in_channels, local_channels)
        self.mlp_global = mlp_bn_relu(local_channels[-1], global_channels)
        self.reset_parameters()

    def forward(self, points, points_feature=None, points_mask=None):
        """points [B,3,N], points_feature [B,C,N] or None, points_mask [B,N] bool or None
        -> {"feature": [B, out_channels], "max_indices": [B, local_channels[-1]]}."""
        x = points if points_feature is None else torch.cat([points, points_feature], dim=1)
        x = self.mlp_local(x)
        if points_mask is not None:
            x = torch.where(points_mask.unsqueeze(1), x, torch.zeros_like(x))
        pooled, max_indices = torch.max(x, 2)
        return {"feature": self.mlp_global(pooled), "max_indices": max_indices}

    def reset_parameters(self):
        zero_biases(self, bn_momentum=0.01)
