"""PointNet++ modules with the reference's constructors and call signatures
(torkit3d/layers/pointnet2.py), built on the fused ops of this package.

Differences from the reference, none of which change the result:
  * ``SetAbstraction`` groups features and centred coordinates into one tensor with
    one op instead of two gathers, a subtraction and ``torch.cat``;
  * ``BallQuery`` and ``FeatureInterpolator`` hand their [B, 3, N] clouds to kernels
    that read that layout, instead of copying them to [B, N, 3];
  * ``FeatureInterpolator`` gets index and weight from one kernel. The reference
    calls ``knn_points`` there without ``transpose=True`` (:127), which its own shape
    check rejects for [B, 3, N] input; this module does what the docstring says.
"""
import torch
from torch import nn

from ..nn import mlp1d_bn_relu, mlp2d_bn_relu
from ..ops.ball_query import ball_query
from ..ops.group_points import group_points, group_points_with_xyz
from ..ops.interpolate_feature import interpolate_feature, three_nn_interpolation
from ..ops.knn_points import knn_points


class SetAbstraction(nn.Module):
    """PointNet++ set abstraction (torkit3d/layers/pointnet2.py:13-68)."""

    def __init__(self, in_channels, mlp_channels, query_neighbor, use_xyz):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = mlp_channels[-1]
        self.query_neighbor = query_neighbor
        self.use_xyz = use_xyz
        self.mlp = mlp2d_bn_relu(in_channels + (3 if use_xyz else 0), mlp_channels)

    def forward(self, in_xyz, out_xyz, in_feature):
        """in_xyz [B,3,N1], out_xyz [B,3,N2], in_feature [B,C1,N1] or None -> [B,C2,N2]."""
        assert in_xyz.size(0) == out_xyz.size(0)
        assert in_xyz.size(1) == out_xyz.size(1) == 3
        with torch.no_grad():
            nbr_index = self.query_neighbor(out_xyz, in_xyz)  # [B, N2, K]
        if self.use_xyz:
            nbr_feature = group_points_with_xyz(in_feature, in_xyz, out_xyz, nbr_index)
        elif in_feature is not None:
            nbr_feature = group_points(in_feature, nbr_index)
        else:
            nbr_feature = in_xyz.new_empty(
                [in_xyz.size(0), 0, nbr_index.size(1), nbr_index.size(2)])
        out_feature = self.mlp(nbr_feature)
        out_feature, _ = torch.max(out_feature, dim=3)
        return out_feature

    def extra_repr(self):
        return "use_xyz={}".format(self.use_xyz)


class BallQuery(nn.Module):
    """(torkit3d/layers/pointnet2.py:71-85); query and key are [B,3,N]."""

    def __init__(self, radius, max_neighbors):
        super().__init__()
        self.radius = radius
        self.max_neighbors = max_neighbors

    def forward(self, query, key):
        return ball_query(query, key, self.radius, self.max_neighbors)

    def extra_repr(self):
        return "radius={}, max_neighbors={}".format(self.radius, self.max_neighbors)


class FeatureInterpolator(nn.Module):
    """(torkit3d/layers/pointnet2.py:108-139): inverse-squared-distance weighted
    interpolation of key features onto the query points."""

    def __init__(self, num_neighbors=3, eps=1e-10):
        super().__init__()
        self.num_neighbors = num_neighbors
        self._eps = eps

    def forward(self, query_xyz, key_xyz, key_feature):
        """query_xyz [B,3,N1], key_xyz [B,3,N2], key_feature [B,C,N2] -> [B,C,N1]."""
        with torch.no_grad():
            if self.num_neighbors == 3:
                _, index, weight = three_nn_interpolation(query_xyz, key_xyz, True, self._eps)
            else:
                distance, index = knn_points(query_xyz, key_xyz, self.num_neighbors,
                                             transpose=True)
                inv_distance = 1.0 / torch.clamp(distance, min=self._eps)
                weight = inv_distance / torch.sum(inv_distance, dim=2, keepdim=True)
        return interpolate_feature(key_feature, index, weight)

    def extra_repr(self):
        return "num_neighbors={}".format(self.num_neighbors)


class FeaturePropagation(nn.Module):
    """PointNet++ feature propagation (torkit3d/layers/pointnet2.py:88-105)."""

    def __init__(self, in_channels, mlp_channels):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = mlp_channels[-1]
        self.mlp = mlp1d_bn_relu(in_channels, mlp_channels)
        self.interpolator = FeatureInterpolator()

    def forward(self, in_xyz, in_feature, out_xyz, out_feature=None):
        interp_feature = self.interpolator(out_xyz, in_xyz, in_feature)
        if out_feature is not None:
            interp_feature = torch.cat([interp_feature, out_feature], dim=1)
        return self.mlp(interp_feature)
