"""PointNet++ (single-scale grouping) for segmentation
(torkit3d/models/segmentation/pointnet2.py)."""
from torch import nn

from ...layers.pointnet2 import BallQuery, FeaturePropagation, SetAbstraction
from .._common import farthest_points_xyz, zero_biases

__all__ = ["PN2SSG"]

_SA_CHANNELS = ((32, 32, 64), (64, 64, 128), (128, 128, 256), (256, 256, 512))


class PN2SSG(nn.Module):
    """Four set abstraction levels down, four feature propagation levels back up to
    per-point features. The defaults are the reference's (ScanNet)."""

    def __init__(self, in_channels=0, num_samples=(2048, 512, 128, 32),
                 radius_list=(0.1, 0.2, 0.4, 0.8), max_neighbors=32, use_xyz=True):
        super().__init__()
        assert len(num_samples) == len(radius_list) == 4
        self.in_channels = in_channels
        self.out_channels = 128 + in_channels
        self.num_samples = num_samples
        self.use_xyz = use_xyz

        self.sa_layers = nn.ModuleList()
        c_in = in_channels
        for channels, radius in zip(_SA_CHANNELS, radius_list):
            self.sa_layers.append(SetAbstraction(
                in_channels=c_in, mlp_channels=channels,
                query_neighbor=BallQuery(radius=radius, max_neighbors=max_neighbors),
                use_xyz=use_xyz))
            c_in = channels[-1]

        # (coarse features + skip features, MLP) from the coarsest level upwards.
        self.fp_layers = nn.ModuleList([
            FeaturePropagation(in_channels=512 + 256, mlp_channels=(256, 256)),
            FeaturePropagation(in_channels=256 + 128, mlp_channels=(256, 256)),
            FeaturePropagation(in_channels=256 + 64, mlp_channels=(256, 128)),
            FeaturePropagation(in_channels=128 + in_channels, mlp_channels=(128, 128, 128)),
        ])
        self.reset_parameters()

    def forward(self, points, points_feature=None):
        """points [B,3,N], points_feature [B,C,N] or None -> {"feature": [B,128,N],
        "fp_feature0".."fp_feature3": the output of every propagation level}."""
        xyz_fps = farthest_points_xyz(points, self.num_samples[0])

        xyz = [points]
        feature = [points_feature]
        for sa_layer, count in zip(self.sa_layers, self.num_samples):
            # A prefix of a farthest point sample is the sample of that size.
            xyz.append(xyz_fps[..., :count])
            feature.append(sa_layer(xyz[-2], xyz[-1], feature[-1]))

        outputs = {}
        coarse = feature[4]
        for step, fp_layer in enumerate(self.fp_layers):
            level = 3 - step
            coarse = fp_layer(xyz[level + 1], coarse, xyz[level], feature[level])
            outputs["fp_feature%d" % level] = coarse
        pred_dict = {"feature": coarse}
        for level in range(4):
            pred_dict["fp_feature%d" % level] = outputs["fp_feature%d" % level]
        return pred_dict

    def reset_parameters(self):
        zero_biases(self)
