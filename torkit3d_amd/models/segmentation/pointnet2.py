"""PointNet++ (single-scale grouping) for segmentation
(torkit3d/models/segmentation/pointnet2.py)."""
from torch import nn

from ...layers.pointnet2 import FeaturePropagation
from .._common import descend, set_abstraction_levels, zero_biases

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
        self.sa_layers = set_abstraction_levels(in_channels, _SA_CHANNELS, radius_list,
                                                (max_neighbors,) * 4, use_xyz)
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
        xyz, features = descend(self.sa_layers, self.num_samples, points, points_feature)
        upward = {}
        coarse = features[4]
        for step, fp_layer in enumerate(self.fp_layers):
            level = 3 - step
            coarse = fp_layer(xyz[level + 1], coarse, xyz[level], features[level])
            upward["fp_feature%d" % level] = coarse
        pred_dict = {"feature": coarse}
        pred_dict.update((key, upward[key]) for key in sorted(upward))
        return pred_dict

    def reset_parameters(self):
        zero_biases(self)
