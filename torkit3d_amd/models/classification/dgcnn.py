"""DGCNN for classification (torkit3d/models/classification/dgcnn.py)."""
import torch
from torch import nn

from ...nn import mlp1d_bn_relu, mlp_bn_relu
from ...ops import native
from ...ops.edge_conv import EdgeConvBlock
from ...ops.knn_points import knn_points
from .._common import zero_biases

__all__ = ["DGCNN"]


def neighbour_index(x, k):
    """Indices [B, N, k] of the k nearest columns of x [B, C, N] to every column.

    Three-channel clouds on the GPU go through the KNN kernel, which reads [B, 3, N] as
    it is and never forms the N x N matrix. Everything else (feature-space neighbours,
    CPU tensors) takes the reference's ``cdist`` + ``topk`` (torkit3d/ops/native.py:4-30).
    The two agree as sets wherever the k-th and (k+1)-th distances differ; EdgeConv
    pools over the neighbours, so their order does not matter."""
    if x.is_cuda and x.size(1) == 3 and x.dtype in (torch.float32, torch.float64):
        with torch.no_grad():
            return knn_points(x, x, k, transpose=True)[1]
    return native.knn(x, x, k, transpose=True)[1]


class DGCNN(nn.Module):
    """EdgeConv blocks on a k-NN graph, concatenated, then PointNet's head."""

    def __init__(self, in_channels=3, edge_conv_channels=(64, 64, 64, 128),
                 local_channels=(1024,), global_channels=(512, 256), k=20, feature_knn=False):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = (tuple(local_channels) + tuple(global_channels))[-1]
        self.k = k
        self.feature_knn = feature_knn

        self.edge_convs = nn.ModuleList()
        widths = []
        c_in = in_channels
        for channels in edge_conv_channels:
            if isinstance(channels, int):
                channels = [channels]
            assert isinstance(channels, (tuple, list))
            self.edge_convs.append(EdgeConvBlock(c_in, channels))
            c_in = channels[-1]
            widths.append(c_in)
        self.mlp_local = mlp1d_bn_relu(sum(widths), local_channels)
        self.mlp_global = mlp_bn_relu(local_channels[-1], global_channels)
        self.reset_parameters()

    def forward(self, points, points_feature=None, knn_ind=None):
        """points [B,3,N], points_feature [B,C,N] or None, knn_ind [B,N,k] or None
        -> {"feature": [B, out_channels], "max_indices": [B, local_channels[-1]]}.

        The graph is built once on the coordinates unless ``feature_knn``, in which case
        every block after the first rebuilds it on its input features."""
        x = points if points_feature is None else torch.cat([points, points_feature], dim=1)
        outputs = []
        for edge_conv in self.edge_convs:
            if knn_ind is None:
                knn_ind = neighbour_index(points, self.k)
            elif self.feature_knn:
                knn_ind = neighbour_index(x, self.k)
            x = edge_conv(x, x, knn_ind)
            outputs.append(x)
        x = self.mlp_local(torch.cat(outputs, dim=1))
        pooled, max_indices = torch.max(x, 2)
        return {"feature": self.mlp_global(pooled), "max_indices": max_indices}

    def reset_parameters(self):
        zero_biases(self, bn_momentum=0.01)
