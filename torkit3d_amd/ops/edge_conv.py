"""EdgeConv block and edge features (API of torkit3d/ops/edge_conv.py)."""
import torch
import torch.utils.checkpoint

from ..nn import mlp2d_bn_relu
from .group_points import group_points


def _check_edge_shapes(query_feature, key_feature, key_ind):
    sizes = [query_feature.size(0), key_feature.size(0), key_ind.size(0)]
    assert sizes[0] == sizes[1] == sizes[2], sizes
    assert key_feature.size(1) == query_feature.size(1)
    assert key_ind.size(1) == query_feature.size(2)


def get_edge_feature_builtin(query_feature, key_feature, key_ind, include_query=True):
    """Edge features with stock ``torch.gather`` (torkit3d/ops/edge_conv.py:48-70)."""
    _check_edge_shapes(query_feature, key_feature, key_ind)
    b, c, n1 = query_feature.size()
    n2, k = key_feature.size(2), key_ind.size(2)
    query_expand = query_feature.unsqueeze(3).expand(b, c, n1, k)
    neighbours = torch.gather(key_feature.unsqueeze(2).expand(b, c, n1, n2), 3,
                              key_ind.unsqueeze(1).expand(b, c, n1, k))
    edge_feature = neighbours - query_expand
    if include_query:
        edge_feature = torch.cat([edge_feature, query_expand], dim=1)
    return edge_feature


def get_edge_feature_custom(query_feature, key_feature, key_ind, include_query=True):
    """Edge features through ``group_points`` (torkit3d/ops/edge_conv.py:73-93):
    [key[idx] - query, query] -> [B, 2C, N1, K] ([B, C, N1, K] without the query)."""
    _check_edge_shapes(query_feature, key_feature, key_ind)
    b, c, n1 = query_feature.size()
    query_expand = query_feature.unsqueeze(3).expand(b, c, n1, key_ind.size(2))
    edge_feature = group_points(key_feature, key_ind) - query_expand
    if include_query:
        edge_feature = torch.cat([edge_feature, query_expand], dim=1)
    return edge_feature


get_edge_feature = get_edge_feature_custom


class EdgeConvBlock(torch.nn.Module):
    """EdgeConv block (torkit3d/ops/edge_conv.py:8-45).

    Args:
        in_channels: input channels
        conv_channels (sequence): intermediate channels
        checkpoint: recompute the convolutions in backward to save memory
    """

    def __init__(self, in_channels, conv_channels, checkpoint=False):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = conv_channels[-1]
        self.checkpoint = checkpoint
        self.convs = mlp2d_bn_relu(in_channels * 2, conv_channels)

    def forward(self, query_feature, key_feature, key_ind):
        """query_feature [B,C,N1], key_feature [B,C,N2], key_ind [B,N1,K] -> [B,C',N1]."""
        edge_feature = get_edge_feature(query_feature, key_feature, key_ind)
        if self.checkpoint and edge_feature.requires_grad:
            edge_feature = torch.utils.checkpoint.checkpoint(self.convs, edge_feature,
                                                             use_reentrant=False)
        else:
            edge_feature = self.convs(edge_feature)
        output, _ = edge_feature.max(dim=3)
        return output
