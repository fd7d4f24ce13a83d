"""The ``torkit3d.nn`` helpers the layers and models are built from: shared MLPs as
1x1 convolutions or linear layers with batch norm and ReLU
(torkit3d/nn/modules/conv.py, torkit3d/nn/modules/linear.py, torkit3d/nn/modules/mlp.py)
and ``batch_index_select`` (torkit3d/nn/functional.py:34-69). Stock torch modules;
sub-module names match the reference so that its checkpoints load.
"""
import torch
from torch import nn

__all__ = ["Conv1dBNReLU", "Conv2dBNReLU", "LinearBNReLU", "mlp_bn_relu", "mlp1d_bn_relu",
           "mlp2d_bn_relu", "batch_index_select"]


class _ConvBNReLU(nn.Module):
    conv_type = None
    bn_type = None

    def __init__(self, in_channels, out_channels, kernel_size, relu=True, bn=True, **kwargs):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.conv = self.conv_type(in_channels, out_channels, kernel_size, bias=(not bn),
                                   **kwargs)
        self.bn = self.bn_type(out_channels) if bn else None
        self.relu = nn.ReLU(inplace=True) if relu else None

    def forward(self, x):
        x = self.conv(x)
        if self.bn is not None:
            x = self.bn(x)
        if self.relu is not None:
            x = self.relu(x)
        return x


class Conv1dBNReLU(_ConvBNReLU):
    conv_type = nn.Conv1d
    bn_type = nn.BatchNorm1d


class Conv2dBNReLU(_ConvBNReLU):
    conv_type = nn.Conv2d
    bn_type = nn.BatchNorm2d


class LinearBNReLU(nn.Module):
    """``nn.Linear`` (named ``fc``), then optional batch norm and ReLU
    (torkit3d/nn/modules/linear.py:6-27); the bias is dropped when batch norm follows."""

    def __init__(self, in_channels, out_channels, relu=True, bn=True):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.fc = nn.Linear(in_channels, out_channels, bias=(not bn))
        self.bn = nn.BatchNorm1d(out_channels) if bn else None
        self.relu = nn.ReLU(inplace=True) if relu else None

    def forward(self, x):
        x = self.fc(x)
        if self.bn is not None:
            x = self.bn(x)
        if self.relu is not None:
            x = self.relu(x)
        return x


def _mlp(block, in_channels, out_channels_list):
    layers = []
    for out_channels in out_channels_list:
        layers.append(block(in_channels, out_channels, 1, relu=True))
        in_channels = out_channels
    return nn.Sequential(*layers)


def mlp_bn_relu(in_channels, out_channels_list):
    layers = []
    for out_channels in out_channels_list:
        layers.append(LinearBNReLU(in_channels, out_channels, relu=True, bn=True))
        in_channels = out_channels
    return nn.Sequential(*layers)


def mlp1d_bn_relu(in_channels, out_channels_list):
    return _mlp(Conv1dBNReLU, in_channels, out_channels_list)


def mlp2d_bn_relu(in_channels, out_channels_list):
    return _mlp(Conv2dBNReLU, in_channels, out_channels_list)


def batch_index_select(input, index, dim):
    """Batched ``torch.index_select``: input [B, ...], index [B, N] or [B]."""
    squeeze = index.dim() == 1
    if squeeze:
        index = index.unsqueeze(1)
    assert index.dim() == 2, "index is expected to be 2-dim (or 1-dim), but %d received." % index.dim()
    assert input.size(0) == index.size(0), "Mismatched batch size: %d vs %d" % (
        input.size(0), index.size(0))
    view = [1] * input.dim()
    view[0], view[dim] = index.size(0), index.size(1)
    shape = list(input.shape)
    shape[dim] = -1
    out = torch.gather(input, dim, index.view(view).expand(shape))
    return out.squeeze(1) if squeeze else out
