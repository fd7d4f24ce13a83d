"""Farthest point sampling (API of torkit3d/ops/sample_farthest_points.py)."""
import torch

from .. import _C, _fused
from ._common import NoGradient


class SampleFarthestPointsFunction(NoGradient):
    """Not differentiable (torkit3d/ops/sample_farthest_points.py:6-14).
    ``channels_first`` (not in the reference) says the cloud is [B, 3, N]."""

    @staticmethod
    def run(points, num_samples, channels_first=False):
        if channels_first:
            return _fused.sample_farthest_points_gather(points, num_samples, True,
                                                        want_xyz=False)[0]
        return _C.sample_farthest_points_cuda(points, num_samples)


def sample_farthest_points(points, num_samples, transpose=False):
    """Indices of ``num_samples`` farthest points per cloud, starting from point 0.

    Args:
        points: [B, N, 3] ([B, 3, N] if ``transpose``).

    Returns:
        index [B, num_samples] int64.
    """
    # The reference copies a [B, 3, N] cloud to [B, N, 3] here; the kernel reads either.
    return SampleFarthestPointsFunction.apply(points.contiguous(), num_samples, bool(transpose))


def sample_farthest_points_gather(points, num_samples, transpose=False):
    """``sample_farthest_points`` plus the coordinates of the picks, from the same
    kernel (the reference's models follow the op with
    ``batch_index_select(points, index, dim=2)``, models/segmentation/pointnet2.py:89-90).

    Returns:
        index [B, num_samples] int64, sampled [B, num_samples, 3]
        ([B, 3, num_samples] if ``transpose``). Not differentiable.
    """
    with torch.no_grad():
        return _fused.sample_farthest_points_gather(points.contiguous(), num_samples,
                                                    bool(transpose))

farthest_point_sample = sample_farthest_points  # the spelling common elsewhere
