"""K nearest neighbours with distances (API of torkit3d/ops/knn_points.py)."""
import torch

from .. import _C, _fused
from ._common import NoGradient, rows_of_points


class KNNDistanceFunction(NoGradient):
    """(query_xyz, key_xyz, k, version) -> (distance, index), not differentiable
    (torkit3d/ops/knn_points.py:6-13)."""

    @staticmethod
    def run(query_xyz, key_xyz, k, version):
        return _C.knn_distance_cuda(query_xyz, key_xyz, k, version)


class KNNDistanceChannelsFirstFunction(NoGradient):
    """The same on [B,3,N] clouds, read in place for k <= 64 (the reference copies them to
    [B,N,3] first, torkit3d/ops/knn_points.py:40-45; so does this for larger k)."""

    @staticmethod
    def run(query_xyz, key_xyz, k, version):
        result = _fused.knn_distance_bcn(query_xyz, key_xyz, k, version)
        if result is None:
            result = _C.knn_distance_cuda(query_xyz.transpose(1, 2).contiguous(),
                                          key_xyz.transpose(1, 2).contiguous(), k, version)
        return result


def knn_points(query, key, k, sorted=False, sqrt_distance=False, transpose=False, version=1):
    """The ``k`` key points nearest to every query point: (distance, index), each
    [B, N1, k], in that order (the order of the reference's return statement,
    torkit3d/ops/knn_points.py:45-51, not of its docstring).

    Clouds are [B, N, 3], or [B, 3, N] with ``transpose``; ``k`` may not exceed the
    number of keys. Distances are squared unless ``sqrt_distance``. Rows come in the
    order the reference's top-k structure leaves them unless ``sorted`` (ascending
    distance). ``version`` selects between the reference's two kernels (0 or 1); here
    both values give the same result from the same kernel.
    """
    if (transpose and query.dim() == 3 and key.dim() == 3
            and query.is_contiguous() and key.is_contiguous()):
        distance, index = KNNDistanceChannelsFirstFunction.apply(query, key, k, version)
    else:
        clouds = [rows_of_points(c, transpose).contiguous() for c in (query, key)]
        distance, index = KNNDistanceFunction.apply(*clouds, k, version)
    if sorted:
        distance, order = distance.sort(dim=2)
        index = index.gather(2, order)
    return (distance.sqrt() if sqrt_distance else distance), index

knn_distance = knn_points  # the spelling of the compiled op (knn_distance_cuda)
