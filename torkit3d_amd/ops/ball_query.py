"""Ball query (API of torkit3d/ops/ball_query.py)."""
from .. import _C, _fused
from ._common import NoGradient


class BallQueryFunction(NoGradient):
    """Not differentiable (torkit3d/ops/ball_query.py:6-14). ``channels_first``
    (not in the reference) says the clouds are [B, 3, N]."""

    @staticmethod
    def run(query, key, radius, max_neighbors, channels_first=False):
        op = _fused.ball_query_bcn if channels_first else _C.ball_query_cuda
        return op(query, key, radius, max_neighbors)


def ball_query(query, key, radius, max_neighbors, transpose=True):
    """Neighbours of each query point within ``radius``.

    Note the default ``transpose=True``: inputs are [B, 3, N] unless told otherwise
    (torkit3d/ops/ball_query.py:17-38).

    Returns:
        index [B, N1, max_neighbors] int64: the first hits in key order, padded with
        the first hit; all -1 where nothing lies within the radius.
    """
    # The reference copies [B, 3, N] clouds to [B, N, 3] here; the kernel reads either.
    query, key = query.contiguous(), key.contiguous()
    return BallQueryFunction.apply(query, key, radius, max_neighbors, bool(transpose))
