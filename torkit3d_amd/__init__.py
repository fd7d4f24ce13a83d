"""MI355X (gfx950) implementation of the torkit3d point-cloud operator library.

``torkit3d_amd.ops`` mirrors ``torkit3d.ops`` of the reference (same modules,
function names, argument order, defaults and return order); ``torkit3d_amd._C``
mirrors the reference's compiled extension ``torkit3d._C``. The arithmetic lives in
hand-written HIP kernels behind the C ABI declared in ``include/tk3d.h``.

The functions are also re-exported here, together with the spellings
``knn_distance``, ``farthest_point_sample``, ``gather_points`` and
``three_interpolate``.
"""
from .ops.ball_query import ball_query
from .ops.chamfer_distance import chamfer_distance, nn_distance
from .ops.group_points import group_points
from .ops.interpolate_feature import interpolate_feature, three_nn_weights
from .ops.knn_points import knn_points
from .ops.sample_farthest_points import sample_farthest_points

knn_distance = knn_points
farthest_point_sample = sample_farthest_points
gather_points = group_points
three_interpolate = interpolate_feature

__version__ = "0.1.0"
__all__ = [
    "ball_query", "chamfer_distance", "nn_distance", "group_points", "interpolate_feature",
    "three_nn_weights", "knn_points", "sample_farthest_points", "knn_distance",
    "farthest_point_sample", "gather_points", "three_interpolate",
]
