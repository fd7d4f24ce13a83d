"""Point-cloud operators with the API of the reference's ``torkit3d.ops`` package.

Module and function names, argument order, defaults and return order follow the
reference file by file (``torkit3d/ops/*.py``); north-star spellings are offered as
aliases at package level.
"""
from .ball_query import ball_query
from .chamfer_distance import chamfer_distance, nn_distance
from .group_points import group_points
from .interpolate_feature import interpolate_feature, three_nn_weights
from .knn_points import knn_points
from .sample_farthest_points import sample_farthest_points

# aliases
knn_distance = knn_points
farthest_point_sample = sample_farthest_points
gather_points = group_points
three_interpolate = interpolate_feature

__all__ = [
    "ball_query", "chamfer_distance", "nn_distance", "group_points", "interpolate_feature",
    "three_nn_weights", "knn_points", "sample_farthest_points", "knn_distance",
    "farthest_point_sample", "gather_points", "three_interpolate",
]
