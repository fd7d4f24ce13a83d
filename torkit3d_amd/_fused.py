"""Shim for the entry points of ``include/tk3d.h`` that have no counterpart among the
nine ``torkit3d._C`` functions: they fuse steps the reference performs in Python
around those functions (layout copies, coordinate gathers, concatenation, weight
arithmetic). Same conventions as ``_C``: tensors are validated, outputs allocated with
torch, raw device pointers and torch's current stream go to the C ABI.
"""
import ctypes

import torch

from . import _lib
from ._C import _check, _check_contiguous_cuda, _check_eq, _check_index, _check_same
from ._lib import i64, ptr, stream_of

__all__ = [
    "sample_farthest_points_gather",
    "ball_query_bcn",
    "knn_distance_bcn",
    "chamfer_forward_bcn",
    "group_points_concat_forward",
    "group_points_concat_backward",
    "three_nn",
]


def _cloud_dims(name, t, channels_first):
    _check_contiguous_cuda(name, t)
    _check_eq(t.dim(), 3, "%s.dim() == 3" % name)
    _check_eq(t.size(1 if channels_first else 2), 3,
              "%s.size(%d) == 3" % (name, 1 if channels_first else 2))
    return t.size(0), t.size(2 if channels_first else 1)


def sample_farthest_points_gather(points, num_samples, channels_first, want_xyz=True):
    """points [B,N,3] (or [B,3,N] with ``channels_first``) -> (index [B,K] int64,
    sampled [B,K,3] (or [B,3,K]) or None). ``index`` equals
    ``_C.sample_farthest_points_cuda`` on the [B,N,3] cloud."""
    b, n = _cloud_dims("points", points, channels_first)
    num_samples = int(num_samples)
    _check(num_samples > 0, "Check failed: num_samples > 0 (%d vs. 0)" % num_samples)
    _check(n >= num_samples,
           "Check failed: points.size(1) >= num_samples (%d vs. %d)" % (n, num_samples))
    with _lib.on_device_of(points):
        index = torch.empty((b, num_samples), dtype=torch.int64, device=points.device)
        sampled = None
        if want_xyz:
            shape = (b, 3, num_samples) if channels_first else (b, num_samples, 3)
            sampled = torch.empty(shape, dtype=points.dtype, device=points.device)
        ws_bytes = _lib.fps_workspace_bytes(b, n, points.element_size())
        ws = None
        if ws_bytes:
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=points.device)
        _lib.call("tk3d_sample_farthest_points_gather", points, ptr(points),
                  ctypes.c_int(1 if channels_first else 0), i64(b), i64(n), i64(num_samples),
                  ptr(index), ptr(sampled) if sampled is not None else ctypes.c_void_p(0),
                  ctypes.c_void_p(ws.data_ptr() if ws is not None else 0),
                  ctypes.c_size_t(ws_bytes), stream_of(points))
    return index, sampled


def ball_query_bcn(query, key, radius, max_neighbors):
    """query [B,3,N1], key [B,3,N2] -> index [B,N1,max_neighbors] int64; equals
    ``_C.ball_query_cuda`` on the transposed clouds."""
    b, n1 = _cloud_dims("query", query, True)
    b2, n2 = _cloud_dims("key", key, True)
    _check_eq(b, b2, "query.size(0) == key.size(0)")
    _check_same("query", query, "key", key)
    max_neighbors = int(max_neighbors)
    _check(max_neighbors >= 0, "max_neighbors must be non-negative.")
    with _lib.on_device_of(query):
        index = torch.empty((b, n1, max_neighbors), dtype=torch.int64, device=query.device)
        _lib.call("tk3d_ball_query_bcn", query, ptr(query), ptr(key), i64(b), i64(n1), i64(n2),
                  ctypes.c_float(float(radius)), i64(max_neighbors), ptr(index),
                  stream_of(query))
    return index


def knn_distance_bcn(query, key, k, version):
    """query [B,3,N1], key [B,3,N2] -> [distance [B,N1,k], index [B,N1,k]]; equals
    ``_C.knn_distance_cuda`` on the transposed clouds. Returns None when the library
    declines this k and launch size on this layout (it has a faster kernel that reads
    [B,N,3] only, or none at all for k > 64): the caller then copies to [B,N,3]."""
    b, n1 = _cloud_dims("query", query, True)
    b2, n2 = _cloud_dims("key", key, True)
    _check_eq(b, b2, "key.size(0) == query.size(0)")
    _check_same("query", query, "key", key)
    k = int(k)
    _check(n2 >= k, "Check failed: key.size(1) >= k (%d vs. %d)" % (n2, k))
    _check(int(version) in (0, 1), "Invalid version")
    _check(k >= 0, "k must be non-negative.")
    if k > 64:
        return None
    with _lib.on_device_of(query):
        distance = torch.empty((b, n1, k), dtype=query.dtype, device=query.device)
        index = torch.empty((b, n1, k), dtype=torch.int64, device=query.device)
        if k > 0 and not _lib.call("tk3d_knn_distance_bcn", query, ptr(query), ptr(key), i64(b),
                                   i64(n1), i64(n2), i64(k), ctypes.c_int(int(version)),
                                   ptr(distance), ptr(index), stream_of(query),
                                   may_decline=True):
            return None
    return [distance, index]


def group_points_concat_forward(feature, xyz, centre, index):
    """feature [B,C,N1] or None, xyz [B,3,N1], centre [B,3,N2], index [B,N2,K] ->
    [B,C+3,N2,K]: grouped features, then grouped coordinates minus their centre."""
    b, n1 = _cloud_dims("xyz", xyz, True)
    b2, n2 = _cloud_dims("centre", centre, True)
    _check_eq(b, b2, "xyz.size(0) == centre.size(0)")
    _check_same("xyz", xyz, "centre", centre)
    _check_contiguous_cuda("index", index)
    _check_index("index", index)
    _check_eq(index.dim(), 3, "index.dim() == 3")
    _check_eq(index.size(0), b, "index.size(0) == xyz.size(0)")
    _check_eq(index.size(1), n2, "index.size(1) == centre.size(2)")
    c = 0
    if feature is not None:
        _check_contiguous_cuda("feature", feature)
        _check_eq(feature.dim(), 3, "feature.dim() == 3")
        _check_eq(feature.size(0), b, "feature.size(0) == xyz.size(0)")
        _check_eq(feature.size(2), n1, "feature.size(2) == xyz.size(2)")
        _check_same("feature", feature, "xyz", xyz)
        c = feature.size(1)
    k = index.size(2)
    with _lib.on_device_of(xyz):
        out = torch.empty((b, c + 3, n2, k), dtype=xyz.dtype, device=xyz.device)
        _lib.call("tk3d_group_points_concat_forward", xyz,
                  ptr(feature) if c > 0 else ctypes.c_void_p(0), ptr(xyz), ptr(centre),
                  ptr(index), i64(b), i64(c), i64(n1), i64(n2), i64(k), ptr(out), stream_of(xyz))
    return out


def group_points_concat_backward(grad_output, index, n1, want_feature, want_xyz):
    """grad_output [B,C+3,N2,K], index [B,N2,K] -> (grad_feature [B,C,n1] or None,
    grad_xyz [B,3,n1] or None)."""
    _check_contiguous_cuda("grad_output", grad_output)
    _check_contiguous_cuda("index", index)
    _check_index("index", index)
    _check_eq(grad_output.dim(), 4, "grad_output.dim() == 4")
    _check_eq(index.dim(), 3, "index.dim() == 3")
    _check_eq(index.size(0), grad_output.size(0), "index.size(0) == grad_output.size(0)")
    _check_eq(index.size(1), grad_output.size(2), "index.size(1) == grad_output.size(2)")
    _check_eq(index.size(2), grad_output.size(3), "index.size(2) == grad_output.size(3)")
    b, ct, n2, k = grad_output.shape
    c = ct - 3
    _check(c >= 0, "grad_output must have at least 3 channels.")
    n1 = int(n1)
    with _lib.on_device_of(grad_output):
        gfeat = gxyz = None
        if want_feature and c > 0:
            gfeat = torch.empty((b, c, n1), dtype=grad_output.dtype, device=grad_output.device)
        if want_xyz:
            gxyz = torch.empty((b, 3, n1), dtype=grad_output.dtype, device=grad_output.device)
        if gfeat is not None or gxyz is not None:
            _lib.call("tk3d_group_points_concat_backward", grad_output, ptr(grad_output),
                      ptr(index), i64(b), i64(c), i64(n1), i64(n2), i64(k),
                      ptr(gfeat) if gfeat is not None else ctypes.c_void_p(0),
                      ptr(gxyz) if gxyz is not None else ctypes.c_void_p(0),
                      stream_of(grad_output))
    return gfeat, gxyz


def three_nn(query, key, channels_first, eps=1e-10):
    """3 nearest keys of every query with inverse-squared-distance weights ->
    (distance [B,N1,3], index [B,N1,3] int64, weight [B,N1,3]); distance and index
    equal ``_C.knn_distance_cuda(query, key, 3, 1)`` on [B,N,3] clouds."""
    b, n1 = _cloud_dims("query", query, channels_first)
    b2, n2 = _cloud_dims("key", key, channels_first)
    _check_eq(b, b2, "query.size(0) == key.size(0)")
    _check_same("query", query, "key", key)
    _check(n2 >= 3, "Check failed: key.size(1) >= k (%d vs. 3)" % n2)
    with _lib.on_device_of(query):
        distance = torch.empty((b, n1, 3), dtype=query.dtype, device=query.device)
        index = torch.empty((b, n1, 3), dtype=torch.int64, device=query.device)
        weight = torch.empty((b, n1, 3), dtype=query.dtype, device=query.device)
        _lib.call("tk3d_three_nn", query, ptr(query), ptr(key),
                  ctypes.c_int(1 if channels_first else 0), i64(b), i64(n1), i64(n2),
                  ctypes.c_double(float(eps)), ptr(distance), ptr(index), ptr(weight),
                  stream_of(query))
    return distance, index, weight


def chamfer_forward_bcn(xyz1, xyz2):
    """xyz1 [B,3,N1], xyz2 [B,3,N2] -> [dist1, idx1, dist2, idx2], the clouds read in place
    (the reference copies them to [B,N,3] first, torkit3d/ops/chamfer_distance.py:52-55)."""
    b, n1 = _cloud_dims("xyz1", xyz1, True)
    b2, n2 = _cloud_dims("xyz2", xyz2, True)
    _check_eq(b, b2, "xyz1.size(0) == xyz2.size(0)")
    _check_same("xyz1", xyz1, "xyz2", xyz2)
    dev = xyz1.device
    with _lib.on_device_of(xyz1):
        dist1 = torch.empty((b, n1), dtype=xyz1.dtype, device=dev)
        idx1 = torch.empty((b, n1), dtype=torch.int64, device=dev)
        dist2 = torch.empty((b, n2), dtype=xyz1.dtype, device=dev)
        idx2 = torch.empty((b, n2), dtype=torch.int64, device=dev)
        if xyz1.dtype == torch.float32:
            ws_bytes = _lib.chamfer_workspace_bytes(b, n1, n2) if max(n1, n2) <= 16384 else 0
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes else None
            fn = _lib.lib().tk3d_chamfer_distance_forward_bcn_f32
            fn.restype = ctypes.c_int
            _lib.check(fn(ptr(xyz1), ptr(xyz2), i64(b), i64(n1), i64(n2), ptr(dist1), ptr(idx1),
                          ptr(dist2), ptr(idx2),
                          ctypes.c_void_p(ws.data_ptr() if ws is not None else 0),
                          ctypes.c_size_t(ws_bytes), stream_of(xyz1)),
                       "tk3d_chamfer_distance_forward_bcn_f32")
        else:
            _lib.call("tk3d_chamfer_distance_forward_bcn", xyz1, ptr(xyz1), ptr(xyz2), i64(b),
                      i64(n1), i64(n2), ptr(dist1), ptr(idx1), ptr(dist2), ptr(idx2),
                      stream_of(xyz1))
    return [dist1, idx1, dist2, idx2]
