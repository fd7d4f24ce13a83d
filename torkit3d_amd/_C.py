"""Drop-in for the reference's compiled extension ``torkit3d._C``.

The reference registers nine functions in a pybind11 module
(torkit3d/csrc/torkit3d.cpp:13-21). This module exposes the same nine names with
the same positional arguments and return values; each validates its tensors the way
the reference's host code does (TORCH_CHECK -> RuntimeError), allocates the outputs
with torch and hands raw device pointers to the C ABI in ``include/tk3d.h``.
Kernels are enqueued on torch's current stream for the tensors' device.

Placing this file (plus ``_lib.py`` and ``libtk3d.so``) inside a checkout of the
reference as ``torkit3d/_C.py`` makes the reference's own ``torkit3d.ops`` run on
MI355X unchanged.
"""
import ctypes

import torch

from . import _lib
from ._lib import i64, ptr, stream_of

__all__ = [
    "sample_farthest_points_cuda",
    "ball_query_cuda",
    "group_points_forward_cuda",
    "group_points_backward_cuda",
    "interpolate_forward_cuda",
    "interpolate_backward_cuda",
    "knn_distance_cuda",
    "chamfer_distance_forward_cuda",
    "chamfer_distance_backward_cuda",
]


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_cuda(name, t):
    _check(isinstance(t, torch.Tensor), "%s must be a tensor." % name)
    _check(t.is_cuda, "%s must be a CUDA tensor." % name)


def _check_contiguous_cuda(name, t):
    _check_cuda(name, t)
    _check(t.is_contiguous(), "%s must be contiguous." % name)


def _check_eq(a, b, what):
    _check(a == b, "Check failed: %s (%s vs. %s)" % (what, a, b))


def _check_index(name, t):
    _check(t.dtype == torch.int64, "%s must be an int64 tensor." % name)


def _check_same(a_name, a, b_name, b):
    _check(a.dtype == b.dtype, "%s and %s must have the same dtype." % (a_name, b_name))
    _check(a.device == b.device, "%s and %s must be on the same device." % (a_name, b_name))


def sample_farthest_points_cuda(points, num_samples):
    """points [B,N,3] -> index [B,num_samples] int64
    (sample_farthest_points_kernel.cu:106-165)."""
    _check_contiguous_cuda("points", points)
    _check_eq(points.dim(), 3, "points.dim() == 3")
    _check_eq(points.size(2), 3, "points.size(2) == 3")
    num_samples = int(num_samples)
    _check(num_samples > 0, "Check failed: num_samples > 0 (%d vs. 0)" % num_samples)
    _check(points.size(1) >= num_samples,
           "Check failed: points.size(1) >= num_samples (%d vs. %d)" % (points.size(1), num_samples))
    b, n = points.size(0), points.size(1)
    with _lib.on_device_of(points):
        index = torch.empty((b, num_samples), dtype=torch.int64, device=points.device)
        ws_bytes = _lib.fps_workspace_bytes(b, n, points.element_size())
        ws = None
        if ws_bytes:
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=points.device)
        _lib.call("tk3d_sample_farthest_points", points, ptr(points), i64(b), i64(n),
                  i64(num_samples), ptr(index),
                  ctypes.c_void_p(ws.data_ptr() if ws is not None else 0),
                  ctypes.c_size_t(ws_bytes), stream_of(points))
    return index


def ball_query_cuda(query, key, radius, max_neighbors):
    """query [B,N1,3], key [B,N2,3] -> index [B,N1,max_neighbors] int64
    (ball_query_kernel.cu:105-173)."""
    _check_contiguous_cuda("query", query)
    _check_contiguous_cuda("key", key)
    _check(query.dim() == 3 and key.dim() == 3, "query and key must be 3-D tensors.")
    _check_eq(query.size(0), key.size(0), "query.size(0) == key.size(0)")
    _check_eq(query.size(2), 3, "query.size(2) == 3")
    _check_eq(key.size(2), 3, "key.size(2) == 3")
    _check_same("query", query, "key", key)
    max_neighbors = int(max_neighbors)
    _check(max_neighbors >= 0, "max_neighbors must be non-negative.")
    b, n1, n2 = query.size(0), query.size(1), key.size(1)
    with _lib.on_device_of(query):
        index = torch.empty((b, n1, max_neighbors), dtype=torch.int64, device=query.device)
        _lib.call("tk3d_ball_query", query, ptr(query), ptr(key), i64(b), i64(n1), i64(n2),
                  ctypes.c_float(float(radius)), i64(max_neighbors), ptr(index),
                  stream_of(query))
    return index


def group_points_forward_cuda(input, index):
    """input [B,C,N1], index [B,N2,K] -> [B,C,N2,K] (group_points_kernel.cu:8-31).
    Like the reference (which goes through at::gather) this accepts
    non-contiguous tensors; they are made contiguous first."""
    _check_cuda("input", input)
    _check_cuda("index", index)
    _check_eq(input.dim(), 3, "input.dim() == 3")
    _check_eq(index.dim(), 3, "index.dim() == 3")
    _check_eq(input.size(0), index.size(0), "input.size(0) == index.size(0)")
    _check_index("index", index)
    input = input.contiguous()
    index = index.contiguous()
    b, c, n1 = input.shape
    n2, k = index.size(1), index.size(2)
    with _lib.on_device_of(input):
        output = torch.empty((b, c, n2, k), dtype=input.dtype, device=input.device)
        _lib.call("tk3d_group_points_forward", input, ptr(input), ptr(index), i64(b), i64(c),
                  i64(n1), i64(n2), i64(k), ptr(output), stream_of(input))
    return output


def group_points_backward_cuda(grad_output, index, n1):
    """grad_output [B,C,N2,K], index [B,N2,K], n1 -> grad_input [B,C,n1]
    (group_points_kernel.cu:67-114)."""
    _check_contiguous_cuda("grad_output", grad_output)
    _check_contiguous_cuda("index", index)
    _check_eq(grad_output.dim(), 4, "grad_output.dim() == 4")
    _check_eq(index.dim(), 3, "index.dim() == 3")
    _check_eq(index.size(0), grad_output.size(0), "index.size(0) == grad_output.size(0)")
    _check_eq(index.size(1), grad_output.size(2), "index.size(1) == grad_output.size(2)")
    _check_eq(index.size(2), grad_output.size(3), "index.size(2) == grad_output.size(3)")
    _check_index("index", index)
    n1 = int(n1)
    b, c, n2, k = grad_output.shape
    with _lib.on_device_of(grad_output):
        grad_input = torch.empty((b, c, n1), dtype=grad_output.dtype, device=grad_output.device)
        _lib.call("tk3d_group_points_backward", grad_output, ptr(grad_output), ptr(index),
                  i64(b), i64(c), i64(n1), i64(n2), i64(k), ptr(grad_input),
                  stream_of(grad_output))
    return grad_input


def _check_interpolate(first_name, first, index, weight):
    _check_contiguous_cuda(first_name, first)
    _check_contiguous_cuda("index", index)
    _check_contiguous_cuda("weight", weight)
    _check_eq(first.dim(), 3, "%s.dim() == 3" % first_name)
    _check_eq(index.dim(), 3, "index.dim() == 3")
    _check_eq(weight.dim(), 3, "weight.dim() == 3")
    _check_eq(first.size(0), index.size(0), "%s.size(0) == index.size(0)" % first_name)
    _check_eq(first.size(0), weight.size(0), "%s.size(0) == weight.size(0)" % first_name)
    _check_eq(index.size(1), weight.size(1), "index.size(1) == weight.size(1)")
    _check_eq(index.size(2), weight.size(2), "index.size(2) == weight.size(2)")
    _check_index("index", index)
    _check_same(first_name, first, "weight", weight)


def interpolate_forward_cuda(input, index, weight):
    """input [B,C,N1], index [B,N2,3], weight [B,N2,3] -> [B,C,N2]
    (interpolate_kernel.cu:49-103)."""
    _check_interpolate("input", input, index, weight)
    _check_eq(index.size(2), 3, "index.size(2) == 3")
    b, c, n1 = input.shape
    n2, k = index.size(1), index.size(2)
    with _lib.on_device_of(input):
        output = torch.empty((b, c, n2), dtype=input.dtype, device=input.device)
        _lib.call("tk3d_interpolate_forward", input, ptr(input), ptr(index), ptr(weight),
                  i64(b), i64(c), i64(n1), i64(n2), i64(k), ptr(output), stream_of(input))
    return output


def interpolate_backward_cuda(grad_output, index, weight, n1):
    """grad_output [B,C,N2], index, weight [B,N2,3], n1 -> grad_input [B,C,n1]
    (interpolate_kernel.cu:147-201)."""
    _check_interpolate("grad_output", grad_output, index, weight)
    _check_eq(grad_output.size(2), index.size(1), "grad_output.size(2) == index.size(1)")
    _check(index.size(2) == 3, "Only support k=3.")
    n1 = int(n1)
    b, c, n2 = grad_output.shape
    k = index.size(2)
    with _lib.on_device_of(grad_output):
        grad_input = torch.empty((b, c, n1), dtype=grad_output.dtype, device=grad_output.device)
        _lib.call("tk3d_interpolate_backward", grad_output, ptr(grad_output), ptr(index),
                  ptr(weight), i64(b), i64(c), i64(n1), i64(n2), i64(k), ptr(grad_input),
                  stream_of(grad_output))
    return grad_input


def knn_distance_cuda(query, key, k, version):
    """query [B,N1,3], key [B,N2,3] -> [distance [B,N1,k], index [B,N1,k] int64],
    squared distances in MinK slot order (knn_distance_kernel.cu:187-298)."""
    _check_contiguous_cuda("query", query)
    _check_contiguous_cuda("key", key)
    _check_eq(query.dim(), 3, "query.dim() == 3")
    _check_eq(query.size(2), 3, "query.size(2) == 3")
    _check_eq(key.dim(), 3, "key.dim() == 3")
    _check_eq(key.size(0), query.size(0), "key.size(0) == query.size(0)")
    k = int(k)
    _check(key.size(1) >= k, "Check failed: key.size(1) >= k (%d vs. %d)" % (key.size(1), k))
    _check_eq(key.size(2), 3, "key.size(2) == 3")
    _check_same("query", query, "key", key)
    _check(int(version) in (0, 1), "Invalid version")
    _check(k >= 0, "k must be non-negative.")
    b, n1, n2 = query.size(0), query.size(1), key.size(1)
    with _lib.on_device_of(query):
        distance = torch.empty((b, n1, k), dtype=query.dtype, device=query.device)
        index = torch.empty((b, n1, k), dtype=torch.int64, device=query.device)
        if k > 0:
            _lib.call("tk3d_knn_distance", query, ptr(query), ptr(key), i64(b), i64(n1),
                      i64(n2), i64(k), ctypes.c_int(int(version)), ptr(distance), ptr(index),
                      stream_of(query))
    return [distance, index]


def chamfer_distance_forward_cuda(xyz1, xyz2):
    """xyz1 [B,N1,3], xyz2 [B,N2,3] -> [dist1, idx1, dist2, idx2]
    (chamfer_distance_kernel.cu:91-151)."""
    _check_contiguous_cuda("xyz1", xyz1)
    _check_contiguous_cuda("xyz2", xyz2)
    _check(xyz1.dim() == 3 and xyz2.dim() == 3, "xyz1 and xyz2 must be 3-D tensors.")
    _check_eq(xyz1.size(0), xyz2.size(0), "xyz1.size(0) == xyz2.size(0)")
    _check_eq(xyz1.size(2), 3, "xyz1.size(2) == 3")
    _check_eq(xyz2.size(2), 3, "xyz2.size(2) == 3")
    _check_same("xyz1", xyz1, "xyz2", xyz2)
    b, n1, n2 = xyz1.size(0), xyz1.size(1), xyz2.size(1)
    dev = xyz1.device
    with torch.cuda.device(dev):
        dist1 = torch.empty((b, n1), dtype=xyz1.dtype, device=dev)
        idx1 = torch.empty((b, n1), dtype=torch.int64, device=dev)
        dist2 = torch.empty((b, n2), dtype=xyz1.dtype, device=dev)
        idx2 = torch.empty((b, n2), dtype=torch.int64, device=dev)
        ws_bytes = _lib.chamfer_workspace_bytes(b, n1, n2) if xyz1.dtype == torch.float32 else 0
        if ws_bytes:
            # clouds of a few thousand points and more: sorted along a space-filling curve
            # in a scratch buffer, and only key tiles near a wave's queries are swept
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
            fn = _lib.lib().tk3d_chamfer_distance_forward_ws_f32
            fn.restype = ctypes.c_int
            _lib.check(fn(ptr(xyz1), ptr(xyz2), i64(b), i64(n1), i64(n2), ptr(dist1), ptr(idx1),
                          ptr(dist2), ptr(idx2), ctypes.c_void_p(ws.data_ptr()),
                          ctypes.c_size_t(ws_bytes), stream_of(xyz1)),
                       "tk3d_chamfer_distance_forward_ws_f32")
        else:
            _lib.call("tk3d_chamfer_distance_forward", xyz1, ptr(xyz1), ptr(xyz2), i64(b),
                      i64(n1), i64(n2), ptr(dist1), ptr(idx1), ptr(dist2), ptr(idx2),
                      stream_of(xyz1))
    return [dist1, idx1, dist2, idx2]


def chamfer_distance_backward_cuda(grad_dist1, grad_dist2, xyz1, xyz2, idx1, idx2):
    """-> [grad_xyz1 [B,N1,3], grad_xyz2 [B,N2,3]] (chamfer_distance_kernel.cu:200-274)."""
    for name, t in (("grad_dist1", grad_dist1), ("grad_dist2", grad_dist2), ("xyz1", xyz1),
                    ("xyz2", xyz2), ("idx1", idx1), ("idx2", idx2)):
        _check_contiguous_cuda(name, t)
    _check(grad_dist1.dim() == 2 and grad_dist2.dim() == 2, "grad_dist must be 2-D tensors.")
    b, n1, n2 = grad_dist1.size(0), grad_dist1.size(1), grad_dist2.size(1)
    _check_eq(grad_dist2.size(0), b, "grad_dist2.size(0) == bs")
    _check(xyz1.dim() == 3 and xyz2.dim() == 3, "xyz1 and xyz2 must be 3-D tensors.")
    _check_eq(xyz1.size(0), b, "xyz1.size(0) == bs")
    _check_eq(xyz2.size(0), b, "xyz2.size(0) == bs")
    _check_eq(xyz1.size(1), n1, "xyz1.size(1) == n1")
    _check_eq(xyz2.size(1), n2, "xyz2.size(1) == n2")
    _check_eq(xyz1.size(2), 3, "xyz1.size(2) == 3")
    _check_eq(xyz2.size(2), 3, "xyz2.size(2) == 3")
    _check_eq(idx1.size(0), b, "idx1.size(0) == bs")
    _check_eq(idx2.size(0), b, "idx2.size(0) == bs")
    _check_eq(idx1.size(1), n1, "idx1.size(1) == n1")
    _check_eq(idx2.size(1), n2, "idx2.size(1) == n2")
    _check_index("idx1", idx1)
    _check_index("idx2", idx2)
    _check_same("grad_dist1", grad_dist1, "xyz1", xyz1)
    _check_same("grad_dist2", grad_dist2, "xyz2", xyz2)
    _check_same("xyz1", xyz1, "xyz2", xyz2)
    dev = xyz1.device
    with torch.cuda.device(dev):
        grad_xyz1 = torch.empty((b, n1, 3), dtype=xyz1.dtype, device=dev)
        grad_xyz2 = torch.empty((b, n2, 3), dtype=xyz1.dtype, device=dev)
        _lib.call("tk3d_chamfer_distance_backward", xyz1, ptr(grad_dist1), ptr(grad_dist2),
                  ptr(xyz1), ptr(xyz2), ptr(idx1), ptr(idx2), i64(b), i64(n1), i64(n2),
                  ptr(grad_xyz1), ptr(grad_xyz2), stream_of(xyz1))
    return [grad_xyz1, grad_xyz2]
