"""CPU oracle for the torkit3d point-cloud ops (numpy in, numpy out).

TEST INFRASTRUCTURE ONLY: a checker for the HIP library and the benchmark's CPU
figure. Product code (``torkit3d_amd``) must never import this package.

Every function mirrors one ``torkit3d._C`` entry point of the reference and runs
the C restatement in ``tk3d_oracle_impl.inc`` (fp32 or fp64, chosen from the dtype
of the first array). ``build()`` compiles the shared library with gcc.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtk3d_oracle.so")
_lib = None


def build(force=False):
    """Compile ``libtk3d_oracle.so`` next to this file (gcc via the Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.tk3d_oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return int(_load().tk3d_oracle_num_threads())


def set_num_threads(n):
    _load().tk3d_oracle_set_num_threads(ctypes.c_int(int(n)))


def _sfx(a):
    if a.dtype == np.float32:
        return "_f32"
    if a.dtype == np.float64:
        return "_f64"
    raise TypeError("oracle supports float32/float64, got %s" % a.dtype)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a if dtype is None else np.asarray(a, dtype=dtype))
    return a


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _i(v):
    return ctypes.c_int64(int(v))


def _call(name, *args, restype=None):
    fn = getattr(_load(), name)
    fn.restype = restype
    return fn(*args)


def chamfer_forward(xyz1, xyz2, fused=True):
    """-> dist1 [B,N1], idx1 [B,N1] int64, dist2 [B,N2], idx2 [B,N2] int64."""
    xyz1, xyz2 = _c(xyz1), _c(xyz2, xyz1.dtype)
    b, n1, _ = xyz1.shape
    n2 = xyz2.shape[1]
    d1 = np.empty((b, n1), xyz1.dtype)
    i1 = np.empty((b, n1), np.int64)
    d2 = np.empty((b, n2), xyz1.dtype)
    i2 = np.empty((b, n2), np.int64)
    name = "tk3d_oracle_chamfer_forward" + ("" if fused else "_unfused")
    _call(name + _sfx(xyz1), _p(xyz1), _p(xyz2), _i(b), _i(n1), _i(n2),
          _p(d1), _p(i1), _p(d2), _p(i2))
    return d1, i1, d2, i2


def chamfer_backward(grad_dist1, grad_dist2, xyz1, xyz2, idx1, idx2, wide=False):
    """-> grad_xyz1 [B,N1,3], grad_xyz2 [B,N2,3]. ``wide``: every term as the reference
    forms it, summed in double and rounded once (the yardstick for fp32 kernels, whose
    summation order differs from the sequential one of ``wide=False``)."""
    xyz1 = _c(xyz1)
    dt = xyz1.dtype
    xyz2, g1, g2 = _c(xyz2, dt), _c(grad_dist1, dt), _c(grad_dist2, dt)
    idx1, idx2 = _c(idx1, np.int64), _c(idx2, np.int64)
    b, n1, _ = xyz1.shape
    n2 = xyz2.shape[1]
    gx1 = np.empty((b, n1, 3), dt)
    gx2 = np.empty((b, n2, 3), dt)
    _call("tk3d_oracle_chamfer_backward" + ("_wide" if wide else "") + _sfx(xyz1), _p(g1), _p(g2), _p(xyz1),
          _p(xyz2), _p(idx1), _p(idx2), _i(b), _i(n1), _i(n2), _p(gx1), _p(gx2))
    return gx1, gx2


def knn(query, key, k):
    """-> distance [B,N1,k] (squared, MinK slot order), index [B,N1,k] int64."""
    query = _c(query)
    key = _c(key, query.dtype)
    b, n1, _ = query.shape
    n2 = key.shape[1]
    assert 0 < k <= n2
    dist = np.empty((b, n1, k), query.dtype)
    idx = np.empty((b, n1, k), np.int64)
    _call("tk3d_oracle_knn" + _sfx(query), _p(query), _p(key), _i(b), _i(n1),
          _i(n2), _i(k), _p(dist), _p(idx))
    return dist, idx


def ball_query(query, key, radius, max_neighbors):
    """-> index [B,N1,k] int64 (first k hits in key order, padded with the first)."""
    query = _c(query)
    key = _c(key, query.dtype)
    b, n1, _ = query.shape
    n2 = key.shape[1]
    idx = np.empty((b, n1, max_neighbors), np.int64)
    _call("tk3d_oracle_ball_query" + _sfx(query), _p(query), _p(key), _i(b),
          _i(n1), _i(n2), ctypes.c_float(radius), _i(max_neighbors), _p(idx))
    return idx


def sample_farthest_points(points, num_samples, tie_rule="reference"):
    """-> index [B,K] int64. ``tie_rule``: "reference" replays the reference
    kernel's threads and tree; "lowest" is the numpy-argmax recurrence."""
    points = _c(points)
    b, n, _ = points.shape
    assert 0 < num_samples <= n
    idx = np.empty((b, num_samples), np.int64)
    name = {"reference": "tk3d_oracle_fps", "lowest": "tk3d_oracle_fps_lowest_index"}[tie_rule]
    _call(name + _sfx(points), _p(points), _i(b), _i(n), _i(num_samples), _p(idx))
    return idx


def group_forward(inp, index):
    """-> output [B,C,N2,K]."""
    inp, index = _c(inp), _c(index, np.int64)
    b, c, n1 = inp.shape
    _, n2, k = index.shape
    out = np.empty((b, c, n2, k), inp.dtype)
    _call("tk3d_oracle_group_forward" + _sfx(inp), _p(inp), _p(index), _i(b), _i(c),
          _i(n1), _i(n2), _i(k), _p(out), restype=ctypes.c_int64)
    return out


def group_backward(grad_output, index, n1, wide=False):
    """-> grad_input [B,C,n1]. ``wide``: sums in double, rounded once."""
    grad_output, index = _c(grad_output), _c(index, np.int64)
    b, c, n2, k = grad_output.shape
    gin = np.empty((b, c, n1), grad_output.dtype)
    _call("tk3d_oracle_group_backward" + ("_wide" if wide else "") + _sfx(grad_output),
          _p(grad_output),
          _p(index), _i(b), _i(c), _i(n1), _i(n2), _i(k), _p(gin),
          restype=ctypes.c_int64)
    return gin


def interpolate_forward(inp, index, weight):
    """-> output [B,C,N2]."""
    inp, index = _c(inp), _c(index, np.int64)
    weight = _c(weight, inp.dtype)
    b, c, n1 = inp.shape
    _, n2, k = index.shape
    out = np.empty((b, c, n2), inp.dtype)
    _call("tk3d_oracle_interpolate_forward" + _sfx(inp), _p(inp), _p(index),
          _p(weight), _i(b), _i(c), _i(n1), _i(n2), _i(k), _p(out),
          restype=ctypes.c_int64)
    return out


def interpolate_backward(grad_output, index, weight, n1, wide=False):
    """-> grad_input [B,C,n1]. ``wide``: terms in the data type, sums in double, rounded
    once."""
    grad_output, index = _c(grad_output), _c(index, np.int64)
    weight = _c(weight, grad_output.dtype)
    b, c, n2 = grad_output.shape
    k = index.shape[2]
    gin = np.empty((b, c, n1), grad_output.dtype)
    _call("tk3d_oracle_interpolate_backward" + ("_wide" if wide else "") + _sfx(grad_output),
          _p(grad_output),
          _p(index), _p(weight), _i(b), _i(c), _i(n1), _i(n2), _i(k), _p(gin),
          restype=ctypes.c_int64)
    return gin


def three_nn_weights(dist2, eps=1e-10):
    """Inverse-squared-distance weights of the reference's FeatureInterpolator
    (torkit3d/layers/pointnet2.py:128-130), in the dtype of ``dist2``."""
    dist2 = np.asarray(dist2)
    one = dist2.dtype.type(1.0)
    inv = one / np.maximum(dist2, dist2.dtype.type(eps))
    return inv / inv.sum(axis=2, keepdims=True)
