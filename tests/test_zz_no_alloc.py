"""tk3d_sample_farthest_points_static_f32: farthest point sampling whose large-cloud
workspace is a fixed array inside the library (for callers that cannot allocate device
memory). Its index output must equal tk3d_sample_farthest_points_f32's bit for bit, call
after call, whatever an earlier call left in the shared array."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_BYTES = 8 << 20


def _entry_points():
    from torkit3d_amd import _lib

    lib = _lib.lib()
    static = lib.tk3d_sample_farthest_points_static_f32
    static.restype = ctypes.c_int
    plain = lib.tk3d_sample_farthest_points_f32
    plain.restype = ctypes.c_int
    return _lib, static, plain


def _both(points, k):
    """Index tensors of the static-workspace entry point and of the existing one."""
    _lib, static, plain = _entry_points()
    b, n, _ = points.shape
    stream = _lib.stream_of(points)
    got = torch.full((b, k), -7, dtype=torch.int64, device=points.device)
    rc = static(_lib.ptr(points), _lib.i64(b), _lib.i64(n), _lib.i64(k), _lib.ptr(got), stream)
    assert rc == 0, _lib.error_string(rc)
    need = _lib.fps_workspace_bytes(b, n, 4)
    work = torch.empty(max(need, 8), dtype=torch.uint8, device=points.device)
    want = torch.full((b, k), -9, dtype=torch.int64, device=points.device)
    rc = plain(_lib.ptr(points), _lib.i64(b), _lib.i64(n), _lib.i64(k), _lib.ptr(want),
               _lib.ptr(work), ctypes.c_size_t(need), stream)
    assert rc == 0, _lib.error_string(rc)
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy(), need


def test_static_workspace_matches_the_allocating_entry_point_twice_in_a_row(cuda):
    import oracle

    g = torch.Generator().manual_seed(41)
    # first call: two clouds above the register kernel's 16384 points (workspace in use)
    big = torch.rand(2, 40000, 3, generator=g)
    got, want, need = _both(big.to(cuda), 48)
    assert 0 < need <= STATIC_BYTES
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, oracle.sample_farthest_points(big.numpy(), 48))
    # second call, smaller: another layout inside the same array, which still holds the
    # first call's minima and candidates
    small = torch.rand(1, 17000, 3, generator=g)
    got, want, need = _both(small.to(cuda), 33)
    assert 0 < need <= STATIC_BYTES
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, oracle.sample_farthest_points(small.numpy(), 33))
    # a cloud the register kernel takes needs no workspace at all
    tiny = torch.rand(3, 1000, 3, generator=g)
    got, want, need = _both(tiny.to(cuda), 100)
    assert need == 0
    np.testing.assert_array_equal(got, want)


def test_static_workspace_rejects_clouds_beyond_its_size(cuda):
    _lib, static, _ = _entry_points()
    n = 3 << 20  # 12 MiB of running minima alone
    assert _lib.fps_workspace_bytes(1, n, 4) > STATIC_BYTES
    points = torch.zeros(1, n, 3, device=cuda)
    index = torch.full((1, 4), -7, dtype=torch.int64, device=cuda)
    rc = static(_lib.ptr(points), _lib.i64(1), _lib.i64(n), _lib.i64(4), _lib.ptr(index),
                _lib.stream_of(points))
    assert rc == -5 and "workspace" in _lib.error_string(rc)
    torch.cuda.synchronize()
    assert (index == -7).all()  # nothing was launched
