"""The C-ABI library: every symbol declared in include/tk3d.h is exported, and the
argument checks reject bad calls before anything is launched (so they can be
exercised without a GPU)."""
import ctypes
import os
import re

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "tk3d.h")


@pytest.fixture(scope="module")
def lib():
    from torkit3d_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from torkit3d_amd import build

        build.build()
    return _lib.lib()


DEBUG_HEADER = os.path.join(REPO, "torkit3d_amd", "csrc", "tk3d_debug.h")


def declared_symbols(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tk3d_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_families():
    names = declared_symbols()
    for family in ("chamfer_distance_forward", "chamfer_distance_backward", "knn_distance",
                   "ball_query", "sample_farthest_points", "group_points_forward",
                   "group_points_backward", "interpolate_forward", "interpolate_backward"):
        assert "tk3d_%s_f32" % family in names
        assert "tk3d_%s_f64" % family in names
    assert "tk3d_version" in names and "tk3d_error_string" in names


def test_every_declared_symbol_is_exported(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), "%s declared in tk3d.h but not exported" % name


def test_test_only_entry_points_are_exported_and_outside_the_boundary(lib):
    # what the tests and the benchmark call besides the boundary: declared in a header of its
    # own, none of it in include/tk3d.h
    debug = declared_symbols(DEBUG_HEADER)
    assert debug and all(name.startswith("tk3d_debug_") for name in debug)
    assert not any(name.startswith("tk3d_debug_") for name in declared_symbols())
    for name in debug:
        assert hasattr(lib, name), "%s declared in tk3d_debug.h but not exported" % name
    fn = lib.tk3d_debug_chamfer_forward_route_f32
    fn.restype = ctypes.c_int
    null = ctypes.c_void_p(0)
    # argument checks come before any launch
    assert fn(null, null, i64(-1), i64(4), i64(4), null, null, null, null, ctypes.c_int(1), null) == -2
    assert fn(null, null, i64(1), i64(4), i64(4), null, null, null, null, ctypes.c_int(1), null) == -1


def test_version_and_error_strings(lib):
    from torkit3d_amd import _lib

    assert lib.tk3d_version() == 100
    assert _lib.error_string(0) == "success"
    assert "Invalid version" in _lib.error_string(-4)
    for code in range(-6, 0):
        assert "unknown" not in _lib.error_string(code)
    assert "unknown" in _lib.error_string(-99)


def i64(v):
    return ctypes.c_int64(v)


NULL = ctypes.c_void_p(0)
FAKE = ctypes.c_void_p(256)  # never dereferenced: the checks below fail first


def test_argument_errors_are_reported_without_launching(lib):
    for sfx in ("_f32", "_f64"):
        fwd = getattr(lib, "tk3d_chamfer_distance_forward" + sfx)
        assert fwd(FAKE, FAKE, i64(-1), i64(4), i64(4), FAKE, FAKE, FAKE, FAKE, NULL) == -2
        assert fwd(NULL, FAKE, i64(1), i64(4), i64(4), FAKE, FAKE, FAKE, FAKE, NULL) == -1
        assert fwd(NULL, NULL, i64(0), i64(4), i64(4), NULL, NULL, NULL, NULL, NULL) == 0
        knn = getattr(lib, "tk3d_knn_distance" + sfx)
        assert knn(FAKE, FAKE, i64(1), i64(8), i64(4), i64(5), 1, FAKE, FAKE, NULL) == -3  # k > N2
        assert knn(FAKE, FAKE, i64(1), i64(8), i64(4), i64(0), 1, FAKE, FAKE, NULL) == -3
        assert knn(FAKE, FAKE, i64(1), i64(8), i64(4), i64(2), 7, FAKE, FAKE, NULL) == -4
        fps = getattr(lib, "tk3d_sample_farthest_points" + sfx)
        assert fps(FAKE, i64(1), i64(10), i64(0), FAKE, NULL, ctypes.c_size_t(0), NULL) == -3
        assert fps(FAKE, i64(1), i64(10), i64(11), FAKE, NULL, ctypes.c_size_t(0), NULL) == -3
        assert fps(NULL, i64(1), i64(10), i64(5), FAKE, NULL, ctypes.c_size_t(0), NULL) == -1
        # a cloud too large for the register kernel needs a workspace
        assert fps(FAKE, i64(1), i64(100000), i64(5), FAKE, NULL, ctypes.c_size_t(0), NULL) == -5
        ball = getattr(lib, "tk3d_ball_query" + sfx)
        assert ball(FAKE, FAKE, i64(1), i64(4), i64(4), ctypes.c_float(0.1), i64(-1), FAKE, NULL) == -3
        interp = getattr(lib, "tk3d_interpolate_forward" + sfx)
        assert interp(FAKE, FAKE, FAKE, i64(1), i64(2), i64(4), i64(4), i64(9), FAKE, NULL) == -3
        group = getattr(lib, "tk3d_group_points_backward" + sfx)
        assert group(FAKE, FAKE, i64(1), i64(-2), i64(4), i64(4), i64(2), FAKE, NULL) == -2
        # entry points that fuse Python-side steps of the reference
        ball = getattr(lib, "tk3d_ball_query_bcn" + sfx)
        assert ball(FAKE, FAKE, i64(1), i64(4), i64(4), ctypes.c_float(0.1), i64(-1), FAKE, NULL) == -3
        assert ball(NULL, FAKE, i64(1), i64(4), i64(4), ctypes.c_float(0.1), i64(2), FAKE, NULL) == -1
        fps = getattr(lib, "tk3d_sample_farthest_points_gather" + sfx)
        assert fps(FAKE, 1, i64(1), i64(10), i64(11), FAKE, NULL, NULL, ctypes.c_size_t(0), NULL) == -3
        assert fps(NULL, 0, i64(1), i64(10), i64(5), FAKE, NULL, NULL, ctypes.c_size_t(0), NULL) == -1
        nn3 = getattr(lib, "tk3d_three_nn" + sfx)
        eps = ctypes.c_double(1e-10)
        assert nn3(FAKE, FAKE, 0, i64(1), i64(8), i64(2), eps, FAKE, FAKE, FAKE, NULL) == -3
        assert nn3(FAKE, FAKE, 1, i64(1), i64(8), i64(4), eps, FAKE, FAKE, NULL, NULL) == -1
        assert nn3(NULL, NULL, 1, i64(0), i64(8), i64(4), eps, NULL, NULL, NULL, NULL) == 0
        cat = getattr(lib, "tk3d_group_points_concat_forward" + sfx)
        assert cat(NULL, FAKE, FAKE, FAKE, i64(1), i64(2), i64(4), i64(4), i64(2), FAKE, NULL) == -1
        assert cat(NULL, FAKE, FAKE, FAKE, i64(1), i64(0), i64(4), i64(-4), i64(2), FAKE, NULL) == -2
        cat = getattr(lib, "tk3d_group_points_concat_backward" + sfx)
        assert cat(FAKE, FAKE, i64(1), i64(2), i64(4), i64(4), i64(2), NULL, NULL, NULL) == 0


def test_fps_workspace_size(lib):
    fn = lib.tk3d_sample_farthest_points_workspace_bytes
    fn.restype = ctypes.c_size_t
    assert fn(i64(16), i64(4096), ctypes.c_size_t(4)) == 0
    assert fn(i64(8), i64(16384), ctypes.c_size_t(4)) == 0
    need = fn(i64(2), i64(100000), ctypes.c_size_t(4))
    assert need >= 2 * 100000 * 4


def test_chamfer_workspace_size_and_argument_checks(lib):
    # the size function is host code: the dispatch rule of the sorted path, no GPU needed
    size = lib.tk3d_chamfer_distance_forward_workspace_bytes
    size.restype = ctypes.c_size_t

    def nbytes(b, n1, n2, always):
        return size(i64(b), i64(n1), i64(n2), ctypes.c_int(always))

    assert nbytes(32, 16384, 16384, 0) > 0          # the benchmark shape is served
    assert nbytes(1, 65536, 65536, 0) > 0
    assert nbytes(2, 1024, 1024, 0) == 0            # too little work to repay the sort
    assert nbytes(16, 4096, 4096, 0) == 0
    assert nbytes(4, 65536, 2048, 0) == 0           # lengths more than a factor of four apart
    assert nbytes(64, 3000, 3000, 0) == 0           # clouds under 4096 points
    for shape in ((2, 1024, 1024), (16, 4096, 4096), (4, 65536, 2048), (1, 1, 1)):
        assert nbytes(*shape, 1) > 0                # ... but can be, on request
    assert nbytes(1, 65537, 4096, 1) == 0 and nbytes(0, 4096, 4096, 1) == 0
    # 16 + 32 bytes per padded point, a box per 32 points, headers, flags and far-key lists
    b, n = 3, 5000
    pad = (n + 127) // 128 * 128
    low = 2 * b * pad * 48
    assert low < nbytes(b, n, n, 1) < low + 2 * b * (pad // 2 + 1024) + 4096
    # null or short workspace: the call is the plain entry point, with its argument checks
    fn = lib.tk3d_chamfer_distance_forward_ws_f32
    args = (FAKE, FAKE, i64(1), i64(8), i64(8), FAKE, FAKE, FAKE)
    assert fn(*args, NULL, NULL, ctypes.c_size_t(0), NULL) == -1          # idx2 missing
    assert fn(FAKE, FAKE, i64(-1), i64(8), i64(8), FAKE, FAKE, FAKE, FAKE, NULL,
              ctypes.c_size_t(0), NULL) == -2
    assert fn(NULL, NULL, i64(0), i64(8), i64(8), NULL, NULL, NULL, NULL, NULL,
              ctypes.c_size_t(0), NULL) == 0
