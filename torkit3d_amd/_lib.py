"""ctypes loader for ``libtk3d.so`` (the hand-written HIP kernels behind a C ABI).

There is no CPU fallback: if the library is missing or a call fails, an exception
is raised.
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library resolves against)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtk3d.so")
_lib = None


def lib():
    """The loaded ``libtk3d.so``; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "torkit3d_amd: %s is missing; build it with `python -m torkit3d_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        handle.tk3d_error_string.restype = ctypes.c_char_p
        handle.tk3d_error_string.argtypes = [ctypes.c_int]
        handle.tk3d_version.restype = ctypes.c_int
        _lib = handle
    return _lib


def error_string(code):
    return lib().tk3d_error_string(int(code)).decode()


def check(code, what):
    """Raise RuntimeError (as TORCH_CHECK does in the reference) on a non-zero code."""
    if code != 0:
        raise RuntimeError("%s failed: %s (code %d)" % (what, error_string(code), code))


def ptr(t):
    """Device pointer of a tensor as a ctypes void pointer (NULL for empty tensors)."""
    return ctypes.c_void_p(t.data_ptr() if t.numel() > 0 else 0)


def i64(v):
    return ctypes.c_int64(int(v))


def stream_of(t):
    """The torch current stream on the tensor's device, as a void pointer."""
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def suffix(t):
    if t.dtype == torch.float32:
        return "_f32"
    if t.dtype == torch.float64:
        return "_f64"
    raise RuntimeError("torkit3d_amd supports float32 and float64 tensors, got %s" % t.dtype)


_functions = {}
_fps_workspace_fn = None


def fps_workspace_bytes(b, n, element_size):
    """Scratch bytes ``tk3d_sample_farthest_points*`` needs for B clouds of N points."""
    global _fps_workspace_fn
    if _fps_workspace_fn is None:
        fn = lib().tk3d_sample_farthest_points_workspace_bytes
        fn.restype = ctypes.c_size_t
        _fps_workspace_fn = fn
    return int(_fps_workspace_fn(i64(b), i64(n), ctypes.c_size_t(element_size)))


_chamfer_workspace_fn = None


def chamfer_workspace_bytes(b, n1, n2, always=False):
    """Scratch bytes ``tk3d_chamfer_distance_forward_ws_f32`` wants for this shape: 0 where
    the sorted path cannot serve it or, unless ``always``, is not the faster route."""
    global _chamfer_workspace_fn
    if _chamfer_workspace_fn is None:
        fn = lib().tk3d_chamfer_distance_forward_workspace_bytes
        fn.restype = ctypes.c_size_t
        _chamfer_workspace_fn = fn
    return int(_chamfer_workspace_fn(i64(b), i64(n1), i64(n2), ctypes.c_int(1 if always else 0)))


ERR_UNSUPPORTED = -6  # TK3D_ERR_UNSUPPORTED


def call(name, tensor_for_dtype, *args, may_decline=False):
    """Call ``name`` + the dtype suffix and raise on an error code. With ``may_decline`` a
    TK3D_ERR_UNSUPPORTED return (nothing was launched) is handed back as False instead."""
    key = (name, tensor_for_dtype.dtype)
    fn = _functions.get(key)
    if fn is None:
        fn = getattr(lib(), name + suffix(tensor_for_dtype))
        fn.restype = ctypes.c_int
        _functions[key] = fn
    code = fn(*args)
    if may_decline and code == ERR_UNSUPPORTED:
        return False
    check(code, name)
    return True


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device_of(t):
    """Context in which the tensor's GPU is current (kernels, allocations and streams
    follow the current device). Switching costs a few microseconds per call, so nothing
    is done when that GPU is current already."""
    if t.device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(t.device)
