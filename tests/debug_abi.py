"""ctypes callers for the library's test-only entry points (``csrc/tk3d_debug.h``): one
named chamfer kernel, the sorted chamfer path with its work counted, the KNN pre-filter
kernel, and the matrix instruction on given terms."""
import ctypes

import torch

ROUTE_EXACT, ROUTE_VECTOR, ROUTE_MATRIX4, ROUTE_MATRIX2, ROUTE_MATRIX_SLICED = 1, 2, 3, 4, 5
UNSUPPORTED = -6


def _fn(name):
    from torkit3d_amd import _lib

    fn = getattr(_lib.lib(), name)
    fn.restype = ctypes.c_int
    return fn


def _chamfer_outputs(x1, x2):
    b, n1, n2 = x1.size(0), x1.size(1), x2.size(1)
    dev = x1.device
    return [torch.empty((b, n1), device=dev), torch.empty((b, n1), dtype=torch.int64, device=dev),
            torch.empty((b, n2), device=dev), torch.empty((b, n2), dtype=torch.int64, device=dev)]


def chamfer_route(x1, x2, route):
    """[dist1, idx1, dist2, idx2] of chamfer forward through one named kernel, or None when
    that kernel does not take the shape. x1, x2: contiguous fp32 device tensors [B,N,3]."""
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    out = _chamfer_outputs(x1, x2)
    with torch.cuda.device(x1.device):
        code = _fn("tk3d_debug_chamfer_forward_route_f32")(
            ptr(x1), ptr(x2), i64(x1.size(0)), i64(x1.size(1)), i64(x2.size(1)),
            *[ptr(t) for t in out], ctypes.c_int(route), stream_of(x1))
    if code == UNSUPPORTED:
        return None
    assert code == 0, _lib.error_string(code)
    return out


def chamfer_sorted(x1, x2, counted=False, stages=7, ws=None, out=None):
    """Chamfer forward on sorted clouds whatever the size (the `always` workspace). Returns
    (outputs, workspace, counters): counters is None unless `counted`, else a list of four
    numbers - matrix instructions of the pruned sweep, waves that swept, queries scanned
    exactly, clouds handed to the sweep of all pairs. `stages` picks the launches (1 sort and
    key terms, 2 pruned sweep, 4 hand-over check) of a call on a given workspace `ws`."""
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    b, n1, n2 = x1.size(0), x1.size(1), x2.size(1)
    nbytes = _lib.chamfer_workspace_bytes(b, n1, n2, True)
    assert nbytes > 0, (b, n1, n2)
    if ws is None:
        ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=x1.device)
    if out is None:
        out = _chamfer_outputs(x1, x2)
    with torch.cuda.device(x1.device):
        if counted or stages != 7:
            counters = torch.empty(4, dtype=torch.int64, device=x1.device) if counted else None
            code = _fn("tk3d_debug_chamfer_forward_sorted_counted_f32")(
                ptr(x1), ptr(x2), i64(b), i64(n1), i64(n2), *[ptr(t) for t in out],
                ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(nbytes),
                ctypes.c_void_p(counters.data_ptr() if counted else 0), ctypes.c_int(stages),
                stream_of(x1))
        else:
            counters = None
            code = _fn("tk3d_chamfer_distance_forward_ws_f32")(
                ptr(x1), ptr(x2), i64(b), i64(n1), i64(n2), *[ptr(t) for t in out],
                ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(nbytes), stream_of(x1))
    assert code == 0, _lib.error_string(code)
    return out, ws, (counters.cpu().tolist() if counted else None)


def knn_filter(query, key, k):
    """(distance, index) of KNN through the pre-filtered kernel, or None when it does not take
    the shape (k > 16 or under 256 keys)."""
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    b, n1, n2 = query.size(0), query.size(1), key.size(1)
    dist = torch.empty((b, n1, k), device=query.device)
    idx = torch.empty((b, n1, k), dtype=torch.int64, device=query.device)
    with torch.cuda.device(query.device):
        code = _fn("tk3d_debug_knn_filter_f32")(ptr(query), ptr(key), i64(b), i64(n1), i64(n2),
                                                i64(k), ptr(dist), ptr(idx), stream_of(query))
    if code == UNSUPPORTED:
        return None
    assert code == 0, _lib.error_string(code)
    return dist, idx


def mfma_dot16(key_terms, query_terms):
    """scores [T,32,32] of one matrix instruction per tile; key_terms, query_terms: int16/uint16
    device tensors [T,32,16] of fp16 bit patterns."""
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    t = key_terms.size(0)
    scores = torch.empty((t, 32, 32), device=key_terms.device)
    with torch.cuda.device(key_terms.device):
        code = _fn("tk3d_debug_mfma_dot16_f16")(ptr(key_terms), ptr(query_terms), i64(t),
                                                ptr(scores), stream_of(key_terms))
    assert code == 0, _lib.error_string(code)
    return scores


def chamfer_scores(keys, queries):
    """scores [T,32,32] approximating |k|^2 - 2 q.k for centred, scaled points [T,32,3]."""
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    t = keys.size(0)
    scores = torch.empty((t, 32, 32), device=keys.device)
    with torch.cuda.device(keys.device):
        code = _fn("tk3d_debug_chamfer_scores_f32")(ptr(keys), ptr(queries), i64(t), ptr(scores),
                                                    stream_of(keys))
    assert code == 0, _lib.error_string(code)
    return scores
