"""Chamfer forward on sorted clouds (tk3d_chamfer_distance_forward_ws_f32) against the CPU
oracle, through the C ABI.

With a workspace the library orders both clouds along a space-filling curve and sweeps,
for every wave of queries, only the key tiles whose boxes are within reach. Whatever the
input, distances and indices must be bit-identical to the oracle (and so to the entry
point without a workspace): these cases aim at the pruning bound, the tie rule under a
permuted key order, the hand-over of clouds the bound does not cover, and the workspace
contract."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from test_gpu_chamfer import HARD_KINDS, _clouds, gen
from util import lattice_cloud, sphere_cloud, uniform_cloud

pytestmark = pytest.mark.gpu


def sorted_forward(a, c, cuda, workspace="exact", always=True):
    """[dist1, idx1, dist2, idx2] of the workspace entry point for CPU clouds a, c."""
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    x1, x2 = a.to(cuda).contiguous(), c.to(cuda).contiguous()
    b, n1, n2 = x1.size(0), x1.size(1), x2.size(1)
    nbytes = _lib.chamfer_workspace_bytes(b, n1, n2, always)
    ws, ws_ptr, ws_len = None, 0, 0
    if workspace == "exact" and nbytes:
        # stale contents must not matter: fill with a pattern that is no valid index
        ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=cuda)
        ws_ptr, ws_len = ws.data_ptr(), nbytes
    elif workspace == "short" and nbytes:
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=cuda)
        ws_ptr, ws_len = ws.data_ptr(), nbytes - 1
    elif workspace == "misaligned" and nbytes:
        ws = torch.empty((nbytes + 256,), dtype=torch.uint8, device=cuda)
        ws_ptr, ws_len = ws.data_ptr() + 16, nbytes
    out = [torch.empty((b, n1), device=cuda), torch.empty((b, n1), dtype=torch.int64, device=cuda),
           torch.empty((b, n2), device=cuda), torch.empty((b, n2), dtype=torch.int64, device=cuda)]
    fn = _lib.lib().tk3d_chamfer_distance_forward_ws_f32
    fn.restype = ctypes.c_int
    with torch.cuda.device(x1.device):
        code = fn(ptr(x1), ptr(x2), i64(b), i64(n1), i64(n2), *[ptr(t) for t in out],
                  ctypes.c_void_p(ws_ptr), ctypes.c_size_t(ws_len), stream_of(x1))
        torch.cuda.synchronize()
    assert code == 0, _lib.error_string(code)
    return out, ws


def handed_over(ws, b):
    """Per (direction, batch element): did the sorted path hand the cloud to the full sweep?"""
    at = (2 * b * 64 + 255) // 256 * 256
    return ws[at:at + 2 * b * 4].view(torch.int32).cpu().tolist()


def check_sorted(a, c, cuda, **kw):
    out, ws = sorted_forward(a, c, cuda, **kw)
    want = oracle.chamfer_forward(a.contiguous().numpy(), c.contiguous().numpy())
    for name, got, exp in zip(("dist1", "idx1", "dist2", "idx2"), out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp, err_msg=name)
    return ws


@pytest.mark.parametrize("b,n1,n2", [(2, 4096, 4096), (3, 2043, 1999), (1, 1, 1), (2, 5, 700),
                                     (2, 5000, 33), (4, 255, 257), (1, 127, 129), (2, 8193, 3001),
                                     (1, 16384, 16385), (1, 20000, 40000), (1, 65536, 4100),
                                     (300, 700, 900), (2, 60000, 16385)])
def test_shapes_on_uniform_and_sphere_clouds(cuda, b, n1, n2):
    # lengths that are no multiple of a tile (32), of the padding (128) or of a wave's
    # queries (64), one-point clouds, and both register layouts of the tile gaps (up to
    # 16384 keys and beyond)
    g = gen(n1 + n2)
    ws = check_sorted(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), cuda)
    assert sum(handed_over(ws, b)) == 0
    ws = check_sorted(sphere_cloud(g, b, n1), sphere_cloud(g, b, n2), cuda)
    assert sum(handed_over(ws, b)) == 0


@pytest.mark.parametrize("kind", HARD_KINDS)
def test_hard_inputs(cuda, kind):
    a, c = _clouds(kind, gen(sum(map(ord, kind)) + 5))
    check_sorted(a.contiguous(), c.contiguous(), cuda)


@pytest.mark.parametrize("kind", ["lattice", "duplicates", "clusters", "far_queries",
                                  "nan_and_inf", "separated"])
def test_hard_inputs_on_longer_clouds(cuda, kind):
    a, c = _clouds(kind, gen(sum(map(ord, kind)) + 6), 2, 6000, 9001)
    check_sorted(a.contiguous(), c.contiguous(), cuda)


def test_ties_go_to_the_lowest_original_index(cuda):
    # every key position occurs many times, at indices far apart: sorted order puts the
    # copies next to each other in an order of its own, the result must still name the
    # lowest original index (the reference's strict '<' over ascending j)
    g = gen(11)
    base = uniform_cloud(g, 2, 300)
    c = base.repeat(1, 12, 1)[:, torch.randperm(3600, generator=g)].contiguous()
    a = uniform_cloud(g, 2, 2500)
    a[:, :300] = base                                # queries that coincide with keys
    ws = check_sorted(a, c, cuda)
    # lattice clouds: exact ties between different positions as well
    check_sorted(lattice_cloud(g, 2, 4096, 6), lattice_cloud(g, 2, 5000, 6), cuda)
    assert ws is not None


def test_clouds_the_bound_does_not_cover_are_handed_over(cuda):
    g = gen(12)
    a, c = sphere_cloud(g, 3, 3000), sphere_cloud(g, 3, 3500)
    c[1, 77, 2] = float("nan")          # batch element 1: a NaN key
    a[2] = a[2] * 1e-30                 # batch element 2: extent below 2^-40
    ws = check_sorted(a, c, cuda)
    flags = handed_over(ws, 3)
    assert flags[0] == 0 and flags[3] == 0          # element 0 stays on the sorted path
    assert flags[1] == 1 and flags[4] == 1 and flags[2] == 1 and flags[5] == 1
    # queries more than 8000 key extents away
    far = sphere_cloud(g, 1, 2500) * 1e-3
    ws = check_sorted(far + 100.0, far, cuda)
    assert handed_over(ws, 1) == [1, 1]


def test_disjoint_and_nested_clouds(cuda):
    g = gen(13)
    a, c = sphere_cloud(g, 2, 3000), sphere_cloud(g, 2, 4000)
    ws = check_sorted(a + 3.0, c, cuda)            # no key tile overlaps any patch
    assert sum(handed_over(ws, 2)) == 0
    ws = check_sorted(a * 0.01, c, cuda)           # all queries deep inside the key cloud;
    assert handed_over(ws, 2) == [0, 0, 1, 1]      # the other way round the keys are dwarfed
    ws = check_sorted(a, c * 0.01, cuda)           # all keys in one small region:
    assert handed_over(ws, 2) == [1, 1, 0, 0]      # boxes cannot prune for the far queries
    ws = check_sorted(a, c * 0.3, cuda)            # a key cloud of a third of the extent stays
    assert sum(handed_over(ws, 2)) == 0


def test_queries_clustered_inside_a_shell_of_keys_are_handed_over(cuda):
    # All queries in a small cluster at the centre of a shell of keys: every key tile is about
    # as far from them as the nearest one, and every wave would sweep nearly all of them.
    # From 256 key tiles (8192 keys) on that direction is handed over as well (the other way
    # round the keys are dwarfed); inside a filled cube of keys the same cluster has a few
    # tiles next to it and stays on the sorted path, and so does a shell of fewer tiles.
    g = gen(22)
    shell, cluster = sphere_cloud(g, 2, 9000), sphere_cloud(g, 2, 8200) * 0.01
    ws = check_sorted(cluster, shell, cuda)
    assert handed_over(ws, 2) == [1, 1, 1, 1]
    ws = check_sorted(shell, cluster, cuda)
    assert handed_over(ws, 2) == [1, 1, 1, 1]
    ws = check_sorted(cluster, uniform_cloud(g, 2, 9000), cuda)
    assert handed_over(ws, 2) == [0, 0, 1, 1]
    ws = check_sorted(cluster + 0.5, uniform_cloud(g, 2, 9000), cuda)   # off centre
    assert handed_over(ws, 2) == [0, 0, 1, 1]
    ws = check_sorted(cluster + 3.0, uniform_cloud(g, 2, 9000), cuda)   # outside the keys
    assert handed_over(ws, 2) == [0, 0, 1, 1]
    ws = check_sorted(cluster, sphere_cloud(g, 2, 8000), cuda)          # 250 tiles
    assert handed_over(ws, 2) == [0, 0, 1, 1]


def test_keys_crowded_into_few_cells_are_handed_over(cuda):
    # A few hundred distinct points on a line, each repeated about 50 times: over a hundred
    # keys per occupied cell of the 32^3 grid, several tiles of equal keys in front of every
    # query. Both directions go to the sweep of all pairs before any wave sweeps; the same
    # repetition spread over a volume (about 50 keys per occupied cell) stays.
    g = gen(21)
    n = 8192
    t = torch.rand(2, n // 50, 1, generator=g) * torch.tensor([1.0, 0.5, -0.25])
    pick1 = torch.randint(0, n // 50, (n,), generator=g)
    pick2 = torch.randint(0, n // 50, (n,), generator=g)
    ws = check_sorted(t[:, pick1].contiguous(), t[:, pick2].contiguous(), cuda)
    assert handed_over(ws, 2) == [1, 1, 1, 1]
    v = sphere_cloud(g, 2, n // 50)
    ws = check_sorted(v[:, pick1].contiguous(), v[:, pick2].contiguous(), cuda)
    assert sum(handed_over(ws, 2)) == 0
    # points on a line without repetition: crowded as well (a cell holds 8192 / ~50 keys)
    line = torch.rand(2, n, 1, generator=g) * torch.tensor([1.0, 0.5, -0.25])
    ws = check_sorted(line, line.flip(1).contiguous() + 1e-3, cuda)
    assert handed_over(ws, 2) == [1, 1, 1, 1]


def test_workspace_contract(cuda):
    from torkit3d_amd import _lib

    g = gen(14)
    a, c = sphere_cloud(g, 2, 5000), sphere_cloud(g, 2, 4500)
    for mode in ("none", "short", "misaligned"):   # falls back to the plain entry point
        check_sorted(a, c, cuda, workspace=mode)
    # the size function: 0 where the path cannot serve or (always = 0) does not pay
    size = _lib.chamfer_workspace_bytes
    assert size(32, 16384, 16384) > 0 and size(1, 65536, 65536) > 0
    assert size(2, 1024, 1024) == 0 and size(2, 1024, 1024, True) > 0
    assert size(4, 65536, 2048) == 0 and size(4, 65536, 2048, True) > 0
    assert size(1, 65537, 65536, True) == 0 and size(0, 4096, 4096, True) == 0
    per_point = size(1, 4096, 4096, True) / 8192
    assert 48 < per_point < 52                     # 16 + 32 bytes per point + boxes


def test_two_calls_share_a_workspace_and_a_stream(cuda):
    # a second call on other clouds reuses the buffer: nothing of the first may leak
    g = gen(15)
    a, c = sphere_cloud(g, 2, 6000), sphere_cloud(g, 2, 6000)
    _, ws = sorted_forward(a, c, cuda)
    a2, c2 = uniform_cloud(g, 2, 6000), uniform_cloud(g, 2, 6000)
    from torkit3d_amd._lib import i64, ptr, stream_of
    from torkit3d_amd import _lib

    x1, x2 = a2.to(cuda), c2.to(cuda)
    out = [torch.empty((2, 6000), device=cuda), torch.empty((2, 6000), dtype=torch.int64, device=cuda),
           torch.empty((2, 6000), device=cuda), torch.empty((2, 6000), dtype=torch.int64, device=cuda)]
    fn = _lib.lib().tk3d_chamfer_distance_forward_ws_f32
    fn.restype = ctypes.c_int
    assert fn(ptr(x1), ptr(x2), i64(2), i64(6000), i64(6000), *[ptr(t) for t in out],
              ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()), stream_of(x1)) == 0
    torch.cuda.synchronize()
    want = oracle.chamfer_forward(a2.numpy(), c2.numpy())
    for got, exp in zip(out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp)


def test_full_size_through_the_python_api_uses_the_sorted_path(cuda):
    # the benchmark shape is inside the domain where the shim lends a workspace; the
    # result is compared with the entry point that takes none
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    assert _lib.chamfer_workspace_bytes(32, 16384, 16384) > 0
    g = gen(16)
    x1, x2 = sphere_cloud(g, 32, 16384).to(cuda), sphere_cloud(g, 32, 16384).to(cuda)
    got = nn_distance(x1, x2)
    ref = [torch.empty_like(got[0]), torch.empty_like(got[1]), torch.empty_like(got[2]),
           torch.empty_like(got[3])]
    _lib.call("tk3d_chamfer_distance_forward", x1, ptr(x1), ptr(x2), i64(32), i64(16384),
              i64(16384), *[ptr(t) for t in ref], stream_of(x1))
    torch.cuda.synchronize()
    for name, a_, b_ in zip(("dist1", "idx1", "dist2", "idx2"), got, ref):
        assert torch.equal(a_, b_), name


def test_captured_in_a_hip_graph_and_replayed(cuda):
    # five launches, no allocation, no memset, flags cleared by a kernel: the call records
    # into a graph as it is; replays on new input contents, with eager work in between,
    # must equal the oracle every time (workspace and outputs held outside the graph)
    from torkit3d_amd import _lib
    from torkit3d_amd._lib import i64, ptr, stream_of

    b, n1, n2 = 2, 5000, 6000
    assert _lib.chamfer_workspace_bytes(b, n1, n2, True) > 0
    g = gen(17)
    x1 = sphere_cloud(g, b, n1).to(cuda)
    x2 = sphere_cloud(g, b, n2).to(cuda)
    ws = torch.empty((_lib.chamfer_workspace_bytes(b, n1, n2, True),), dtype=torch.uint8,
                     device=cuda)
    out = [torch.empty((b, n1), device=cuda), torch.empty((b, n1), dtype=torch.int64, device=cuda),
           torch.empty((b, n2), device=cuda), torch.empty((b, n2), dtype=torch.int64, device=cuda)]
    fn = _lib.lib().tk3d_chamfer_distance_forward_ws_f32
    fn.restype = ctypes.c_int

    def call():
        assert fn(ptr(x1), ptr(x2), i64(b), i64(n1), i64(n2), *[ptr(t) for t in out],
                  ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()),
                  stream_of(x1)) == 0

    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    with torch.cuda.stream(side):
        call()                        # warm-up outside the capture
    torch.cuda.current_stream(cuda).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for seed, kind in ((18, sphere_cloud), (19, uniform_cloud), (20, lattice_cloud)):
        g = gen(seed)
        a = kind(g, b, n1) if kind is not lattice_cloud else lattice_cloud(g, b, n1, 8)
        c = kind(g, b, n2) if kind is not lattice_cloud else lattice_cloud(g, b, n2, 8)
        x1.copy_(a)
        x2.copy_(c)
        for t in out:
            t.zero_()
        (x1.sum() + x2.sum()).item()  # eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        want = oracle.chamfer_forward(a.numpy(), c.numpy())
        for name, got, exp in zip(("dist1", "idx1", "dist2", "idx2"), out, want):
            np.testing.assert_array_equal(got.cpu().numpy(), exp, err_msg="%s seed %d" % (name, seed))


def test_stray_points_stay_on_the_sorted_path(cuda):
    # a few points far outside the cloud would blow up its bounding box, and with it the
    # cells of the sort and the scale of the fp16 terms: the frame is trimmed instead and
    # the strays are compared with every query directly
    g = gen(21)
    a, c = sphere_cloud(g, 3, 5000), sphere_cloud(g, 3, 6000)
    c[0, 17] = torch.tensor([300.0, -2.0, 5.0])            # one stray key
    c[1, ::1000] = c[1, ::1000] * 50.0 + 40.0              # six of them
    c[1, 4000] = c[1, 3000]                                # two strays at one position: the lower index wins
    a[2, 123] = torch.tensor([-80.0, 90.0, 10.0])          # a stray query
    a[2, 124] = c[2, 5999] = torch.tensor([25.0, 25.0, 25.0])  # a stray query on a stray key
    ws = check_sorted(a, c, cuda)
    assert sum(handed_over(ws, 3)) == 0
    far_keys = ws[: 2 * 3 * 64].view(torch.int32).view(2, 3, 16)[:, :, 13].cpu().tolist()
    assert far_keys[1][0] == 1 and far_keys[1][1] == 6 and far_keys[1][2] == 1 and far_keys[0][2] == 2
    # more strays than the list holds: the cloud is handed over
    c2 = sphere_cloud(g, 1, 6000)
    c2[0, ::60] = c2[0, ::60] * 100.0
    ws = check_sorted(sphere_cloud(g, 1, 5000), c2, cuda)
    assert handed_over(ws, 1)[0] == 1
    # strays that are the nearest keys of far queries, and a far cloud of queries
    a3, c3 = sphere_cloud(g, 2, 4000), sphere_cloud(g, 2, 4000)
    c3[:, 5] = torch.tensor([60.0, 0.0, 0.0])
    a3[:, 100:140] = a3[:, 100:140] + torch.tensor([59.0, 0.0, 0.0])
    check_sorted(a3, c3, cuda)


def test_stray_queries_beyond_the_reach_of_the_fp16_terms(cuda):
    # a few queries more than 8000 key extents away are scanned exactly against all keys;
    # the cloud stays on the sorted path in both directions (as keys they are far keys)
    g = gen(22)
    a, c = sphere_cloud(g, 2, 5000), sphere_cloud(g, 2, 4500)
    a[0, 11] = torch.tensor([3.0e4, 0.0, 0.0])
    a[1, 4000] = torch.tensor([-1.0e5, 2.0e5, 7.0e4])
    a[1, 4999] = torch.tensor([5.0e5, 5.0e5, 5.0e5])
    ws = check_sorted(a, c, cuda)
    assert sum(handed_over(ws, 2)) == 0
    # a wave of nothing but stray queries and padding: 4480 + 30 queries, the last 30 far away
    a2 = sphere_cloud(g, 1, 4510)
    a2[0, 4480:] = a2[0, 4480:] * 10.0 + 4.0e4
    ws = check_sorted(a2, sphere_cloud(g, 1, 4500), cuda)
    assert sum(handed_over(ws, 1)) == 0
    # too many of them for exact scans: handed over
    a3 = sphere_cloud(g, 1, 5000)
    a3[0, ::3] = a3[0, ::3] + 5.0e4
    ws = check_sorted(a3, sphere_cloud(g, 1, 4500), cuda)
    assert handed_over(ws, 1)[0] == 1


def test_a_cloud_of_identical_points(cuda):
    # all keys in one place: the answer is key 0 for every query, without a sweep; the
    # other way round (identical queries) is an ordinary, small patch
    g = gen(23)
    a = sphere_cloud(g, 2, 5000)
    c = torch.tensor([0.3, -0.2, 0.9]).expand(2, 4500, 3).contiguous()
    ws = check_sorted(a, c, cuda)
    assert sum(handed_over(ws, 2)) == 0
    ws = check_sorted(c, c.clone(), cuda)
    assert sum(handed_over(ws, 2)) == 0
    far = (c * 3.0e19).contiguous()          # distances overflow: (+inf, -1)
    check_sorted(-far, far, cuda)
