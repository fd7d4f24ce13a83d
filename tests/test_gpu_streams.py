"""The library keeps no device state between calls (scratch lives in the caller's outputs
and workspace), so calls on different streams may overlap. Two streams (default
priority) run the ops on different inputs at the same time; each result must equal the
one obtained alone."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def ops(points, keys, feature):
    from torkit3d_amd import _C

    d1, i1, d2, i2 = _C.chamfer_distance_forward_cuda(points, keys)       # key-sliced sweep
    sel = _C.sample_farthest_points_cuda(points, 64)                       # register kernel
    far = _C.sample_farthest_points_cuda(keys, 40)                         # one launch per step
    kd, ki = _C.knn_distance_cuda(points, keys, 16, 1)
    nbr = _C.ball_query_cuda(points[:, :256].contiguous(), keys, 0.3, 16)
    grouped = _C.group_points_forward_cuda(feature, nbr)
    back = _C.group_points_backward_cuda(grouped, nbr, feature.size(2))
    return [d1, i1, d2, i2, sel, far, kd, ki, nbr, grouped, back]


def test_calls_on_two_streams_overlap_safely(cuda):
    g = torch.Generator().manual_seed(3)
    data = []
    for _ in range(2):
        data.append((torch.rand(2, 3000, 3, generator=g).to(cuda),
                     torch.rand(2, 20000, 3, generator=g).to(cuda),
                     torch.randn(2, 8, 20000, generator=g).to(cuda)))
    alone = [ops(*d) for d in data]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(3):
        together = []
        for st, d in zip(streams, data):
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                together.append(ops(*d))
        for st in streams:
            torch.cuda.current_stream().wait_stream(st)
        torch.cuda.synchronize()
        for a_list, t_list in zip(alone, together):
            for i, (a, t) in enumerate(zip(a_list, t_list)):
                assert torch.equal(a, t), "output %d differs when two streams overlap" % i
