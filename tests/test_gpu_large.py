"""Largest shapes: tensors past 2^31 elements (the reference's interpolate kernels index
with 32-bit ints, torkit3d/csrc/cuda/interpolate_kernel.cu:19-33, and would wrap there)
and single clouds far beyond the benchmark sizes. Checked against stock torch ops on the
GPU where those are exact, against the oracle otherwise."""
import numpy as np
import pytest
import torch

import oracle
from util import uniform_cloud

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def test_group_points_past_two_to_the_32_elements(cuda):
    from torkit3d_amd import _C

    b, c, n1, n2, k = 2, 128, 1024, 262144 + 192, 64
    assert b * c * n2 * k > 2 ** 32
    g = gen(1)
    feat = torch.randn(b, c, n1, generator=g).to(cuda)
    index = torch.randint(0, n1, (b, n2, k), generator=g).to(cuda)
    out = _C.group_points_forward_cuda(feat, index)
    flat = index.view(b, 1, n2 * k).expand(b, c, n2 * k)
    want = torch.gather(feat, 2, flat).view(b, c, n2, k)
    assert torch.equal(out, want)
    del want
    # Integer-valued gradients: every partial sum is exact in fp32, in any order.
    torch.manual_seed(1)
    out.copy_(torch.randint(-3, 4, (c, n2, k), device=cuda).unsqueeze(0))
    got = _C.group_points_backward_cuda(out, index, n1)
    want = torch.zeros(b, c, n1, device=cuda).scatter_add_(2, flat, out.view(b, c, n2 * k))
    assert torch.equal(got, want)


def test_interpolate_past_two_to_the_31_elements(cuda):
    from torkit3d_amd import _C

    b, c, n1, n2 = 2, 256, 2048, 4194304 + 64
    assert b * c * n2 > 2 ** 31
    g = gen(2)
    feat = torch.randint(-8, 9, (b, c, n1), generator=g).float().to(cuda)
    index = torch.randint(0, n1, (b, n2, 3), generator=g).to(cuda)
    # Weights k/4: products and sums of three stay exact in fp32.
    weight = (torch.randint(0, 5, (b, n2, 3), generator=g).float() / 4).to(cuda)
    out = _C.interpolate_forward_cuda(feat, index, weight)
    want = torch.zeros_like(out)
    for i in range(3):
        want += torch.gather(feat, 2, index[:, None, :, i].expand(b, c, n2)) * weight[:, None, :, i]
    assert torch.equal(out, want)
    del want
    torch.manual_seed(2)
    out.copy_(torch.randint(-2, 3, (c, n2), device=cuda).unsqueeze(0))
    got = _C.interpolate_backward_cuda(out, index, weight, n1)
    want = torch.zeros(b, c, n1, device=cuda)
    for i in range(3):
        want.scatter_add_(2, index[:, None, :, i].expand(b, c, n2), out * weight[:, None, :, i])
    assert torch.equal(got, want)


def test_chamfer_on_one_large_cloud(cuda):
    from torkit3d_amd import _C

    a, c = uniform_cloud(gen(3), 1, 150000), uniform_cloud(gen(4), 1, 200001)
    want = oracle.chamfer_forward(a.numpy(), c.numpy())
    got = _C.chamfer_distance_forward_cuda(a.to(cuda), c.to(cuda))
    for w, t in zip(want, got):
        assert np.array_equal(t.cpu().numpy(), w)
    g1 = torch.randn(1, 150000, generator=gen(5))
    g2 = torch.randn(1, 200001, generator=gen(6))
    want = oracle.chamfer_backward(g1.numpy(), g2.numpy(), a.numpy(), c.numpy(), want[1], want[3])
    got = _C.chamfer_distance_backward_cuda(g1.to(cuda), g2.to(cuda), a.to(cuda), c.to(cuda),
                                            got[1], got[3])
    for w, t in zip(want, got):
        np.testing.assert_allclose(t.cpu().numpy(), w, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("k", [3, 16, 40])
def test_knn_against_very_many_keys(cuda, k):
    from torkit3d_amd import _C

    q, key = uniform_cloud(gen(7), 1, 9000), uniform_cloud(gen(8), 1, 700001)
    want_d, want_i = oracle.knn(q.numpy(), key.numpy(), k)
    d, i = _C.knn_distance_cuda(q.to(cuda), key.to(cuda), k, 1)
    assert np.array_equal(i.cpu().numpy(), want_i)
    assert np.array_equal(d.cpu().numpy(), want_d)


def test_ball_query_against_very_many_keys(cuda):
    from torkit3d_amd import _C

    q, key = uniform_cloud(gen(9), 2, 3000), uniform_cloud(gen(10), 2, 1000003)
    # Radius 0.02: about 4 hits in a million keys, so most rows scan every key and many
    # stay short of max_neighbors.
    want = oracle.ball_query(q.numpy(), key.numpy(), 0.02, 8)
    got = _C.ball_query_cuda(q.to(cuda), key.to(cuda), 0.02, 8)
    assert np.array_equal(got.cpu().numpy(), want)
    assert (want[:, :, 0] < 0).any() and (want[:, :, -1] != want[:, :, 0]).any()


@pytest.mark.parametrize("n,k", [(1000003, 96), (300000, 700)])
def test_fps_on_one_very_large_cloud(cuda, n, k):
    from torkit3d_amd import _C

    pts = uniform_cloud(gen(11), 2, n)
    want = oracle.sample_farthest_points(pts.numpy(), k)
    got = _C.sample_farthest_points_cuda(pts.to(cuda), k)
    assert np.array_equal(got.cpu().numpy(), want)
