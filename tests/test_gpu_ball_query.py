"""Ball query on the GPU: indices bit-identical to the oracle, plus the reference's
own test construction in fp64."""
import numpy as np
import pytest
import torch

import oracle
from util import ball_query_numpy, lattice_cloud

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("b,n1,n2,r,k,transpose", [(2, 64, 128, 0.1, 32, True),
                                                    (3, 65, 129, 0.1, 32, True),
                                                    (3, 65, 129, 10.0, 32, True),
                                                    (3, 65, 129, 0.1, 32, False),
                                                    (32, 512, 1024, 0.1, 64, True)])
def test_reference_cases_fp64(cuda, b, n1, n2, r, k, transpose):
    # tests/ops/test_ball_query.py:6-60
    from torkit3d_amd.ops.ball_query import ball_query

    np.random.seed(0)
    key = np.random.randn(b, n2, 3)
    query = np.array([p[np.random.choice(n2, n1, replace=False)] for p in key])
    want = oracle.ball_query(query, key, r, k)
    if b <= 3:
        np.testing.assert_array_equal(want, ball_query_numpy(query, key, r, k))
    qt, kt = torch.tensor(query).to(cuda), torch.tensor(key).to(cuda)
    if transpose:
        qt, kt = qt.transpose(1, 2).contiguous(), kt.transpose(1, 2).contiguous()
    got = ball_query(qt, kt, r, k, transpose=transpose)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_grouping_config_fp32(cuda):
    # benchmark config 3: B=16, 4096 support points in the unit cube, 1024 centres taken
    # by FPS, radius 0.2, 32 neighbours
    from torkit3d_amd import _C

    g = gen(3)
    xyz = torch.rand(16, 4096, 3, generator=g)
    centres_idx = oracle.sample_farthest_points(xyz.numpy(), 1024)
    centres = np.take_along_axis(xyz.numpy(), centres_idx[:, :, None], 1)
    got = _C.ball_query_cuda(torch.from_numpy(centres).to(cuda), xyz.to(cuda), 0.2, 32)
    np.testing.assert_array_equal(got.cpu().numpy(),
                                  oracle.ball_query(centres, xyz.numpy(), 0.2, 32))


@pytest.mark.parametrize("n2,n1,r,k", [(16384, 4096, 0.1, 32), (4096, 1024, 0.2, 32),
                                       (1024, 256, 0.4, 64)])
def test_set_abstraction_chain_shapes(cuda, n2, n1, r, k):
    # benchmark config 5, B=8
    from torkit3d_amd import _C

    g = gen(5)
    key = torch.rand(8, n2, 3, generator=g)
    query = key[:, torch.randperm(n2, generator=g)[:n1]].contiguous()
    got = _C.ball_query_cuda(query.to(cuda), key.to(cuda), r, k)
    np.testing.assert_array_equal(got.cpu().numpy(),
                                  oracle.ball_query(query.numpy(), key.numpy(), r, k))


def test_edge_cases(cuda):
    from torkit3d_amd import _C

    g = gen(8)
    key = lattice_cloud(g, 2, 700, 8)
    query = torch.cat([key[:, :45], torch.full((2, 3, 3), 9.0)], dim=1).contiguous()
    for r, k in ((0.25, 16), (0.25, 1), (0.125, 100), (5.0, 700), (1e-6, 4)):
        got = _C.ball_query_cuda(query.to(cuda), key.to(cuda), r, k).cpu().numpy()
        np.testing.assert_array_equal(got, oracle.ball_query(query.numpy(), key.numpy(), r, k))
    assert (got[:, 45:] == -1).all()  # no hit: the row stays -1
    # tiny radius, queries are key points: the only hits are coincident points, first one padded
    # (a lattice cloud repeats positions, so a row lists up to 4 coincident key indices in
    # ascending order and pads with the first)
    own = key[:, :10].contiguous()
    got = _C.ball_query_cuda(own.to(cuda), key.to(cuda), 1e-6, 4).cpu().numpy()
    np.testing.assert_array_equal(got, oracle.ball_query(own.numpy(), key.numpy(), 1e-6, 4))
    hit = torch.gather(key, 1, torch.from_numpy(got).reshape(2, -1, 1).expand(-1, -1, 3))
    assert torch.equal(hit.view(2, 10, 4, 3), own[:, :, None, :].expand(-1, -1, 4, -1))
    assert (got[:, :, 0] <= np.arange(10)[None, :]).all()  # the first coincident key
    # empty key cloud and k = 0
    out = _C.ball_query_cuda(query.to(cuda), torch.zeros(2, 0, 3, device=cuda), 0.5, 5)
    assert (out == -1).all()
    assert _C.ball_query_cuda(query.to(cuda), key.to(cuda), 0.5, 0).shape == (2, 48, 0)
