"""Chamfer / nearest-neighbour distance on the GPU against the CPU oracle.

Indices and distances must be bit-identical to the oracle (same canonical
arithmetic); fp32 gradients within 1e-5 relative / 1e-6 absolute of the oracle's sums
taken in double and rounded once (the kernel sums in 64-bit fixed point, the reference's
atomics in an order that changes from run to run)."""
import numpy as np
import pytest
import torch

import oracle
from util import lattice_cloud, sphere_cloud, uniform_cloud

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-5, 1e-6


def gen(seed):
    return torch.Generator().manual_seed(seed)


def check_forward(a, c, cuda):
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    out = nn_distance(a.to(cuda), c.to(cuda))
    want = oracle.chamfer_forward(a.numpy(), c.numpy())
    for name, got, exp in zip(("dist1", "idx1", "dist2", "idx2"), out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp, err_msg=name)
    return out


@pytest.mark.parametrize("b,n1,n2", [(2, 1024, 1024),     # benchmark config 1
                                     (32, 2048, 2048),    # reference test, NWC
                                     (3, 2043, 1999),     # not multiples of any tile
                                     (1, 1, 1), (2, 5000, 33), (2, 33, 5000), (4, 255, 257)])
def test_forward_matches_oracle(cuda, b, n1, n2):
    g = gen(1)
    check_forward(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), cuda)


def test_forward_fp64_and_transpose(cuda):
    # reference test, NCW layout (tests/ops/test_chamfer_distance.py:86-99), here in fp64
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    g = gen(2)
    a = torch.rand(4, 3, 2043, generator=g, dtype=torch.float64)
    c = torch.rand(4, 3, 2043, generator=g, dtype=torch.float64)
    out = nn_distance(a.to(cuda), c.to(cuda), transpose=True)
    want = oracle.chamfer_forward(a.transpose(1, 2).contiguous().numpy(),
                                  c.transpose(1, 2).contiguous().numpy())
    for got, exp in zip(out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp)
    D = ((a[:, :, :, None] - c[:, :, None, :]) ** 2).sum(1)
    assert torch.equal(out[1].cpu(), D.argmin(2)) and torch.equal(out[3].cpu(), D.argmin(1))


def check_backward(a, c, gd1, gd2, i1, i2, cuda, exact_nonfinite=False):
    """tk3d_chamfer_distance_backward through _C against the double-summing oracle."""
    from torkit3d_amd import _C

    got = _C.chamfer_distance_backward_cuda(gd1.to(cuda), gd2.to(cuda), a.to(cuda), c.to(cuda),
                                            torch.as_tensor(i1).to(cuda), torch.as_tensor(i2).to(cuda))
    want = oracle.chamfer_backward(gd1.numpy(), gd2.numpy(), a.numpy(), c.numpy(),
                                   np.asarray(i1), np.asarray(i2), wide=True)
    for name, g, w in zip(("grad_xyz1", "grad_xyz2"), got, want):
        g = g.cpu().numpy()
        if exact_nonfinite:
            assert np.array_equal(np.isnan(g), np.isnan(w)), name
            assert np.array_equal(np.isposinf(g), np.isposinf(w)), name
            assert np.array_equal(np.isneginf(g), np.isneginf(w)), name
            ok = np.isfinite(w)
            g, w = g[ok], w[ok]
        np.testing.assert_allclose(g, w, rtol=RTOL, atol=ATOL, err_msg=name)
    return got


def test_stress_config_full_size(cuda):
    # benchmark config 5: B=32, N=M=16384, points on unit spheres + N(0, 0.01) noise,
    # forward and backward
    g = gen(5)
    a, c = sphere_cloud(g, 32, 16384), sphere_cloud(g, 32, 16384)
    d1, i1, d2, i2 = check_forward(a, c, cuda)
    # size-independent invariants: each distance is the distance to the reported point
    ga = torch.gather(c.to(cuda), 1, i1[:, :, None].expand(-1, -1, 3))
    np.testing.assert_allclose(((a.to(cuda) - ga) ** 2).sum(-1).cpu().numpy(),
                               d1.cpu().numpy(), rtol=1e-5, atol=1e-7)
    assert float(d1.max()) < 0.05 and int(i1.min()) >= 0 and int(i1.max()) < 16384
    gd1, gd2 = torch.randn(32, 16384, generator=g), torch.randn(32, 16384, generator=g)
    gx1, gx2 = check_backward(a, c, gd1, gd2, i1.cpu(), i2.cpu(), cuda)
    # the terms sent to the other cloud cancel the own terms: both gradients sum to the
    # same total with opposite sign (each pass adds v to one cloud and -v to the other)
    t1 = gx1.double().sum(1).cpu().numpy()
    t2 = gx2.double().sum(1).cpu().numpy()
    np.testing.assert_allclose(t1, -t2, rtol=1e-4, atol=1e-3)


def test_lattice_ties_pick_lowest_index(cuda):
    g = gen(3)
    a, c = lattice_cloud(g, 3, 700, 4), lattice_cloud(g, 3, 900, 4)
    _, i1, _, i2 = check_forward(a, c, cuda)
    D = ((a[:, :, None, :].double() - c[:, None, :, :].double()) ** 2).sum(-1)
    assert torch.equal(i1.cpu(), D.argmin(2)) and torch.equal(i2.cpu(), D.argmin(1))


def test_identical_clouds_and_swapped_arguments(cuda):
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    g = gen(4)
    a = uniform_cloud(g, 2, 3000).to(cuda)
    d1, i1, d2, i2 = nn_distance(a, a)
    assert float(d1.abs().max()) == 0 and float(d2.abs().max()) == 0
    assert torch.equal(i1.cpu(), torch.arange(3000).expand(2, -1))
    c = uniform_cloud(g, 2, 777).to(cuda)
    x, y = nn_distance(a, c), nn_distance(c, a)
    for u, v in zip(x, (y[2], y[3], y[0], y[1])):
        assert torch.equal(u, v)


def test_empty_and_nan_clouds(cuda):
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    a = torch.zeros(2, 5, 3, device=cuda)
    d1, i1, d2, i2 = nn_distance(a, torch.zeros(2, 0, 3, device=cuda))
    assert torch.isinf(d1).all() and (i1 == -1).all() and d2.shape == (2, 0)
    d1, i1, _, _ = nn_distance(a, torch.full((2, 7, 3), float("nan"), device=cuda))
    assert torch.isinf(d1).all() and (i1 == -1).all()
    out = nn_distance(torch.zeros(0, 5, 3, device=cuda), torch.zeros(0, 4, 3, device=cuda))
    assert out[0].shape == (0, 5) and out[3].shape == (0, 4)
    # 2-D inputs get a batch dimension (torkit3d/ops/chamfer_distance.py:48-51)
    out = nn_distance(torch.rand(6, 3, device=cuda), torch.rand(4, 3, device=cuda))
    assert out[0].shape == (1, 6) and out[2].shape == (1, 4)


@pytest.mark.parametrize("b,n1,n2", [(2, 1024, 1024), (3, 300, 5000), (5, 4097, 9000)])
def test_backward_matches_oracle(cuda, b, n1, n2):
    from torkit3d_amd.ops.chamfer_distance import chamfer_distance

    g = gen(1)
    a, c = uniform_cloud(g, b, n1), uniform_cloud(g, b, n2)
    gd1, gd2 = torch.randn(b, n1, generator=g), torch.randn(b, n2, generator=g)
    ad, cd = a.to(cuda).requires_grad_(), c.to(cuda).requires_grad_()
    d1, d2 = chamfer_distance(ad, cd)
    torch.autograd.backward([d1, d2], [gd1.to(cuda), gd2.to(cuda)])
    _, i1, _, i2 = oracle.chamfer_forward(a.numpy(), c.numpy())
    gx1, gx2 = oracle.chamfer_backward(gd1.numpy(), gd2.numpy(), a.numpy(), c.numpy(), i1, i2,
                                       wide=True)
    np.testing.assert_allclose(ad.grad.cpu().numpy(), gx1, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(cd.grad.cpu().numpy(), gx2, rtol=RTOL, atol=ATOL)


def test_backward_with_an_empty_cloud_or_unmatched_points(cuda):
    from torkit3d_amd import _C
    from torkit3d_amd.ops.chamfer_distance import chamfer_distance

    g = gen(2)
    # one cloud empty: no point has a match, every gradient is zero
    a = uniform_cloud(g, 2, 700).to(cuda).requires_grad_()
    for empty_first in (False, True):
        e = torch.zeros(2, 0, 3, device=cuda, requires_grad=True)
        d1, d2 = chamfer_distance(e, a) if empty_first else chamfer_distance(a, e)
        a.grad = None
        torch.autograd.backward([d1, d2], [torch.ones_like(d1), torch.ones_like(d2)])
        assert a.grad.shape == (2, 700, 3) and float(a.grad.abs().max()) == 0.0
        assert e.grad.shape == (2, 0, 3)
    # all-NaN keys: the forward reports index -1, which the backward must skip
    an, cn = uniform_cloud(g, 2, 300), torch.full((2, 200, 3), float("nan"))
    _, i1, _, i2 = _C.chamfer_distance_forward_cuda(an.to(cuda), cn.to(cuda))
    assert (i1 == -1).all()
    gd1, gd2 = torch.randn(2, 300, generator=g), torch.zeros(2, 200)
    gx1, gx2 = _C.chamfer_distance_backward_cuda(gd1.to(cuda), gd2.to(cuda), an.to(cuda),
                                                 cn.to(cuda), i1, torch.full_like(i2, -1))
    assert float(gx1.abs().max()) == 0.0 and float(gx2.abs().max()) == 0.0


@pytest.mark.parametrize("n2,where", [(5000, 300), (20000, 1500), (20000, 19999), (70000, 8000)])
def test_backward_outlier_missed_by_the_magnitude_sample(cuda, n2, where):
    # The fixed-point scale comes from the terms of the first round of senders: runs of 1024
    # consecutive senders, every rounds-th run, rounds = ceil(n2 / 8192). A term far above 8x
    # that maximum in a later round must send the workgroup through its second attempt with
    # the exact bound. (With 5000 senders there is one round and the bound is exact at once.)
    g = gen(3)
    a, c = uniform_cloud(g, 2, 3000), uniform_cloud(g, 2, n2)
    gd1, gd2 = torch.randn(2, 3000, generator=g), torch.randn(2, n2, generator=g)
    rounds = -(-n2 // 8192)
    assert rounds == 1 or (where // 1024) % rounds != 0
    gd2[1, where] = 2.0e6
    _, i1, _, i2 = oracle.chamfer_forward(a.numpy(), c.numpy())
    check_backward(a, c, gd1, gd2, i1, i2, cuda)


def test_backward_non_finite_input_follows_float_arithmetic(cuda):
    # inf and NaN have no fixed-point image: a workgroup that meets one sums in floating
    # point and must give what float addition gives
    g = gen(4)
    a, c = uniform_cloud(g, 2, 2000), uniform_cloud(g, 2, 2500)
    gd1, gd2 = torch.randn(2, 2000, generator=g), torch.randn(2, 2500, generator=g)
    _, i1, _, i2 = oracle.chamfer_forward(a.numpy(), c.numpy())
    gd2[0, 100] = float("inf")
    gd2[0, 900] = float("nan")
    gd1[1, 17] = -float("inf")
    c = c.clone()
    c[1, 40, 1] = float("inf")          # a coordinate: its own term and what it sends
    check_backward(a, c, gd1, gd2, i1, i2, cuda, exact_nonfinite=True)


def test_gradcheck_fp64(cuda):
    # as the reference does (tests/ops/test_chamfer_distance.py:72-81,101-113)
    from torkit3d_amd.ops.chamfer_distance import chamfer_distance

    # Finite differences are only valid away from a change of nearest neighbour: the
    # seed is chosen so that first and second neighbour are never closer than 1e-4
    # (with seed 6, for example, two candidates are 7e-8 apart and gradcheck fails
    # on the numerical side).
    g = gen(18)
    a = torch.rand(2, 64, 3, generator=g, dtype=torch.float64)
    c = torch.rand(2, 64, 3, generator=g, dtype=torch.float64)
    D = ((a[:, :, None, :] - c[:, None, :, :]) ** 2).sum(-1)
    for dim in (1, 2):
        two = D.sort(dim=dim).values.narrow(dim, 0, 2)
        assert float((two.select(dim, 1) - two.select(dim, 0)).min()) > 1e-4
    a, c = a.to(cuda).requires_grad_(), c.to(cuda).requires_grad_()
    assert torch.autograd.gradcheck(chamfer_distance, (a, c, False))
    at = a.detach().transpose(1, 2).contiguous().requires_grad_()
    ct = c.detach().transpose(1, 2).contiguous().requires_grad_()
    assert torch.autograd.gradcheck(chamfer_distance, (at, ct, True))


def test_sqrt_option(cuda):
    from torkit3d_amd.ops.chamfer_distance import chamfer_distance

    g = gen(7)
    a, c = uniform_cloud(g, 2, 100).to(cuda), uniform_cloud(g, 2, 90).to(cuda)
    d1, d2 = chamfer_distance(a, c)
    s1, s2 = chamfer_distance(a, c, sqrt=True)
    assert torch.equal(s1, torch.sqrt(torch.clamp(d1, 1e-12)))
    assert torch.equal(s2, torch.sqrt(torch.clamp(d2, 1e-12)))


# ---- inputs chosen against the pre-filtered fp32 kernel ------------------------------
# Large fp32 clouds go through a kernel that rules pairs out with a cheaper score and
# re-evaluates only candidate tiles exactly. Whatever the input, the result must be
# bit-identical to the oracle: these cases aim at its error bound, its candidate
# bookkeeping and its fallbacks.

def _clouds(kind, g, b=2, n1=1500, n2=3001):
    if kind == "lattice":            # exact ties everywhere: many candidate tiles
        return lattice_cloud(g, b, max(n1, 2048), 4), lattice_cloud(g, b, max(n1, 2048), 4)
    if kind == "coarse_lattice":     # 27 distinct positions: every tile ties
        return lattice_cloud(g, b, n1 - 400, 2), lattice_cloud(g, b, n1 - 200, 2)
    if kind == "duplicates":
        return uniform_cloud(g, b, n1), uniform_cloud(g, b, 1).expand(b, n2, 3).contiguous()
    if kind == "far_from_origin":    # magnitude >> spacing: the bound is loose
        return uniform_cloud(g, b, n1) + 1000.0, uniform_cloud(g, b, n2) + 1000.0
    if kind == "separated":          # queries far from every key
        return uniform_cloud(g, b, n1) + 50.0, uniform_cloud(g, b, n2)
    if kind == "wide_range":
        return (uniform_cloud(g, b, n1) * 1e6, uniform_cloud(g, b, n2) * 1e6)
    if kind == "tiny":               # squares underflow
        return uniform_cloud(g, b, n1) * 1e-20, uniform_cloud(g, b, n2) * 1e-20
    if kind == "huge":               # squares overflow the bound's range
        return uniform_cloud(g, b, n1) * 1e18, uniform_cloud(g, b, n2) * 1e18
    if kind == "overflowing":        # distances overflow to +inf
        return uniform_cloud(g, b, n1) * 3e19, -uniform_cloud(g, b, n2).abs() * 3e19
    if kind == "clusters":           # tight clusters far apart
        centres = uniform_cloud(g, b, 8) * 100.0
        def mk(n):
            pick = torch.randint(0, 8, (b, n), generator=g)
            base = torch.gather(centres, 1, pick[:, :, None].expand(-1, -1, 3))
            return base + 1e-3 * uniform_cloud(g, b, n)
        return mk(n1), mk(n2)
    if kind == "nan_and_inf":
        a, c = uniform_cloud(g, b, n1), uniform_cloud(g, b, n2)
        c[0, ::7, 1] = float("nan")
        c[1, 5, 0] = float("inf")
        a[0, 3, 2] = float("nan")
        a[1, ::50] = float("inf")
        return a, c
    if kind == "all_nan_keys":
        return uniform_cloud(g, b, n1), torch.full((b, n2, 3), float("nan"))
    if kind == "scaled_small":       # inside the range the matrix pre-filter rescales
        return uniform_cloud(g, b, n1) * 1e-9, uniform_cloud(g, b, n2) * 1e-9
    if kind == "scaled_large":
        return uniform_cloud(g, b, n1) * 3e9 + 1e9, uniform_cloud(g, b, n2) * 3e9 + 1e9
    if kind == "outliers_off_sample":
        # The matrix pre-filter places its centre and scale from every (n/1024)-th key;
        # keys at positions the sample skips lie far outside what it saw: a few within
        # the range of the 16-bit pieces, in batch 1 one beyond it.
        a, c = uniform_cloud(g, b, n1), uniform_cloud(g, b, n2)
        for cloud in (a, c):
            n = cloud.shape[1]
            seen = set((i * n) // 1024 for i in range(1024))
            skipped = [j for j in range(n) if j not in seen]
            if n <= 1024:            # every point is in the sample
                continue
            assert len(skipped) >= 3
            cloud[:, skipped[0]] = torch.tensor([40.0, -3.0, 0.5])
            cloud[:, skipped[len(skipped) // 2]] *= 100.0
            cloud[1::2, skipped[-1], 1] = 3.0e4
        return a, c
    if kind == "far_queries":        # some queries beyond the range of the 16-bit pieces
        a, c = uniform_cloud(g, b, n1), uniform_cloud(g, b, n2)
        a[:, ::97] *= 1.0e5
        a[:, 5::211, 2] += 2.0e4
        c[:, 7::301] += 7.0e6
        return a, c
    raise ValueError(kind)


HARD_KINDS = ["lattice", "coarse_lattice", "duplicates", "far_from_origin", "separated",
              "wide_range", "tiny", "huge", "overflowing", "clusters", "nan_and_inf",
              "all_nan_keys", "scaled_small", "scaled_large", "outliers_off_sample",
              "far_queries"]


@pytest.mark.parametrize("kind", HARD_KINDS)
def test_prefiltered_kernel_is_exact_on_hard_inputs(cuda, kind):
    a, c = _clouds(kind, gen(sum(map(ord, kind))))
    check_forward(a.contiguous(), c.contiguous(), cuda)


# Launches of 512 workgroups or more on clouds of 2048 points or more run the pre-filter
# on the matrix cores (scores from two-piece fp16 splits of the centred, rescaled
# coordinates): the same inputs again at a batch size and cloud lengths that reach it.
@pytest.mark.parametrize("kind", HARD_KINDS)
def test_matrix_prefilter_with_a_short_cloud_on_hard_inputs(cuda, kind):
    # one cloud of a few hundred points against one of a few thousand: the long cloud is cut
    # into key slices for the short cloud's queries, the short one fills half a stage
    b, n1, n2 = 40, 2900, 200
    a, c = _clouds(kind, gen(sum(map(ord, kind)) + 2), b, n1, n2)
    if kind in ("lattice", "coarse_lattice"):
        c = c[:, :n2].contiguous()
    assert b * ((a.shape[1] + 511) // 512 + (c.shape[1] + 511) // 512) >= 96 and a.shape[1] >= 1024
    check_forward(a.contiguous(), c.contiguous(), cuda)


@pytest.mark.parametrize("b", [48, 72])  # two and four query blocks per wave
@pytest.mark.parametrize("kind", HARD_KINDS)
def test_matrix_prefilter_is_exact_on_hard_inputs(cuda, kind, b):
    n1, n2 = 2500, 3001
    assert min(n1 - 400, n2) >= 2048 and b * ((n1 - 400 + 511) // 512 + (n2 + 511) // 512) >= 512
    assert (b * ((n1 + 511) // 512 + (n2 + 511) // 512) <= 640) == (b == 48)
    a, c = _clouds(kind, gen(sum(map(ord, kind)) + 1), b, n1, n2)
    check_forward(a.contiguous(), c.contiguous(), cuda)


@pytest.mark.parametrize("b,n1,n2", [(1, 1024, 1024), (2, 1025, 4097), (3, 8191, 1031),
                                     (1, 20000, 1024), (64, 1024, 1100),
                                     (64, 2049, 4100), (20, 6000, 7777), (512, 2048, 2048)])
def test_prefiltered_kernel_shapes(cuda, b, n1, n2):
    g = gen(n1 + n2)
    check_forward(sphere_cloud(g, b, n1), sphere_cloud(g, b, n2), cuda)


# ---- split sweeps ----------------------------------------------------------------------
# When a launch would leave most of the chip idle, each query's sweep is cut into key
# slices handled by different workgroups, and the partial results meet in a packed
# 64-bit minimum. The merged result must still be the reference's: smallest distance,
# lowest key index among equals, (inf, -1) without a finite distance.

@pytest.mark.parametrize("b,n1,n2", [(1, 4096, 4096), (2, 3000, 5000), (1, 20000, 700),
                                     (1, 777, 65536 + 5), (4, 512, 512), (1, 16384, 16384),
                                     (1, 8192, 8192), (2, 16384, 9000), (1, 2048, 65536 + 5),
                                     # clouds of very different lengths: each direction gets
                                     # its own number of key slices
                                     (1, 20000, 2048), (2, 1500, 70000), (3, 100000, 1024),
                                     (32, 8192, 1024), (1, 1024, 300000),
                                     # ... down to key clouds of a few points on one side
                                     (1, 200000, 512), (1, 100000, 100), (8, 16384, 256),
                                     (16, 4096, 5), (2, 50000, 1), (3, 70000, 33)])
def test_split_sweep_shapes(cuda, b, n1, n2):
    g = gen(n1 * 3 + n2)
    check_forward(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), cuda)


@pytest.mark.parametrize("n1,n2,spots", [
    (2048, 8192, (100, 101, 3000, 3001, 8000, 8191)),        # vector pre-filter, sliced
    (4096, 16384, (100, 101, 7000, 7001, 16000, 16383))])    # matrix pre-filter, sliced
def test_split_sweep_ties_across_slices_keep_the_lowest_index(cuda, n1, n2, spots):
    from torkit3d_amd import _C

    g = gen(77)
    a, c = uniform_cloud(g, 1, n1), uniform_cloud(g, 1, n2) + 5.0
    # The same three points sit in the first, a middle and the last part of the key cloud.
    for j in spots:
        c[0, j] = torch.tensor([0.25, -0.5, 0.125]) if j % 2 == 0 else torch.tensor([-0.5, 0.5, 0.75])
    c[0, 4000] = c[0, 100]
    check_forward(a, c, cuda)
    _, i1, _, i2 = _C.chamfer_distance_forward_cuda(a.to(cuda), c.to(cuda))
    assert set(i1.unique().tolist()) <= {100, 101}
    # The batch replicated until the launch no longer splits must give the same rows.
    many = _C.chamfer_distance_forward_cuda(a.expand(96, -1, -1).contiguous().to(cuda),
                                            c.expand(96, -1, -1).contiguous().to(cuda))
    one = _C.chamfer_distance_forward_cuda(a.to(cuda), c.to(cuda))
    for m, o in zip(many, one):
        assert torch.equal(m[0], o[0]) and torch.equal(m[95], o[0])


@pytest.mark.parametrize("n1,n2", [(1500, 6000),       # vector pre-filter, sliced
                                   (4096, 16384),      # matrix pre-filter, sliced
                                   (1024, 60000)])     # one direction in 59 slices, the other whole
def test_split_sweep_with_slices_that_hold_no_finite_distance(cuda, n1, n2):
    g = gen(78)
    a, c = uniform_cloud(g, 2, n1), uniform_cloud(g, 2, n2)
    c[0, :n2 * 5 // 12] = float("nan")          # leading slices without a candidate
    c[0, n2 * 5 // 6:, 1] = float("inf")        # trailing slices at infinite distance
    c[1] = float("nan")                 # a cloud without any candidate: (inf, -1) everywhere
    a[0, 7] = float("nan")
    check_forward(a, c, cuda)


# ---- channel-first clouds, read in place ---------------------------------------------------

def check_forward_channels_first(a, c, cuda):
    """nn_distance(transpose=True) on [B,3,N] device tensors against the oracle on [B,N,3]."""
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    a_bcn = a.to(cuda).transpose(1, 2).contiguous()
    c_bcn = c.to(cuda).transpose(1, 2).contiguous()
    out = nn_distance(a_bcn, c_bcn, transpose=True)
    want = oracle.chamfer_forward(a.contiguous().numpy(), c.contiguous().numpy())
    for name, got, exp in zip(("dist1", "idx1", "dist2", "idx2"), out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp, err_msg=name)


@pytest.mark.parametrize("b,n1,n2", [(2, 1024, 1024), (3, 2043, 1999), (1, 1, 1), (2, 5000, 33),
                                     (2, 33, 5000), (4, 255, 257), (2, 4096, 4100),
                                     (8, 8192, 8192),     # the sorted path, [3,N] read in place
                                     (5, 16384, 6000),    # sorted path, four parts per cloud
                                     (1, 20000, 3001),    # beyond the sorted path's [3,N] reach
                                     (40, 1500, 1100)])
def test_forward_channels_first(cuda, b, n1, n2):
    # reference: chamfer_distance / nn_distance with transpose=True
    # (torkit3d/ops/chamfer_distance.py:52-55,68-70; tests/ops/test_chamfer_distance.py:86-99)
    g = gen(31)
    check_forward_channels_first(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), cuda)
    check_forward_channels_first(sphere_cloud(g, b, n1), sphere_cloud(g, b, n2), cuda)


@pytest.mark.parametrize("kind", HARD_KINDS)
def test_channels_first_on_hard_inputs(cuda, kind):
    a, c = _clouds(kind, gen(sum(map(ord, kind)) + 9), 2, 2500, 3001)
    check_forward_channels_first(a, c, cuda)
    a, c = _clouds(kind, gen(sum(map(ord, kind)) + 10), 3, 5000, 6001)   # sorted path sizes
    check_forward_channels_first(a, c, cuda)


def test_channels_first_fp64_and_gradients(cuda):
    from torkit3d_amd.ops.chamfer_distance import chamfer_distance, nn_distance

    g = gen(33)
    a = torch.rand(3, 3, 700, generator=g, dtype=torch.float64)
    c = torch.rand(3, 3, 900, generator=g, dtype=torch.float64)
    out = nn_distance(a.to(cuda), c.to(cuda), transpose=True)
    want = oracle.chamfer_forward(a.transpose(1, 2).contiguous().numpy(),
                                  c.transpose(1, 2).contiguous().numpy())
    for got, exp in zip(out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp)
    # gradients of the channel-first call equal those of the [B,N,3] call, transposed
    for dtype in (torch.float32, torch.float64):
        x1 = a.to(dtype).to(cuda).requires_grad_()
        x2 = c.to(dtype).to(cuda).requires_grad_()
        d1, d2 = chamfer_distance(x1, x2, transpose=True)
        (d1.sum() + 2 * d2.sum()).backward()
        y1 = a.to(dtype).transpose(1, 2).contiguous().to(cuda).requires_grad_()
        y2 = c.to(dtype).transpose(1, 2).contiguous().to(cuda).requires_grad_()
        e1, e2 = chamfer_distance(y1, y2)
        (e1.sum() + 2 * e2.sum()).backward()
        assert torch.equal(d1, e1) and torch.equal(d2, e2)
        assert torch.equal(x1.grad, y1.grad.transpose(1, 2))
        assert torch.equal(x2.grad, y2.grad.transpose(1, 2))
