"""Seeded differential runs of the kernels that rule pairs out before they evaluate them -
chamfer forward on sorted clouds (pruning by tile boxes + matrix-core scores), the chamfer
matrix and vector pre-filters, and the KNN pre-filter - against the CPU oracle, each kernel
forced through the test-only entry points whatever the dispatcher would pick for the shape.

The two clouds of a case are drawn independently from: uniform, lattice (exact ties), sphere,
Gaussian mixture, scaled by 1e-8..1e8, offset, on a line, points within a few units in the
last place of each other at |x| of 1e2..1e3, and clouds where all but a few points are one
and the same; then, with some probability, scaled by 10^+-8, offset by up to 1e4, or moved
onto the other cloud's region. Sizes run from 1 to 65536 points. Every distance and index
must equal the oracle's bit for bit (lowest index among equal distances:
torkit3d/csrc/cuda/chamfer_distance_kernel.cu:60-78; MinK's slot order:
torkit3d/csrc/include/mink.cuh:61-89). A run stops at its first difference and names the
case."""
import math

import numpy as np
import pytest
import torch

import oracle
from debug_abi import (ROUTE_MATRIX2, ROUTE_MATRIX4, ROUTE_MATRIX_SLICED, ROUTE_VECTOR,
                       chamfer_route, chamfer_sorted, knn_filter)
from test_gpu_random_shapes import _cloud as _plain_cloud

pytestmark = pytest.mark.gpu
NAMES = ("dist1", "idx1", "dist2", "idx2")


def _near_identical(rng, g, b, n):
    """Points within 0..4 units in the last place of one point at |x| of 1e2..1e3 per axis,
    a random share of them exactly that point."""
    centre = torch.tensor([float(rng.uniform(100.0, 1000.0)) * (1 if rng.random() < 0.5 else -1)
                           for _ in range(3)], dtype=torch.float32)
    bits = centre.view(torch.int32)[None, None, :].repeat(b, n, 1)
    nudge = torch.randint(-4, 5, (b, n, 3), generator=g, dtype=torch.int32)
    same = torch.rand(b, n, 1, generator=g) < float(rng.choice([0.0, 0.5, 0.9]))
    nudge = torch.where(same, torch.zeros_like(nudge), nudge)
    return (bits + nudge).view(torch.float32).contiguous()


def _mostly_identical(rng, g, b, n):
    """One point repeated, except for m points spread around it at a random scale."""
    base = (torch.rand(b, 1, 3, generator=g) * 2 - 1) * float(10.0 ** rng.uniform(-1, 3))
    x = base.repeat(1, n, 1)
    m = int(min(n, rng.integers(0, 41)))
    if m:
        where = torch.randperm(n, generator=g)[:m]
        spread = float(10.0 ** rng.uniform(-6, 1))
        x[:, where] = base + spread * (torch.rand(b, m, 3, generator=g) * 2 - 1)
    return x.contiguous()


def draw_cloud(rng, g, b, n):
    pick = rng.random()
    if pick < 0.12:
        x = _near_identical(rng, g, b, n)
    elif pick < 0.24:
        x = _mostly_identical(rng, g, b, n)
    else:
        x = _plain_cloud(rng, g, b, n)
    if rng.random() < 0.25:
        x = x * float(10.0 ** rng.uniform(-8, 8))
    if rng.random() < 0.25:
        x = x + torch.tensor([float(rng.uniform(-1, 1) * 10.0 ** rng.uniform(-2, 4))
                              for _ in range(3)], dtype=torch.float32)
    return x.float().contiguous()


def draw_pair(rng, g, b, n1, n2):
    a, c = draw_cloud(rng, g, b, n1), draw_cloud(rng, g, b, n2)
    if rng.random() < 0.3:  # the second cloud moved onto the first one's region
        c = (c - c.mean(dim=1, keepdim=True) + a.mean(dim=1, keepdim=True)).contiguous()
    return a, c


def log_size(rng, lo, hi):
    return int(min(hi, max(lo, round(2.0 ** rng.uniform(math.log2(lo), math.log2(hi))))))


def first_difference(out, want):
    for name, got, exp in zip(NAMES, out, want):
        got = got.cpu().numpy()
        same = np.array_equal(got.view(np.int32), exp.view(np.int32)) if exp.dtype == np.float32 \
            else np.array_equal(got, exp)
        if not same:
            at = np.argwhere(got.view(np.int64 if exp.dtype == np.int64 else np.int32)
                             != exp.view(np.int64 if exp.dtype == np.int64 else np.int32))[0]
            return "%s at %s: got %r, want %r" % (name, at.tolist(), got[tuple(at)], exp[tuple(at)])
    return None


def chamfer_cases(seed, count, lo, hi, need_long=0):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    done = 0
    while done < count:
        b = int(rng.choice([1, 1, 2, 3, 5]))
        n1, n2 = log_size(rng, lo, hi), log_size(rng, lo, hi)
        if max(n1, n2) < need_long:
            continue
        if b * n1 * n2 > 4e8:
            b = 1
        a, c = draw_pair(rng, g, b, n1, n2)
        done += 1
        yield (seed, done, b, n1, n2), a, c


@pytest.mark.parametrize("seed", [31, 32, 33, 34])
def test_chamfer_sorted_path(cuda, seed):
    # forced through the workspace entry point with the `always` size; 100 cases per seed,
    # about a third of them with a cloud that the path hands to the sweep of all pairs
    handed = 0
    for case, a, c in chamfer_cases(seed, 100, 1, 65536):
        out, ws, _ = chamfer_sorted(a.to(cuda), c.to(cuda))
        b = case[2]
        at = (2 * b * 64 + 255) // 256 * 256
        handed += int(ws[at:at + 2 * b * 4].view(torch.int32).sum().item() > 0)
        diff = first_difference(out, oracle.chamfer_forward(a.numpy(), c.numpy()))
        assert diff is None, (case, diff)
    assert handed < 100  # (some cases must stay on the sorted path for the run to mean anything)


@pytest.mark.parametrize("seed,route", [(41, ROUTE_MATRIX4), (42, ROUTE_MATRIX2),
                                        (43, ROUTE_MATRIX_SLICED), (44, ROUTE_MATRIX4)])
def test_chamfer_matrix_prefilter(cuda, seed, route):
    for case, a, c in chamfer_cases(seed, 60, 1, 40000, need_long=1024):
        out = chamfer_route(a.to(cuda), c.to(cuda), route)
        assert out is not None, case
        diff = first_difference(out, oracle.chamfer_forward(a.numpy(), c.numpy()))
        assert diff is None, (case, route, diff)


@pytest.mark.parametrize("seed", [51, 52])
def test_chamfer_vector_prefilter(cuda, seed):
    for case, a, c in chamfer_cases(seed, 50, 512, 20000):
        out = chamfer_route(a.to(cuda), c.to(cuda), ROUTE_VECTOR)
        assert out is not None, case
        diff = first_difference(out, oracle.chamfer_forward(a.numpy(), c.numpy()))
        assert diff is None, (case, diff)


@pytest.mark.parametrize("seed", [61, 62, 63])
def test_knn_prefilter(cuda, seed):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    for done in range(80):
        b = int(rng.choice([1, 1, 2, 4]))
        n1, n2 = log_size(rng, 1, 20000), log_size(rng, 256, 16384)
        k = int(rng.integers(1, 17))
        if b * n1 * n2 > 2e8:
            b = 1
        q, key = draw_pair(rng, g, b, n1, n2)
        got = knn_filter(q.to(cuda), key.to(cuda), k)
        assert got is not None
        od, oi = oracle.knn(q.numpy(), key.numpy(), k)
        case = (seed, done, b, n1, n2, k)
        gd = got[0].cpu().numpy()
        # (NaN distances of non-finite input compare by bit pattern)
        assert np.array_equal(gd.view(np.int32), od.view(np.int32)), case
        assert np.array_equal(got[1].cpu().numpy(), oi), case
