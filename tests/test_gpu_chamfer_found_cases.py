"""Inputs on which a chamfer kernel once broke the reference's tie rule, kept as a fixture
(``tests/golden/chamfer_found_cases.npz``; expected outputs from the exact-rational
restatement, see ``tests/golden/make_chamfer_cases.py``) and run through every forward
route: the plain entry point, the sorted path with its workspace, and each named kernel.

"zero_extent_frame": keys within one unit in the last place of each other near coordinate
900, most of them identical. A frame (or sampled extent) of zero left the fp16 terms of the
pre-filters without precision and an equal-distance tie went to key 144 instead of key 0;
the reference keeps the lowest index (strict '<' over ascending j,
torkit3d/csrc/cuda/chamfer_distance_kernel.cu:60-78)."""
import os

import numpy as np
import pytest
import torch

import oracle
from debug_abi import (ROUTE_EXACT, ROUTE_MATRIX2, ROUTE_MATRIX4, ROUTE_MATRIX_SLICED,
                       ROUTE_VECTOR, chamfer_route, chamfer_sorted)

NAMES = ("dist1", "idx1", "dist2", "idx2")
ROUTES = {"exact": ROUTE_EXACT, "vector": ROUTE_VECTOR, "matrix4": ROUTE_MATRIX4,
          "matrix2": ROUTE_MATRIX2, "matrix_sliced": ROUTE_MATRIX_SLICED}


@pytest.fixture(scope="module")
def case():
    here = os.path.dirname(os.path.abspath(__file__))
    g = np.load(os.path.join(here, "golden", "chamfer_found_cases.npz"))
    return {k[len("zero_extent_frame_"):]: g[k] for k in g.files}


def _check(out, want, what):
    for name, got, exp in zip(NAMES, out, want):
        np.testing.assert_array_equal(got.cpu().numpy(), exp, err_msg="%s %s" % (what, name))


def test_fixture_agrees_with_the_oracle(case):  # (runs without a GPU)
    want = oracle.chamfer_forward(case["xyz1"], case["xyz2"])
    for name, w in zip(NAMES, want):
        np.testing.assert_array_equal(w, case[name], err_msg=name)
    # the tie that went wrong: several keys at the minimum distance, the lowest index wanted
    x1, x2 = case["xyz1"].astype(np.float64), case["xyz2"].astype(np.float64)
    d = ((x1[:, :, None] - x2[:, None]) ** 2).sum(-1)
    ties = (d == d.min(-1, keepdims=True)).sum(-1)
    assert ties.max() >= 10


@pytest.mark.gpu
def test_as_found(case, cuda):
    x1 = torch.from_numpy(case["xyz1"]).to(cuda)
    x2 = torch.from_numpy(case["xyz2"]).to(cuda)
    want = [case[n] for n in NAMES]
    from torkit3d_amd.ops.chamfer_distance import nn_distance

    _check(nn_distance(x1, x2), want, "plain entry point")
    _check(chamfer_sorted(x1, x2)[0], want, "sorted path")
    _check(chamfer_route(x1, x2, ROUTE_EXACT), want, "exact sweep")
    # the other way round as well (the near-identical cloud as queries)
    swapped = [case[n] for n in ("dist2", "idx2", "dist1", "idx1")]
    _check(chamfer_sorted(x2, x1)[0], swapped, "sorted path, swapped")


@pytest.mark.gpu
@pytest.mark.parametrize("copies,route", [(5, "matrix4"), (5, "matrix2"), (5, "matrix_sliced"),
                                          (3, "vector"), (5, "vector"), (5, "exact"),
                                          (5, "sorted"), (40, "sorted"), (40, "matrix4"),
                                          (40, "matrix_sliced")])
def test_repeated_to_the_sizes_of_the_other_kernels(case, cuda, copies, route):
    # The key cloud repeated end to end reaches the sizes the pre-filter kernels take (512
    # and 1024 keys). Every added key repeats an earlier one at a higher index, so the
    # nearest key of each query keeps its index; the repeated cloud's own results repeat.
    x1 = torch.from_numpy(case["xyz1"]).to(cuda)
    x2 = torch.from_numpy(np.tile(case["xyz2"], (1, copies, 1))).to(cuda)
    want = [case["dist1"], case["idx1"], np.tile(case["dist2"], (1, copies)),
            np.tile(case["idx2"], (1, copies))]
    out = chamfer_sorted(x1, x2)[0] if route == "sorted" else chamfer_route(x1, x2, ROUTES[route])
    if out is not None:  # (the vector pre-filter wants 512 points in both clouds)
        _check(out, want, route)
    # both clouds long: the near-identical cloud against itself shifted by a few keys
    y1 = torch.roll(x2, 7, dims=1).contiguous()
    want2 = oracle.chamfer_forward(y1.cpu().numpy(), x2.cpu().numpy())
    out2 = chamfer_sorted(y1, x2)[0] if route == "sorted" else chamfer_route(y1, x2, ROUTES[route])
    assert out2 is not None
    _check(out2, want2, route + " (both clouds repeated)")
