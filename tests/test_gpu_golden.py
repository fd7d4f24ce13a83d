"""Every op, through the ``_C`` shim and the C ABI, on the committed golden vectors:
outputs must be bit-identical (backward passes: within rounding of a different
summation order)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def host(t):
    return t.cpu().numpy()


@pytest.mark.parametrize("case", ["rand", "lat", "known"])
def test_chamfer_forward(golden, cuda, case):
    from torkit3d_amd import _C

    out = _C.chamfer_distance_forward_cuda(dev(golden[f"chamfer_{case}_xyz1"], cuda),
                                           dev(golden[f"chamfer_{case}_xyz2"], cuda))
    for name, got in zip(("dist1", "idx1", "dist2", "idx2"), out):
        np.testing.assert_array_equal(host(got), golden[f"chamfer_{case}_{name}"], err_msg=name)


def test_chamfer_backward(golden, cuda):
    from torkit3d_amd import _C

    g = golden
    gx1, gx2 = _C.chamfer_distance_backward_cuda(
        dev(g["chamfer_rand_gd1"], cuda), dev(g["chamfer_rand_gd2"], cuda),
        dev(g["chamfer_rand_xyz1"], cuda), dev(g["chamfer_rand_xyz2"], cuda),
        dev(g["chamfer_rand_idx1"], cuda), dev(g["chamfer_rand_idx2"], cuda))
    np.testing.assert_allclose(host(gx1), g["chamfer_rand_gx1"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(host(gx2), g["chamfer_rand_gx2"], rtol=1e-5, atol=1e-6)


def test_knn(golden, cuda):
    from torkit3d_amd import _C

    for version in (0, 1):
        for k in (3, 5):
            d, i = _C.knn_distance_cuda(dev(golden["knn_rand_query"], cuda),
                                        dev(golden["knn_rand_key"], cuda), k, version)
            np.testing.assert_array_equal(host(d), golden[f"knn_rand_k{k}_dist"])
            np.testing.assert_array_equal(host(i), golden[f"knn_rand_k{k}_idx"])
    d, i = _C.knn_distance_cuda(dev(golden["knn_lat_query"], cuda),
                                dev(golden["knn_lat_key"], cuda), 4, 1)
    np.testing.assert_array_equal(host(d), golden["knn_lat_k4_dist"])
    np.testing.assert_array_equal(host(i), golden["knn_lat_k4_idx"])


def test_ball_query(golden, cuda):
    from torkit3d_amd import _C

    r = float(golden["ball_radius"])
    for k in (8, 3):
        got = _C.ball_query_cuda(dev(golden["ball_query"], cuda), dev(golden["ball_key"], cuda), r, k)
        np.testing.assert_array_equal(host(got), golden[f"ball_idx_k{k}"])
    got = _C.ball_query_cuda(dev(golden["ball_lat_query"], cuda), dev(golden["ball_lat_key"], cuda),
                             float(golden["ball_lat_radius"]), 6)
    np.testing.assert_array_equal(host(got), golden["ball_lat_idx_k6"])


@pytest.mark.parametrize("case,k", [("rand", 20), ("lat", 40), ("dup", 12)])
def test_fps(golden, cuda, case, k):
    from torkit3d_amd import _C

    got = _C.sample_farthest_points_cuda(dev(golden[f"fps_{case}_points"], cuda), k)
    np.testing.assert_array_equal(host(got), golden[f"fps_{case}_idx"])


def test_group_and_interpolate(golden, cuda):
    from torkit3d_amd import _C

    g = golden
    out = _C.group_points_forward_cuda(dev(g["group_input"], cuda), dev(g["group_index"], cuda))
    np.testing.assert_array_equal(host(out), g["group_output"])
    gin = _C.group_points_backward_cuda(dev(g["group_grad_output"], cuda),
                                        dev(g["group_index"], cuda), 11)
    np.testing.assert_allclose(host(gin), g["group_grad_input"], rtol=1e-5, atol=1e-6)
    out = _C.interpolate_forward_cuda(dev(g["interp_input"], cuda), dev(g["interp_index"], cuda),
                                      dev(g["interp_weight"], cuda))
    np.testing.assert_array_equal(host(out), g["interp_output"])
    gin = _C.interpolate_backward_cuda(dev(g["interp_grad_output"], cuda),
                                       dev(g["interp_index"], cuda),
                                       dev(g["interp_weight"], cuda), 11)
    np.testing.assert_allclose(host(gin), g["interp_grad_input"], rtol=1e-5, atol=1e-6)
