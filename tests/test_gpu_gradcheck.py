"""Numerical differentiation (torch.autograd.gradcheck, fp64) of every differentiable
function of the package: an oracle-free check that each backward kernel is the
derivative of its forward kernel."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def leaf(*shape, seed=0, device="cuda:0"):
    return torch.randn(*shape, generator=gen(seed), dtype=torch.float64).to(device).requires_grad_()


def test_group_points(cuda):
    from torkit3d_amd.ops.group_points import group_points

    feat = leaf(2, 5, 9, seed=1)
    index = torch.randint(0, 9, (2, 4, 3), generator=gen(2)).to(cuda)
    index[0, 0] = 7  # repeated neighbours accumulate
    assert torch.autograd.gradcheck(group_points, (feat, index))


@pytest.mark.parametrize("with_feature", [True, False])
def test_group_points_with_xyz(cuda, with_feature):
    from torkit3d_amd.ops.group_points import group_points_with_xyz

    feat = leaf(2, 4, 11, seed=3) if with_feature else None
    xyz, centre = leaf(2, 3, 11, seed=4), leaf(2, 3, 5, seed=5)
    index = torch.randint(0, 11, (2, 5, 6), generator=gen(6)).to(cuda)
    assert torch.autograd.gradcheck(
        lambda f, x, c: group_points_with_xyz(f, x, c, index), (feat, xyz, centre))


def test_interpolate_feature(cuda):
    from torkit3d_amd.ops.interpolate_feature import interpolate_feature

    feat = leaf(2, 6, 7, seed=7)
    index = torch.randint(0, 7, (2, 10, 3), generator=gen(8)).to(cuda)
    weight = torch.rand(2, 10, 3, generator=gen(9), dtype=torch.float64).to(cuda)
    assert torch.autograd.gradcheck(lambda f: interpolate_feature(f, index, weight), (feat,))


def test_edge_features_agree_with_the_gather_form(cuda):
    from torkit3d_amd.ops.edge_conv import get_edge_feature_builtin, get_edge_feature_custom

    q, k = leaf(2, 3, 6, seed=10), leaf(2, 3, 8, seed=11)
    index = torch.randint(0, 8, (2, 6, 4), generator=gen(12)).to(cuda)
    for include_query in (True, False):
        assert torch.equal(get_edge_feature_custom(q, k, index, include_query),
                           get_edge_feature_builtin(q, k, index, include_query))
        assert torch.autograd.gradcheck(
            lambda a, b: get_edge_feature_custom(a, b, index, include_query), (q, k))


def test_feature_propagation_layer(cuda):
    """Interpolation inside the layer: gradient to the coarse features only (index and
    weight come from a no_grad block, as in the reference)."""
    from torkit3d_amd.layers.pointnet2 import FeatureInterpolator

    fine = (torch.rand(2, 3, 12, generator=gen(13), dtype=torch.float64) * 2 - 1).to(cuda)
    coarse = (torch.rand(2, 3, 5, generator=gen(14), dtype=torch.float64) * 2 - 1).to(cuda)
    feat = leaf(2, 4, 5, seed=15)
    layer = FeatureInterpolator()
    assert torch.autograd.gradcheck(lambda f: layer(fine, coarse, f), (feat,))
