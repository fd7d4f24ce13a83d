"""Pins the CPU oracle for group points and feature interpolation against the
golden vectors, torch.gather / index_add_ and autograd."""
import numpy as np
import pytest
import torch

import oracle


def gen(seed):
    return torch.Generator().manual_seed(seed)


def test_group_and_interpolate_golden(golden):
    g = golden
    np.testing.assert_array_equal(oracle.group_forward(g["group_input"], g["group_index"]),
                                  g["group_output"])
    np.testing.assert_array_equal(
        oracle.group_backward(g["group_grad_output"], g["group_index"], 11), g["group_grad_input"])
    np.testing.assert_array_equal(
        oracle.interpolate_forward(g["interp_input"], g["interp_index"], g["interp_weight"]),
        g["interp_output"])
    np.testing.assert_array_equal(
        oracle.interpolate_backward(g["interp_grad_output"], g["interp_index"],
                                    g["interp_weight"], 11), g["interp_grad_input"])


@pytest.mark.parametrize("b,c,n1,n2,k", [(2, 3, 512, 128, 32), (5, 64, 513, 129, 33)])
def test_group_matches_torch_gather(b, c, n1, n2, k):
    # The reference's oracle: torch.gather on expanded views
    # (tests/ops/test_group_points.py:6-12), forward exact, backward with ones upstream.
    g = gen(0)
    feat = torch.randn(b, c, n1, generator=g, requires_grad=True)
    index = torch.randint(0, n1, (b, n2, k), generator=g)
    want = feat.unsqueeze(2).expand(b, c, n2, n1).gather(3, index.unsqueeze(1).expand(b, c, n2, k))
    got = oracle.group_forward(feat.detach().numpy(), index.numpy())
    np.testing.assert_array_equal(got, want.detach().numpy())
    want.backward(torch.ones_like(want))
    gin = oracle.group_backward(np.ones((b, c, n2, k), np.float32), index.numpy(), n1)
    np.testing.assert_array_equal(gin, feat.grad.numpy())
    # ones upstream = occurrence counts
    counts = np.stack([np.bincount(i.reshape(-1), minlength=n1) for i in index.numpy()])
    np.testing.assert_array_equal(gin, np.broadcast_to(counts[:, None, :], gin.shape))


def test_group_backward_matches_index_add_fp64():
    g = gen(1)
    b, c, n1, n2, k = 3, 7, 50, 40, 9
    go = torch.randn(b, c, n2, k, generator=g, dtype=torch.float64)
    index = torch.randint(0, n1, (b, n2, k), generator=g)
    want = torch.zeros(b, c, n1, dtype=torch.float64)
    for bi in range(b):
        want[bi].index_add_(1, index[bi].reshape(-1), go[bi].reshape(c, -1))
    got = oracle.group_backward(go.numpy(), index.numpy(), n1)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("b,c,n1,n2", [(2, 64, 128, 512), (3, 65, 129, 513)])
def test_interpolate_matches_gather_weight_sum_fp64(b, c, n1, n2):
    # The reference's oracle: gather * weight, summed over the 3 neighbours, fp64
    # (tests/ops/test_interpolate_feature.py:15-22, :38-67).
    g = gen(0)
    feat = torch.randn(b, c, n1, generator=g, dtype=torch.float64, requires_grad=True)
    index = torch.randint(0, n1, (b, n2, 3), generator=g)
    weight = torch.rand(b, n2, 3, generator=g, dtype=torch.float64)
    weight = weight / weight.sum(2, keepdim=True)
    grouped = feat.unsqueeze(2).expand(b, c, n2, n1).gather(3, index.unsqueeze(1).expand(b, c, n2, 3))
    want = (grouped * weight.unsqueeze(1)).sum(-1)
    got = oracle.interpolate_forward(feat.detach().numpy(), index.numpy(), weight.numpy())
    np.testing.assert_allclose(got, want.detach().numpy(), rtol=1e-13, atol=1e-14)
    go = torch.randn(b, c, n2, generator=g, dtype=torch.float64)
    want.backward(go)
    gin = oracle.interpolate_backward(go.numpy(), index.numpy(), weight.numpy(), n1)
    np.testing.assert_allclose(gin, feat.grad.numpy(), rtol=1e-12, atol=1e-13)


def test_interpolate_one_hot_weights_reduce_to_gather():
    g = gen(2)
    feat = torch.randn(2, 5, 30, generator=g).numpy()
    index = torch.randint(0, 30, (2, 17, 3), generator=g).numpy()
    weight = np.zeros((2, 17, 3), np.float32)
    weight[:, :, 1] = 1
    got = oracle.interpolate_forward(feat, index, weight)
    want = np.stack([feat[b][:, index[b, :, 1]] for b in range(2)])
    np.testing.assert_array_equal(got, want)


def test_three_nn_weights_recipe():
    # layers/pointnet2.py:128-130: inverse squared distance, clamped at 1e-10, normalised.
    d2 = np.array([[[0.0, 1.0, 4.0], [2.0, 2.0, 2.0]]], np.float32)
    w = oracle.three_nn_weights(d2)
    assert w.dtype == np.float32
    np.testing.assert_allclose(w.sum(2), 1.0, rtol=1e-6)
    np.testing.assert_allclose(w[0, 1], [1 / 3] * 3, rtol=1e-6)
    assert w[0, 0, 0] > 0.999999  # a coincident neighbour takes all the weight
    inv = 1.0 / torch.clamp(torch.from_numpy(d2), min=1e-10)
    np.testing.assert_array_equal(w, (inv / inv.sum(2, keepdim=True)).numpy())


def test_out_of_range_indices_are_counted_not_read():
    feat = np.arange(12, dtype=np.float32).reshape(1, 2, 6)
    index = np.array([[[0, 6, -1, 5]]], np.int64)
    out = oracle.group_forward(feat, index)
    np.testing.assert_array_equal(out[0, :, 0], [[0, 0, 0, 5], [6, 0, 0, 11]])


def test_wide_backward_variants_sum_in_double():
    # fp32 terms summed in float64 by numpy and rounded once; duplicate-heavy indices
    g = gen(9)
    b, c, n1, n2, k = 2, 5, 37, 300, 6
    index = torch.randint(0, n1, (b, n2, k), generator=g).numpy()
    index[:, :, 3:] = index[:, :, :1]       # padded rows: the first hit repeated
    index[0, 4, 2] = -1                      # skipped
    go = torch.randn(b, c, n2, k, generator=g).numpy()
    want = np.zeros((b, c, n1))
    for bi in range(b):
        flat = index[bi].reshape(-1)
        ok = flat >= 0
        for ch in range(c):
            np.add.at(want[bi, ch], flat[ok], go[bi, ch].reshape(-1)[ok].astype(np.float64))
    got = oracle.group_backward(go, index, n1, wide=True)
    np.testing.assert_array_equal(got, want.astype(np.float32))
    seq = oracle.group_backward(go, index, n1)
    np.testing.assert_allclose(got, seq, rtol=1e-4, atol=1e-4)
    assert not np.array_equal(got, seq)

    index3 = torch.randint(0, n1, (b, n2, 3), generator=g).numpy()
    weight = torch.rand(b, n2, 3, generator=g).numpy()
    go3 = torch.randn(b, c, n2, generator=g).numpy()
    want = np.zeros((b, c, n1))
    for bi in range(b):
        for ch in range(c):
            term = go3[bi, ch][:, None] * weight[bi]        # fp32 products
            assert term.dtype == np.float32
            np.add.at(want[bi, ch], index3[bi].reshape(-1), term.reshape(-1).astype(np.float64))
    got = oracle.interpolate_backward(go3, index3, weight, n1, wide=True)
    np.testing.assert_array_equal(got, want.astype(np.float32))
