"""K nearest neighbours on the GPU: bit-identical (distances, indices, slot order)
to the oracle's MinK restatement; the reference's own checks against cdist/topk."""
import numpy as np
import pytest
import torch

import oracle
from util import lattice_cloud, uniform_cloud

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def check_raw(q, key, k, cuda, version=1):
    from torkit3d_amd import _C

    d, i = _C.knn_distance_cuda(q.to(cuda), key.to(cuda), k, version)
    od, oi = oracle.knn(q.numpy(), key.numpy(), k)
    np.testing.assert_array_equal(d.cpu().numpy(), od)
    np.testing.assert_array_equal(i.cpu().numpy(), oi)


@pytest.mark.parametrize("b,n1,n2,k,transpose", [(1, 512, 1024, 3, True), (2, 512, 1024, 32, False),
                                                  (3, 511, 1025, 31, True),
                                                  (32, 2048, 8192, 64, False)])
def test_reference_cases_fp64(cuda, b, n1, n2, k, transpose):
    # tests/ops/test_knn_distance.py:6-32: fp64 randn, compared with cdist + topk as
    # sqrt distances (atol 5e-5, rtol 1e-4) and exact sorted indices.
    from torkit3d_amd.ops.knn_points import knn_points
    from torkit3d_amd.ops.native import knn

    torch.manual_seed(0)
    q = torch.randn(b, n1, 3, dtype=torch.float64)
    key = torch.randn(b, n2, 3, dtype=torch.float64)
    if transpose:
        q, key = q.transpose(1, 2), key.transpose(1, 2)
    qd, kd = q.to(cuda), key.to(cuda)
    want_d, want_i = knn(qd, kd, k, sorted=True, transpose=transpose)
    got_d, got_i = knn_points(qd, kd, k, sorted=True, sqrt_distance=True, transpose=transpose)
    torch.testing.assert_close(got_d, want_d, atol=5e-5, rtol=1e-4)
    assert torch.equal(got_i, want_i)
    if b <= 3:
        qc = (q.transpose(1, 2) if transpose else q).contiguous()
        kc = (key.transpose(1, 2) if transpose else key).contiguous()
        check_raw(qc, kc, k, cuda)


@pytest.mark.parametrize("k", [16, 3])
def test_interpolation_config_fp32(cuda, k):
    # benchmark config 4: B=32, N=8192 queries, M=2048 keys, uniform in [-1,1]^3
    g = gen(4)
    q, key = uniform_cloud(g, 32, 8192), uniform_cloud(g, 32, 2048)
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("b,n1,n2,k", [(2, 300, 2048, 1), (2, 100, 500, 4), (2, 77, 130, 5),
                                        (2, 100, 500, 8), (1, 200, 3000, 17), (2, 100, 500, 64),
                                        (1, 50, 300, 100), (2, 33, 40, 40), (2, 10, 5, 5),
                                        (1, 1000, 1025, 33), (2, 300, 1000, 65),
                                        (2, 200, 700, 128), (1, 100, 400, 129),
                                        (4, 1000, 4096, 32), (1, 70, 70000, 20),
                                        (1, 40, 66000, 7), (40, 4096, 300, 6),
                                        (2, 150, 1000, 200), (1, 70, 256, 256),
                                        (1, 100, 3000, 257), (1, 64, 66000, 130)])
def test_all_k_variants_and_versions(cuda, b, n1, n2, k):
    g = gen(k)
    q, key = uniform_cloud(g, b, n1), uniform_cloud(g, b, n2)
    check_raw(q, key, k, cuda, version=0)
    check_raw(q, key, k, cuda, version=1)


def test_lattice_ties_follow_mink_eviction_order(cuda):
    g = gen(9)
    q, key = lattice_cloud(g, 2, 400, 4), lattice_cloud(g, 2, 1500, 4)
    for k in (3, 6, 16, 33, 64, 100, 180):
        check_raw(q, key, k, cuda)


@pytest.mark.parametrize("k", [3, 8, 16, 24, 64])
def test_non_finite_keys_follow_mink(cuda, k):
    # MinK compares with '<' and '>' only: a NaN distance taken during the fill is never
    # the maximum unless it sits in slot 0, where it blocks every later insertion; an
    # infinite distance is an ordinary large value.
    g = gen(11)
    q, key = uniform_cloud(g, 4, 200), uniform_cloud(g, 4, 600)
    key[0, 0, 1] = float("nan")        # slot 0 of every query in cloud 0
    key[1, 2, 0] = float("nan")        # a later fill slot
    key[1, 300, 2] = float("nan")      # beyond the fill: never inserted
    key[2, 1, 0] = float("inf")        # infinite distance inside the fill
    key[2, 400, 1] = -float("inf")
    key[3, 0, 0] = float("inf")
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("b,n1,n2,k", [(1, 200, 3000, 17), (2, 100, 500, 64), (2, 200, 700, 128),
                                        (1, 70, 70000, 20), (2, 33, 40, 40), (1, 100, 400, 129)])
def test_fp64_beyond_16_neighbours_keeps_mink_order(cuda, b, n1, n2, k):
    # fp64 with k = 17..128 keeps its slots in LDS as a tournament tree, as fp32 does
    g = gen(k + 1)
    q, key = uniform_cloud(g, b, n1).double(), uniform_cloud(g, b, n2).double()
    check_raw(q, key, k, cuda)
    q, key = lattice_cloud(g, b, n1, 4).double(), lattice_cloud(g, b, n2, 4).double()
    check_raw(q, key, k, cuda)                     # exact ties everywhere
    key = uniform_cloud(g, b, n2).double()
    key[0, 0, 1] = float("nan")                    # slot 0 of the fill: nothing is inserted later
    key[-1, 2, 0] = float("nan")                   # a later fill slot keeps its NaN
    key[-1, n2 // 2, 2] = float("nan")             # beyond the fill: never inserted
    key[0, 1, 0] = float("inf")
    check_raw(q, key, k, cuda)


def test_k1_equals_chamfer_argmin(cuda):
    from torkit3d_amd import _C

    g = gen(10)
    q, key = uniform_cloud(g, 2, 2000).to(cuda), uniform_cloud(g, 2, 1500).to(cuda)
    d, i = _C.knn_distance_cuda(q, key, 1, 1)
    cd, ci, _, _ = _C.chamfer_distance_forward_cuda(q, key)
    assert torch.equal(d[..., 0], cd) and torch.equal(i[..., 0], ci)


def test_errors(cuda):
    from torkit3d_amd import _C

    q = torch.zeros(2, 8, 3, device=cuda)
    with pytest.raises(RuntimeError):
        _C.knn_distance_cuda(q, q, 9, 1)  # k > N2 (knn_distance_kernel.cu:199)
    with pytest.raises(RuntimeError, match="Invalid version"):
        _C.knn_distance_cuda(q, q, 2, 3)
    with pytest.raises(RuntimeError):
        _C.knn_distance_cuda(q, torch.zeros(3, 8, 3, device=cuda), 2, 1)
    with pytest.raises(RuntimeError, match="contiguous"):
        _C.knn_distance_cuda(q.transpose(0, 1), q, 2, 1)


# ---- few queries, many keys: four waves share the keys of every 64 queries, the waves
# other than the first log what they insert and the first replays the logs. The result
# must still be MinK's, slot for slot. ----

@pytest.mark.parametrize("b,n1,n2,k", [(1, 1000, 4096, 16), (2, 700, 5001, 9), (1, 64, 2048, 5),
                                        (3, 2000, 4100, 8), (1, 16384, 16384, 16),
                                        (1, 300, 65536, 12), (2, 100, 2049, 7),
                                        (1, 5000, 8191, 13), (1, 500, 9000, 20),
                                        (2, 300, 8192, 32), (1, 200, 65536, 17)])
def test_shared_key_sweep_shapes(cuda, b, n1, n2, k):
    g = gen(n1 + n2 + k)
    check_raw(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), k, cuda)


@pytest.mark.parametrize("k", [6, 16, 24])
def test_shared_key_sweep_with_overflowing_logs(cuda, k):
    # keys ordered from far to near: every key beats the k best before it, so every key of
    # every slice is logged and the logs overflow
    g = gen(31)
    q = uniform_cloud(g, 2, 500) * 0.01
    r = torch.linspace(5.0, 0.1, 9000)
    key = torch.stack([r, torch.zeros_like(r), torch.zeros_like(r)], dim=1)[None].repeat(2, 1, 1)
    key = key + 1e-4 * uniform_cloud(g, 2, 9000)
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("k,n2", [(5, 4500), (16, 4500), (28, 9000)])
def test_shared_key_sweep_ties_and_nan(cuda, k, n2):
    g = gen(32)
    q, key = lattice_cloud(g, 2, 800, 4), lattice_cloud(g, 2, n2, 4)
    check_raw(q, key, k, cuda)
    q, key = uniform_cloud(g, 2, 800), uniform_cloud(g, 2, n2)
    key[0, 0, 1] = float("nan")          # slot 0 of the fill: the lane never inserts again
    key[1, 3, 0] = float("nan")          # a later fill slot
    key[1, 1152, 2] = float("nan")       # first key of the second slice (4 slices of 1152)
    if n2 > 4512:
        key[1, 4512, 2] = float("nan")   # first key of the second of 2 slices of 4512
    key[0, 3000:3100] = float("nan")
    key[1, n2 - 1] = float("inf")
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("b,n1,n2,k", [(1, 1000, 3000, 3), (2, 700, 5001, 4), (1, 64, 1024, 1),
                                        (3, 2000, 4096, 2), (1, 300, 65536, 3),
                                        (1, 32768, 1500, 3), (2, 100, 1025, 4)])
def test_shared_key_sweep_for_k_up_to_4(cuda, b, n1, n2, k):
    g = gen(n1 + n2 + k)
    check_raw(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), k, cuda)


@pytest.mark.parametrize("k", [1, 3, 4])
def test_shared_key_sweep_for_small_k_on_hard_inputs(cuda, k):
    g = gen(41)
    # far-to-near keys: every key is inserted, the logs overflow
    q = uniform_cloud(g, 2, 300) * 0.01
    r = torch.linspace(5.0, 0.1, 3000)
    key = torch.stack([r, torch.zeros_like(r), torch.zeros_like(r)], dim=1)[None].repeat(2, 1, 1)
    check_raw(q, key + 1e-4 * uniform_cloud(g, 2, 3000), k, cuda)
    # exact ties
    check_raw(lattice_cloud(g, 2, 500, 4), lattice_cloud(g, 2, 2500, 4), k, cuda)
    # NaN in the fill, at the start of a slice, in a run; an infinite key
    q, key = uniform_cloud(g, 2, 500), uniform_cloud(g, 2, 2500)
    key[0, 0, 1] = float("nan")
    key[1, min(k - 1, 2), 0] = float("nan")
    key[1, 640, 2] = float("nan")        # first key of the second slice (4 slices of 640)
    key[0, 1500:1600] = float("nan")
    key[1, 2499] = float("inf")
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("b,n1,n2,k", [(1, 100, 262144, 3), (2, 70, 65537, 1), (1, 130, 100000, 16),
                                        (1, 64, 131072, 32), (1, 50, 70000, 20),
                                        (1, 100, 262145, 4), (1, 40, 131073, 17),
                                        (2, 90, 150001, 8), (1, 60, 600000, 3),
                                        (1, 40, 300001, 16), (1, 30, 400000, 32)])
def test_shared_key_sweep_beyond_65536_keys(cuda, b, n1, n2, k):
    """Few queries against key clouds too long for 16-bit key indices: the slots hold 32-bit
    indices and the logs positions within a slice of at most 65536 keys; clouds longer than
    the waves' slices together (262144 keys for k <= 16, 131072 for k <= 32) are taken in
    several groups of slices."""
    g = gen(n1 + n2 + k)
    check_raw(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), k, cuda)


@pytest.mark.parametrize("n2", [90001, 300000])
@pytest.mark.parametrize("k", [2, 7, 16, 30])
def test_shared_key_sweep_beyond_65536_keys_on_hard_inputs(cuda, k, n2):
    g = gen(43)
    # far-to-near keys: every key is inserted and every log overflows
    q = uniform_cloud(g, 1, 80) * 0.01
    r = torch.linspace(5.0, 0.1, n2)
    key = torch.stack([r, torch.zeros_like(r), torch.zeros_like(r)], dim=1)[None]
    check_raw(q, key + 1e-5 * uniform_cloud(g, 1, n2), k, cuda)
    # exact ties, also across slices
    check_raw(lattice_cloud(g, 1, 100, 4), lattice_cloud(g, 1, n2, 4), k, cuda)
    # NaN in the fill, at the start of slices (90001 keys: four of 22528, two of 45024;
    # 300000 keys: two groups of four slices of 37504, three groups of two of 50016), in a
    # run that covers a slice boundary; infinite keys at the end
    q, key = uniform_cloud(g, 1, 100), uniform_cloud(g, 1, n2)
    key[0, 0, 1] = float("nan")
    for j in (22528, 45024, 45056, 37504, 150016, 100032, 200064):
        if j < n2:
            key[0, j, j % 3] = float("nan")
    key[0, 67500:67700] = float("nan")
    key[0, n2 - 2:] = float("inf")
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("k", [3, 4, 5, 8, 16, 17, 33, 130])
def test_slot_order_of_the_hand_worked_mink_run(cuda, k, dtype):
    # Expected rows are literals worked out by hand from mink.cuh:61-89 (tests/util.py):
    # a rejected key equal to the maximum, two slots tying for the new maximum (the lower
    # one is the next victim), and an insertion that leaves the maximum in the written slot
    # although a lower slot ties. Every kernel family sees the run (k selects registers,
    # the LDS tree or the global variant; 70 queries span two waves, 5000 far keys behind
    # the run exercise the chunked sweeps and must all be rejected).
    from torkit3d_amd import _C
    from util import MINK_STATES, mink_worked_example

    for m in sorted(MINK_STATES):
        key, dist, idx = mink_worked_example(m, k, np.float64)
        for tail in (0, 5000):
            far = np.zeros((1, tail, 3))
            far[0, :, 0] = 50.0 + np.arange(tail) % 7
            keys = torch.from_numpy(np.concatenate([key, far], 1)).to(dtype).to(cuda)
            query = torch.zeros(1, 70, 3, dtype=dtype, device=cuda)
            got_d, got_i = _C.knn_distance_cuda(query, keys, k, 1)
            want_d = torch.from_numpy(dist).to(dtype).to(cuda).expand(70, -1)
            want_i = torch.from_numpy(idx).to(cuda).expand(70, -1)
            assert torch.equal(got_d[0], want_d), "distances, m=%d tail=%d" % (m, tail)
            assert torch.equal(got_i[0], want_i), "indices, m=%d tail=%d" % (m, tail)


# ---- many queries: the pre-filtered kernel. A cheaper score rules pairs out, candidates wait
# in per-lane queues and are inserted later with the exact arithmetic. Whatever the input,
# distances, indices and slot order must be MinK's: these cases aim at its error bound, its
# queues, its stage boundaries and its fallbacks. (Sizes are chosen inside the range where
# the dispatcher takes this kernel: 65536 queries or more against 2048 keys or more.) ----

def _filter_case(kind, g, k, b=8, n1=8192 + 5, n2=2048 + 37):  # ragged: partial workgroup, partial chunk
    q, key = uniform_cloud(g, b, n1), uniform_cloud(g, b, n2)
    if kind == "uniform":
        pass
    elif kind == "lattice":                      # exact ties everywhere
        q, key = lattice_cloud(g, b, n1, 4), lattice_cloud(g, b, n2, 4)
    elif kind == "far_to_near":                  # every key is inserted: queues always full
        r = torch.linspace(5.0, 0.1, n2)
        key = torch.stack([r, torch.zeros_like(r), torch.zeros_like(r)], dim=1)[None].repeat(b, 1, 1)
        key = key + 1e-4 * uniform_cloud(g, b, n2)
        q = q * 0.01
    elif kind == "near_to_far":                  # nothing after the fill is inserted
        r = torch.linspace(0.1, 5.0, n2)
        key = torch.stack([r, torch.zeros_like(r), torch.zeros_like(r)], dim=1)[None].repeat(b, 1, 1)
        q = q * 0.01
    elif kind == "far_from_origin":              # magnitude >> spacing: a loose bound
        q, key = q + 1000.0, key + 1000.0
    elif kind == "separated":                    # queries far from every key
        q = q + 50.0
    elif kind == "tiny":                         # squares underflow
        q, key = q * 1e-20, key * 1e-20
    elif kind == "huge":                         # squares overflow the bound's range
        q, key = q * 1e18, key * 1e18
    elif kind == "huge_queries":                 # only the queries are beyond the bound
        q = q * 3e18
    elif kind == "scaled_small":                 # inside the range the matrix scores rescale
        q, key = q * 1e-9, key * 1e-9
    elif kind == "scaled_large":
        q, key = q * 3e9 + 1e9, key * 3e9 + 1e9
    elif kind == "far_queries":                  # some queries beyond the fp16 pieces' range
        q[:, ::97] *= 400.0                      # (200 times the key cloud's extent)
        q[:, 5::211, 2] += 2.0e4
        q[:, 11::301] *= 150.0                   # inside the range, thresholds of order 1e4
    elif kind == "clusters":
        centres = uniform_cloud(g, b, 8) * 100.0
        def mk(n):
            pick = torch.randint(0, 8, (b, n), generator=g)
            return torch.gather(centres, 1, pick[:, :, None].expand(-1, -1, 3)) \
                + 1e-3 * uniform_cloud(g, b, n)
        q, key = mk(n1), mk(n2)
    elif kind == "duplicates":                   # every distance of a query ties
        key = uniform_cloud(g, b, 1).expand(b, n2, 3).contiguous()
    elif kind == "nan_and_inf":
        key[0, 0, 1] = float("nan")              # slot 0 of the fill: nothing is inserted later
        key[1, min(k - 1, 2), 0] = float("nan")  # a later fill slot keeps its NaN
        key[2, 700, 2] = float("nan")            # beyond the fill: never inserted
        key[3, 1, 0] = float("inf")              # an infinite coordinate: exact fallback
        key[4, 1500, 1] = -float("inf")
        key[5, 512:700] = float("nan")           # a run across a stage boundary
        q[6, 3, 2] = float("nan")
        q[7, ::50] = float("inf")
    else:
        raise ValueError(kind)
    return q.contiguous(), key.contiguous()


@pytest.mark.parametrize("k", [1, 3, 4, 7, 9, 13, 16, 17, 25, 32])
@pytest.mark.parametrize("kind", ["uniform", "lattice", "far_to_near", "near_to_far",
                                  "far_from_origin", "separated", "tiny", "huge", "huge_queries",
                                  "scaled_small", "scaled_large", "far_queries",
                                  "clusters", "duplicates", "nan_and_inf"])
def test_prefiltered_kernel_is_exact_on_hard_inputs(cuda, kind, k):
    q, key = _filter_case(kind, gen(sum(map(ord, kind)) + k), k)
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("k", [5, 8, 9, 12, 16, 17, 24, 32])
@pytest.mark.parametrize("steps", [1, 2, 16])
def test_prefiltered_kernel_with_sorted_slots_on_equal_distances(cuda, steps, k):
    # For 5 to 32 neighbours the kernel keeps a query's distances in descending order and the
    # slot numbers beside them; among equal distances MinK's rescan (mink.cuh:74-87) decides
    # which slot is overwritten next: the slot just written if nothing is strictly above it,
    # else the lowest slot holding the largest distance. Lattices of 3, 5 and 33 positions
    # per axis: a handful of distinct distances, so nearly every insertion meets equals, and
    # runs of equals that are longer than the list.
    g = gen(100 * steps + k)
    check_raw(lattice_cloud(g, 4, 8192 + 5, steps), lattice_cloud(g, 4, 2048 + 37, steps), k, cuda)
    # the same keys sorted from far to near the first query, so that every key is inserted
    key = lattice_cloud(g, 4, 2048 + 37, steps)
    order = key.norm(dim=2).argsort(dim=1, descending=True)
    key = torch.gather(key, 1, order[:, :, None].expand(-1, -1, 3)).contiguous()
    check_raw(0.01 * uniform_cloud(g, 4, 8192 + 5), key, k, cuda)


# ---- k = 17..32 with 32768 to 131071 queries against 4096 keys or more: the same matrix
# sweep feeding the LDS tournament tree (one query per lane, two blocks of 32 per wave) ----

@pytest.mark.parametrize("k", [17, 32])
@pytest.mark.parametrize("kind", ["uniform", "lattice", "far_to_near", "near_to_far",
                                  "far_from_origin", "separated", "tiny", "huge", "huge_queries",
                                  "scaled_small", "scaled_large", "far_queries",
                                  "clusters", "duplicates", "nan_and_inf"])
def test_tree_kernel_with_matrix_sweep_on_hard_inputs(cuda, kind, k):
    q, key = _filter_case(kind, gen(sum(map(ord, kind)) + k), k, b=8, n1=4096 + 5, n2=4096 + 37)
    assert 32768 <= q.shape[0] * q.shape[1] < 131072 and key.shape[1] >= 4096
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("b,n1,n2,k", [(32, 2048, 8192, 32), (16, 2048, 4096, 20), (5, 8000, 4097, 31),
                                        (2, 20000, 65536, 24), (33, 1000, 4096 + 255, 18)])
def test_tree_kernel_with_matrix_sweep_shapes(cuda, b, n1, n2, k):
    g = gen(n1 + n2 + k)
    check_raw(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), k, cuda)


@pytest.mark.parametrize("b,n1,n2,k", [(4, 8192, 8192, 12),     # 32768 queries, long key cloud
                                        (64, 4096, 1024, 2),     # 262144 queries, two stages
                                        (128, 2048, 513, 3),     # one key into the second stage
                                        (128, 2048, 512, 4),     # exactly one stage
                                        (2, 70000, 2048, 5), (40, 4096, 4097, 9)])
def test_prefiltered_kernel_shapes(cuda, b, n1, n2, k):
    g = gen(n1 + n2 + k)
    check_raw(uniform_cloud(g, b, n1), uniform_cloud(g, b, n2), k, cuda)


def test_prefiltered_three_nn_on_both_layouts(cuda):
    from torkit3d_amd.ops.interpolate_feature import three_nn_interpolation

    g = gen(43)
    q, key = uniform_cloud(g, 9, 8192 + 3), uniform_cloud(g, 9, 2048 + 1)
    od, oi = oracle.knn(q.numpy(), key.numpy(), 3)
    ow = oracle.three_nn_weights(od)
    for transpose in (False, True):
        a = q.to(cuda).transpose(1, 2).contiguous() if transpose else q.to(cuda)
        c = key.to(cuda).transpose(1, 2).contiguous() if transpose else key.to(cuda)
        d, i, w = three_nn_interpolation(a, c, transpose)
        np.testing.assert_array_equal(d.cpu().numpy(), od)
        np.testing.assert_array_equal(i.cpu().numpy(), oi)
        np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=3e-7, atol=0)


@pytest.mark.parametrize("k", [3, 4, 5, 8, 16, 20, 32])
def test_prefiltered_kernel_on_the_hand_worked_mink_run(cuda, k):
    # the literal rows of tests/util.py again, now with enough queries (140000 copies) and
    # keys (5000 far ones behind the run) for the dispatcher to take the pre-filtered kernel
    from torkit3d_amd import _C
    from util import MINK_STATES, mink_worked_example

    for m in sorted(MINK_STATES):
        key, dist, idx = mink_worked_example(m, k, np.float32)
        far = np.zeros((1, 5000, 3), np.float32)
        far[0, :, 0] = 50.0 + np.arange(5000) % 7
        keys = torch.from_numpy(np.concatenate([key, far], 1)).to(cuda)
        query = torch.zeros(1, 140000, 3, device=cuda)
        got_d, got_i = _C.knn_distance_cuda(query, keys, k, 1)
        want_d = torch.from_numpy(dist).to(cuda)
        want_i = torch.from_numpy(idx).to(cuda)
        assert bool((got_d[0] == want_d).all()), "distances, m=%d" % m
        assert bool((got_i[0] == want_i).all()), "indices, m=%d" % m


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("b,n1,n2,k", [(2, 700, 900, 3), (8, 8192 + 1, 2048 + 3, 4),   # pre-filtered
                                        (2, 300, 1000, 7), (16, 8192, 2048, 16),        # pre-filtered
                                        (2, 300, 1000, 16), (1, 100, 9000, 6),           # LDS tree
                                        (8, 2048, 2048, 20),   # the k = 20 graph of DGCNN
                                        (2, 500, 3000, 40), (1, 200, 70000, 12),
                                        (1, 100, 500, 33), (1, 64, 300, 64),
                                        (1, 40, 200, 65)])                               # copies
def test_channels_first_clouds_are_read_in_place_or_copied(cuda, b, n1, n2, k, dtype):
    # reference: knn_points(transpose=True), torkit3d/ops/knn_points.py:40-45
    # knn_points(transpose=True) on [B,3,N] clouds: same rows as on the [B,N,3] clouds
    from torkit3d_amd import _fused
    from torkit3d_amd.ops.knn_points import knn_points

    g = gen(n1 + k)
    q, key = uniform_cloud(g, b, n1).to(dtype), uniform_cloud(g, b, n2).to(dtype)
    od, oi = oracle.knn(q.numpy(), key.numpy(), k)
    qt = q.to(cuda).transpose(1, 2).contiguous()
    kt = key.to(cuda).transpose(1, 2).contiguous()
    d, i = knn_points(qt, kt, k, transpose=True)
    np.testing.assert_array_equal(d.cpu().numpy(), od)
    np.testing.assert_array_equal(i.cpu().numpy(), oi)
    raw = _fused.knn_distance_bcn(qt, kt, k, 1)
    # the library reads [B,3,N] in place for every k <= 64 (fp32: the pre-filtered sweep, the
    # register kernel or the LDS tree kernel); beyond it declines and the wrapper copies
    declined = k > 64
    assert (raw is None) == declined
    if raw is not None:
        assert torch.equal(raw[0], d) and torch.equal(raw[1], i)


@pytest.mark.parametrize("b,n1,n2,k", [(32, 2048, 8192, 32), (4, 512, 10000, 64),
                                        (4, 10000, 512, 3)])
def test_shapes_the_reference_author_profiled(cuda, b, n1, n2, k):
    # tests/ops/test_knn_distance.py:58-61 (profile runs, randn clouds, no recorded result)
    g = gen(8)
    q = torch.randn(b, n1, 3, generator=g)
    key = torch.randn(b, n2, 3, generator=g)
    check_raw(q, key, k, cuda)


@pytest.mark.parametrize("n2,k", [(65536, 16), (65537, 16), (70001, 11)])
def test_prefilter_kernel_around_the_16_bit_index_limit(cuda, n2, k):
    # With up to 65536 keys the 16-slot pre-filter kernel keeps its slots' key indices in LDS
    # as 16-bit values, beyond that in registers; both forced through the test-only entry
    # point, with the winners placed at the far end of the cloud
    from debug_abi import knn_filter

    g = gen(n2 + k)
    q, key = uniform_cloud(g, 1, 700), uniform_cloud(g, 1, n2)
    key[0, -40:] = q[0, :40] + 1e-4      # the last keys are the nearest of the first queries
    got = knn_filter(q.to(cuda), key.to(cuda), k)
    assert got is not None
    od, oi = oracle.knn(q.numpy(), key.numpy(), k)
    np.testing.assert_array_equal(got[0].cpu().numpy(), od)
    np.testing.assert_array_equal(got[1].cpu().numpy(), oi)
    assert int(oi.max()) >= n2 - 40
