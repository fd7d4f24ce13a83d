"""The error bound the matrix-core pre-filters rely on, checked against the hardware.

The chamfer and KNN pre-filters compute their scores with v_mfma_f32_32x32x16_f16 and stay
exact only because every score is within a stated distance of the exact value; everything
inside that distance is re-evaluated in the canonical fp32 form. The part of the bound that
no amount of reading can establish is how the matrix core adds its 16 products. What it does
(measured here): the products are aligned to the largest exponent among them and cut off
about 25 bits below it, where the exponent of a product is the sum of its factors' exponent
fields - so a subnormal fp16 factor counts as 2^-14 however small it is, and a tiny product
of a subnormal and a large factor can cost the other products some of their low bits. With
m(v) = max(|v|, 2^-14) for v != 0, the "magnitude as the matrix core sees it", the kernels
budget

    |mfma(a, b) - sum_i a_i b_i|  <=  32 u * sum_i m(a_i) m(b_i),        u = 2^-24

(one unit in the last place of the running sum per addition). For the terms the kernels
build, sum m(a_i) m(b_i) <= 1.02 R with R = (max|k'| + |q'|)^2, provided the cloud holds a key
with |k'| >= 1/4 (the kernels check that): a term with a subnormal piece is seen as at most
2^-14 times the other factor, which is below 2^-10 R. The products of two fp16 values are
exact in fp32 and in float64; the exact sums below are taken with math.fsum.

test_accumulation_of_sixteen_products aims term sets at that budget: products that cancel,
subnormal fp16 pieces, |k'|^2 pieces at the top of the range, terms spread over the whole
exponent range of fp16 (where the error reaches 147 u times the largest true product, which
is why the budget is not stated in true magnitudes), and random patterns.
test_chamfer_score_end_to_end checks the whole score of the chamfer kernels - splitting
into fp16 pieces, |k'|^2 as staged, the matrix instruction - against |k'|^2 - 2 q'.k' in
exact arithmetic:

    |score - exact|  <=  (2 + 7 + 3.2 + 33) u R      (pieces, subnormal pieces at
                                                      max|k'| >= 1/4, |k'|^2, the additions)

and test_small_key_norms_break_the_bound shows what the check on max|k'| is for.
"""
import math

import numpy as np
import pytest
import torch

from debug_abi import chamfer_scores, mfma_dot16

pytestmark = pytest.mark.gpu
U = 2.0 ** -24


def f16_value(bits):
    return bits.astype(np.uint16).view(np.float16).astype(np.float64)


def f16_bits(values):
    return np.asarray(values, np.float64).astype(np.float16).view(np.uint16)


def term_sets(rng):
    """(name, key_terms [T,32,16], query_terms [T,32,16]) as fp16 bit patterns."""
    T = 24
    sets = []
    # 1. products that cancel: equal magnitudes with alternating signs, and a small remainder
    k = np.abs(rng.normal(size=(T, 32, 16))) + 0.5
    q = np.abs(rng.normal(size=(T, 32, 16))) + 0.5
    k[:, :, 1::2] = k[:, :, 0::2]
    q[:, :, 1::2] = -q[:, :, 0::2]
    k[:, :, 14:] = rng.normal(size=(T, 32, 2)) * 1e-3
    q[:, :, 14:] = 1.0
    sets.append(("cancelling", f16_bits(k * rng.choice([1.0, 50.0, 1e-2], size=(T, 1, 1))),
                 f16_bits(q * rng.choice([1.0, 100.0], size=(T, 1, 1)))))
    # 2. subnormal fp16 pieces on the key side (exponent field 0), on the query side, on both
    sub = rng.integers(0, 1024, size=(T, 32, 16)).astype(np.uint16) | \
        (rng.integers(0, 2, size=(T, 32, 16)).astype(np.uint16) << 15)
    norm = f16_bits(rng.normal(size=(T, 32, 16)) * rng.choice([1.0, 1e3, 1e-3], size=(T, 1, 1)))
    sets.append(("subnormal keys", sub, norm))
    sets.append(("subnormal queries", norm, sub))
    sets.append(("subnormal both", sub, np.roll(sub, 5, axis=2)))
    # mixed: a few normal terms among subnormal ones
    mixed = sub.copy()
    mixed[:, :, ::5] = norm[:, :, ::5]
    sets.append(("subnormal and normal mixed", mixed, norm))
    # 3. |k'|^2 pieces at the top of the range against 1, beside coordinate products:
    #    n0 up to 181^2 (the matrix kernel's limit) and 16 (the sorted path's), residual pieces
    k = rng.normal(size=(T, 32, 16))
    q = rng.normal(size=(T, 32, 16)) * 2.0
    n = rng.uniform(0.0, 1.0, size=(T, 32)) * rng.choice([16.0, 32761.0], size=(T, 1))
    n0 = f16_value(f16_bits(n))
    n1 = f16_value(f16_bits(n - n0))
    k[:, :, 12], k[:, :, 13], k[:, :, 14], k[:, :, 15] = n0, n1, n - n0 - n1, 0.0
    q[:, :, 12:15] = 1.0
    q[:, :, 15] = 0.0
    big = rng.choice([1.0, 100.0], size=(T, 1, 1))
    k[:, :, :12] *= big
    q[:, :, :12] *= big
    sets.append(("norm pieces at the top", f16_bits(k), f16_bits(q)))
    # 4. every term at its own place in fp16's exponent range (2^-24 .. 2^15), random signs
    e = rng.integers(-24, 16, size=(T, 32, 16))
    k = np.ldexp(rng.uniform(1.0, 2.0, size=e.shape), e) * rng.choice([-1.0, 1.0], size=e.shape)
    e2 = rng.integers(-24, 16, size=(T, 32, 16))
    q = np.ldexp(rng.uniform(1.0, 2.0, size=e.shape), e2) * rng.choice([-1.0, 1.0], size=e.shape)
    sets.append(("whole exponent range", f16_bits(k), f16_bits(q)))
    # one huge product among tiny ones, and the largest finite values
    k = np.full((T, 32, 16), 2.0 ** -20)
    q = np.full((T, 32, 16), 2.0 ** -4) * rng.choice([-1.0, 1.0], size=(T, 32, 16))
    k[:, :, 3] = 65504.0
    q[:, :, 3] = 60000.0
    sets.append(("one huge product", f16_bits(k), f16_bits(q)))
    # 5. random finite bit patterns
    def finite(shape):
        b = rng.integers(0, 1 << 16, size=shape).astype(np.uint16)
        return np.where((b & 0x7c00) == 0x7c00, b & 0x83ff, b).astype(np.uint16)
    sets.append(("random patterns", finite((T, 32, 16)), finite((T, 32, 16))))
    return sets


def exact_dot(kv, qv):
    """[T,32,32] correctly rounded sums of the 16 exact products, and the sums of their
    magnitudes."""
    prod = kv[:, :, None, :] * qv[:, None, :, :]          # exact in float64
    flat = prod.reshape(-1, 16)
    exact = np.fromiter((math.fsum(row) for row in flat), np.float64, len(flat))
    # magnitudes as the matrix core sees them: a subnormal factor counts as 2^-14
    mk = np.maximum(np.abs(kv), 2.0 ** -14) * (kv != 0)
    mq = np.maximum(np.abs(qv), 2.0 ** -14) * (qv != 0)
    seen = mk[:, :, None, :] * mq[:, None, :, :]
    return exact.reshape(prod.shape[:3]), seen.sum(-1), seen.max(-1), np.abs(prod).max(-1)


def test_accumulation_of_sixteen_products(cuda):
    rng = np.random.default_rng(71)
    worst_budget, worst_seen, worst_true = 0.0, 0.0, 0.0
    for name, kt, qt in term_sets(rng):
        got = mfma_dot16(torch.from_numpy(kt.view(np.int16)).to(cuda),
                         torch.from_numpy(qt.view(np.int16)).to(cuda)).cpu().numpy().astype(np.float64)
        exact, seen_sum, seen_max, true_max = exact_dot(f16_value(kt), f16_value(qt))
        assert np.isfinite(got).all(), name
        err = np.abs(got - exact)
        bound = 32.0 * U * seen_sum
        assert (err <= bound).all(), (name, float((err / np.maximum(seen_sum, 1e-300)).max() / U))
        ok = seen_sum > 0
        worst_budget = max(worst_budget, float((err[ok] / seen_sum[ok]).max() / U))
        worst_seen = max(worst_seen, float((err[ok] / seen_max[ok]).max() / U))
        worst_true = max(worst_true, float((err[ok] / true_max[ok]).max() / U))
    print("worst error: %.2f u x sum of seen magnitudes, %.2f u x largest seen product, "
          "%.2f u x largest true product" % (worst_budget, worst_seen, worst_true))
    # the margin the budget leaves: measured 4.5 u times the sum and 6.4 u times the largest seen
    # product; it must not come closer than half the budget
    assert worst_budget <= 16.0


def score_error_in_u_r(cuda, kmax, qmax):
    # keys of norm up to kmax (the sorted path sweeps keys within 4 units of the frame, the
    # matrix kernel within 181) and queries up to qmax from the centre (8000 and 16000 are the
    # kernels' limits); every tile holds a key of norm kmax, as the scaling guarantees a key
    # of norm >= 1/4 in the cloud
    rng = np.random.default_rng(int(kmax * 1000 + qmax))
    T = 24
    k = rng.normal(size=(T, 32, 3))
    k = k / np.linalg.norm(k, axis=2, keepdims=True) * rng.uniform(0, kmax, size=(T, 32, 1))
    k[:, 0] = k[:, 0] / np.linalg.norm(k[:, 0], axis=1, keepdims=True) * kmax
    # some keys with subnormal second pieces: coordinates that are almost fp16 numbers
    k[:, 1:4] = f16_value(f16_bits(k[:, 1:4])) + 2.0 ** -26 * rng.integers(-3, 4, size=(T, 3, 3))
    q = rng.normal(size=(T, 32, 3))
    q = q / np.linalg.norm(q, axis=2, keepdims=True) * rng.uniform(0, 1, size=(T, 32, 1)) ** 3 * qmax
    k32, q32 = k.astype(np.float32), q.astype(np.float32)
    got = chamfer_scores(torch.from_numpy(k32).to(cuda),
                         torch.from_numpy(q32).to(cuda)).cpu().numpy().astype(np.float64)
    kd, qd = k32.astype(np.float64), q32.astype(np.float64)
    # exact |k|^2 - 2 q.k of the fp32 inputs: seven products of 24-bit numbers, summed exactly
    terms = np.concatenate([np.broadcast_to((kd * kd)[:, :, None, :], (T, 32, 32, 3)),
                            -2.0 * kd[:, :, None, :] * qd[:, None, :, :]], axis=-1)
    flat = terms.reshape(-1, 6)
    exact = np.fromiter((math.fsum(row) for row in flat), np.float64, len(flat)).reshape(T, 32, 32)
    knorm = np.linalg.norm(kd, axis=2).max(axis=1)[:, None, None]
    qnorm = np.linalg.norm(qd, axis=2)[:, None, :]
    R = (knorm + qnorm) ** 2
    return float((np.abs(got - exact) / R).max() / U)


@pytest.mark.parametrize("kmax,qmax", [(1.0, 2.0), (4.0, 8.0), (4.0, 8000.0), (181.0, 16000.0),
                                       (0.25, 0.0), (0.25, 0.5), (0.25, 8000.0), (1.0, 0.0)])
def test_chamfer_score_end_to_end(cuda, kmax, qmax):
    worst = score_error_in_u_r(cuda, kmax, qmax)
    print("kmax %g qmax %g: worst |score - exact| = %.2f u R" % (kmax, qmax, worst))
    assert worst <= 45.2


def test_small_key_norms_break_the_bound(cuda):
    # With every key within 0.02 of the centre the pieces' absolute floor (2^-25 per piece,
    # fp16's subnormal spacing) is no longer small against R: the score is off by a thousand
    # u R. This is why a cloud whose largest swept key norm is under 1/4 is not served by the
    # pre-filters (the sorted path hands it over; the matrix kernel's scale makes it >= 1).
    assert score_error_in_u_r(cuda, 0.02, 0.0) > 45.2
