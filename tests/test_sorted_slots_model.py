"""The rule by which the KNN kernels keep MinK's slots as a sorted list, against the oracle.

`knn_filter_kernel_f32<..., SORTED>` (torkit3d_amd/csrc/knn.hip) does not keep a query's k
distances in slot order as the reference's MinK does (csrc/include/mink.cuh:61-89) but in
descending order, with the slot number of every position beside them, and moves slot numbers
by one rule: the new key takes the slot of the evicted maximum (position 0) and goes to
position 0 if nothing that stays is strictly above it, else behind everything above it and
behind the equal distances of lower slot numbers. This file restates that rule in a few lines
of Python and checks it against the CPU oracle's literal MinK on sequences where equal
distances are everywhere, which is where the slot order shows. It runs without a GPU; the
kernel itself is checked against the oracle by tests/test_gpu_knn.py.
"""
import math
import random

import numpy as np

import oracle


def sorted_list_knn(dist, k, kmax):
    """MinK's (distances, key indices) in slot order for one query, by the sorted-list rule."""
    neg = -math.inf
    value = [neg] * kmax            # descending; unused slots and NaNs of the fill at the end
    slot_of = list(range(kmax))     # slot number of every position
    key_in = [0] * kmax             # key index by slot
    nan_slots, frozen = set(), False
    for s in range(min(k, len(dist))):     # the fill: key s goes to slot s
        x = dist[s]
        if x != x:
            nan_slots.add(s)
            frozen |= s == 0                # MinK's maximum stays a NaN: nothing is inserted
            x = neg
        m = min(sum(1 for p in range(kmax) if value[p] >= x), s)
        for p in range(s, m, -1):
            value[p], slot_of[p] = value[p - 1], slot_of[p - 1]
        value[m], slot_of[m], key_in[s] = x, s, s
    for j in range(k, len(dist)):
        x = dist[j]
        if frozen or not x < value[0]:      # MinK's strict test against the maximum
            continue
        slot = slot_of[0]
        above = sum(1 for p in range(1, kmax) if value[p] > x)
        before = sum(1 for p in range(1, kmax) if value[p] == x and slot_of[p] < slot)
        m = 0 if above == 0 else above + before
        value = value[1:m + 1] + [x] + value[m + 1:]
        slot_of = slot_of[1:m + 1] + [slot] + slot_of[m + 1:]
        key_in[slot] = j
    out_d, out_i = [None] * k, [None] * k
    for p in range(kmax):
        if slot_of[p] < k:
            out_d[slot_of[p]], out_i[slot_of[p]] = value[p], key_in[slot_of[p]]
    for s in nan_slots:
        out_d[s] = dist[s]
    return out_d, out_i


def test_sorted_list_rule_reproduces_mink_slot_order():
    rnd = random.Random(1)
    for trial in range(400):
        k = rnd.choice([5, 8, 9, 12, 16, 17, 20, 32])
        kmax = 8 if k <= 8 else 16 if k <= 16 else 32
        n = rnd.choice([k, k + 1, 40, 150, 400])
        n = max(n, k)
        levels = rnd.choice([2, 3, 5, 17, 1000])   # distinct coordinates: few = ties everywhere
        xs = [float(rnd.randrange(levels)) for _ in range(n)]
        if rnd.random() < 0.2:
            xs.sort(reverse=True)                   # far to near: every key is inserted
        if rnd.random() < 0.15:
            for _ in range(3):
                xs[rnd.randrange(min(n, k + 3))] = math.nan
        if rnd.random() < 0.1:
            xs[rnd.randrange(n)] = math.inf
        key = np.zeros((1, n, 3), np.float32)
        key[0, :, 0] = xs
        want_d, want_i = oracle.knn(np.zeros((1, 1, 3), np.float32), key, k)
        dist = [float(np.float32(x) * np.float32(x)) for x in xs]   # as the oracle forms them
        got_d, got_i = sorted_list_knn(dist, k, kmax)
        np.testing.assert_array_equal(np.asarray(got_i), want_i[0, 0], err_msg="trial %d" % trial)
        np.testing.assert_array_equal(np.asarray(got_d, np.float32), want_d[0, 0],
                                      err_msg="trial %d" % trial)
