"""CPU: the radix levels of topk_slice_kernel (csrc/topk.hip) under a caller's row bound.

With a bound per row (td_topk_bounded) the kernel measures every score from the bound instead of
from the row maximum: d = top - bits for non-negative scores, top + |bits| for negative ones
(top = bits of the bound), or bits - top when the bound is negative.  This file restates that
mapping and the loop that narrows the window [lo, lo + limit) in 8192 bins until the bin of the
k-th smallest d is small enough, and checks on the CPU
  * that the loop ends after a few rounds for every valid bound, at the bin that holds the k-th
    largest score (against a numpy sort), for the score distributions of the GPU tests,
  * that it also ends when the bound is NOT a bound (a score above it wraps to a d beyond the range
    and is never counted: without the end-of-range rule the loop would spin for ever when k needs
    such an element -- a row of +inf under a finite bound did that).
The selection rule itself follows decode_select_k (kernels/include/topk/decode_select_k.cuh:25-62
of the reference): the k largest scores of a row."""
import numpy as np
import pytest

NO_ELEMENT = 0xFFFFFFFF
BINS, LIST = 8192, 1024
M32 = 1 << 32


def nbits(x):
    return int(x).bit_length()


def map_to_d(row, bound, sixteen_bit=False):
    u = np.asarray(row, dtype=np.float32).view(np.uint32).astype(np.uint64)
    top = int(np.float32(np.float32(bound) + np.float32(0)).view(np.uint32))
    if sixteen_bit:   # room for scores rounded up past an fp32 bound
        if top < 0x80000000:
            top += 0x10000
        else:
            top = top - 0x10000 if top - 0x10000 >= 0x80000000 else 0
    mixed = top < 0x80000000
    dmax = top + 0x7F800000 if mixed else 0xFF800000 - top
    neg_add = (top - 0x80000000) % M32 if mixed else (-top) % M32
    d = np.where(u < 0x80000000, (top - u) % M32, (u + neg_add) % M32)
    return d, dmax


def level_loop(d, dmax, k):
    """-> (rounds, lo, s, krem, gave_up); the threshold lies in [lo, lo + 2^s)"""
    lo, krem = 0, k
    s, limit = max(nbits(dmax) - 13, 0), dmax + 1
    if s > 16:
        s, limit = 16, (BINS - 1) << 16
    rounds = 0
    while dmax != 0:
        rounds += 1
        assert rounds <= 8, "the level loop does not end"
        x = (d - lo) % M32
        inside = x < limit
        total = int(inside.sum())
        if krem > total:                      # not in this window
            if limit > dmax - lo:             # ... and the window reached the end of the range
                return rounds, NO_ELEMENT, 0, 0, True
            krem -= total
            lo += limit
            rem = dmax - lo
            s, limit = max(nbits(rem) - 13, 0), rem + 1
            continue
        hist = np.bincount((x[inside] >> s).astype(np.int64), minlength=BINS)
        assert len(hist) == BINS, "a bin index beyond the histogram"
        before = np.cumsum(hist) - hist
        tb = int(np.searchsorted(np.cumsum(hist), krem))
        krem -= int(before[tb])
        lo += tb << s
        if s == 0 or hist[tb] <= LIST:
            break
        limit, s = 1 << s, (s - 13 if s > 13 else 0)
    return rounds, lo, s, krem, False


def rows_for_the_loop():
    g = np.random.default_rng(5)
    n = 5000
    yield "normal", g.standard_normal(n).astype(np.float32)
    yield "all negative", (-10 + 2 * g.standard_normal(n)).astype(np.float32)
    yield "few positive", (-3 + g.standard_normal(n)).astype(np.float32)
    wide = (g.random(n) * 1e-30).astype(np.float32)
    wide[:100] = 0.5 + 0.5 * g.random(100)
    yield "100 binades", wide
    zeros = -g.random(n).astype(np.float32)
    zeros[::3] = 0.0
    zeros[1::3] = -0.0
    yield "signed zeros", zeros
    yield "denormals", (g.standard_normal(n) * 1e-41).astype(np.float32)
    yield "one value", np.full(n, 3.25, np.float32)
    minus_inf = g.standard_normal(n).astype(np.float32)
    minus_inf[::7] = -np.inf
    yield "-inf", minus_inf
    yield "crowded bin", (1.0 + g.random(n) * 1e-3).astype(np.float32)


@pytest.mark.parametrize("name,row", list(rows_for_the_loop()))
def test_valid_bounds_find_the_kth_largest(name, row):
    top = float(row.max())
    for bound in (top, top + 0.37 * abs(top) + 3.0, top + 1e-3 * abs(top), abs(top) * 64 + 1e-30):
        if not np.isfinite(bound) or bound < top:
            continue
        d, dmax = map_to_d(row, bound)
        assert (d <= dmax).all(), "a valid bound leaves no score beyond the range"
        order = np.sort(d)
        for k in (1, 7, len(row) // 16, len(row) - 1, len(row)):
            rounds, lo, s, krem, gave_up = level_loop(d, dmax, k)
            assert not gave_up and rounds <= 5, (name, bound, k, rounds)
            kth = int(order[k - 1])
            assert lo <= kth < lo + (1 << s), (name, bound, k)
            inside = np.sort(d[(d >= lo) & (d < lo + (1 << s))])
            assert int(inside[krem - 1]) == kth, (name, bound, k)


def test_d_orders_scores_as_their_values():
    g = np.random.default_rng(1)
    row = np.concatenate([g.standard_normal(500), [0.0, -0.0, 1e-42, -1e-42, -np.inf]]).astype(np.float32)
    for bound in (float(row.max()), 17.0):
        d, _ = map_to_d(row, bound)
        for i in range(0, len(row), 7):
            for j in range(0, len(row), 11):
                if row[i] > row[j]:
                    assert d[i] < d[j]
                elif row[i] == row[j]:
                    assert d[i] == d[j]          # -0 and +0 are one score
    neg = (-1 - g.random(300)).astype(np.float32)
    d, _ = map_to_d(neg, float(neg.max()))
    assert (np.argsort(d, kind="stable") == np.argsort(-neg, kind="stable")).all()


def test_a_bound_below_a_score_ends_the_loop():
    """What hung the first build: a row of +inf under the largest finite value as its 'bound'."""
    row = np.full(64, np.inf, np.float32)
    d, dmax = map_to_d(row, 3.4028234663852886e38)
    assert (d > dmax).all()                      # nothing is ever counted
    rounds, lo, s, krem, gave_up = level_loop(d, dmax, 5)
    assert gave_up and rounds <= 3 and lo == NO_ELEMENT and s == 0 and krem == 0
    g = np.random.default_rng(2)
    row = g.standard_normal(4000).astype(np.float32)
    for bound in (0.0, 1.0, -5.0, float(np.sort(row)[-3])):
        d, dmax = map_to_d(row, bound)
        for k in (1, 100, 3999, 4000):
            level_loop(d, dmax, k)               # ends (the assert inside), whatever it selects
