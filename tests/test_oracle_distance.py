"""Pins of the oracle's distance (oracle/oracle.c, after
extension/inc/distance.h:31-55): float64 as an independent value, and inputs
whose float32 result depends on the summation order, worked out by hand."""
import numpy as np
import pytest

import oracle


@pytest.mark.parametrize('d', [8, 16, 96, 128, 200, 768])
def test_matches_float64(d):
    # test_operators.py:116-136 uses atol 1e-3 against cdist^2
    rng = np.random.default_rng(d)
    storage = rng.normal(size=(500, d)).astype(np.float32)
    q = rng.normal(size=d).astype(np.float32)
    nodes = rng.integers(0, 500, size=77).astype(np.int64)
    out = oracle.square_dist(q, storage, nodes)
    exact = ((q.astype(np.float64) - storage[nodes].astype(np.float64)) ** 2).sum(-1)
    assert np.allclose(out, exact, rtol=2e-6, atol=0)
    assert np.allclose(out, exact, atol=1e-3)


def one(diffs):
    d = len(diffs)
    q = np.zeros(d, np.float32)
    row = -np.array([diffs], np.float32)      # q - row = diffs
    return float(oracle.square_dist(q, row, np.zeros(1, np.int64))[0])


def test_lanes_are_added_left_to_right():
    """Squares 2^24, 1, 1, 1, 1, 1, 1, 1 in lanes 0..7.  Adding from lane 0
    upwards every +1 is lost to rounding (2^24 + 1 rounds to even): 2^24.
    Any pairwise order would keep some of the ones."""
    diffs = [4096.0] + [1.0] * 7
    assert one(diffs) == 16777216.0
    # lane 7 large instead: the seven ones add up first and survive
    assert one([1.0] * 7 + [4096.0]) == 16777216.0 + 8.0  # 7 rounds to even 8


def test_element_j_goes_to_lane_j_mod_8():
    """d = 16.  Elements 0 and 8 share lane 0: fma(1, 1, 2^24) is 2^24, so
    the one is lost inside the lane.  Put the one into element 9 instead
    (lane 1) and it is still lost in the left-to-right sum; put it in front
    of the large value (element 0 small, element 8 large) and it is lost as
    well — in each case the result is exactly 2^24, while a single running
    sum over 16 elements in index order would give 2^24 for the first and
    third case only if it added in exactly this order."""
    big, z = 4096.0, 0.0
    assert one([big] + [z] * 7 + [1.0] + [z] * 7) == 16777216.0
    assert one([1.0] + [z] * 7 + [big] + [z] * 7) == 16777216.0
    # three ones in three different lanes of the second group, large value in
    # lane 0: left to right 2^24 + 1 + 1 + 1 stays 2^24; had the second group
    # been summed on its own first (3) the result would be 2^24 + 4
    assert one([big] + [z] * 7 + [z, 1.0, 1.0, 1.0] + [z] * 4) == 16777216.0


def test_one_fma_per_element():
    """Lane 0 sees the differences 2^-12 and then t = 1 + 2^-12.  The first
    leaves 2^-24 in the accumulator.  t^2 = 1 + 2^-11 + 2^-24 exactly, so a
    fused multiply-add gives 1 + 2^-11 + 2^-23, which float32 holds; with a
    rounded product (1 + 2^-11, the tie going to even) the 2^-24 is lost
    twice and the result is 1 + 2^-11."""
    d = 16
    q = np.zeros(d, np.float32)
    row = np.zeros((1, d), np.float32)
    row[0, 0], row[0, 8] = -(2.0 ** -12), -(1.0 + 2.0 ** -12)
    got = float(oracle.square_dist(q, row, np.zeros(1, np.int64))[0])
    assert got == 1.0 + 2.0 ** -11 + 2.0 ** -23


def test_rejects_bad_dimension():
    with pytest.raises(RuntimeError):
        oracle.square_dist(np.zeros(12, np.float32), np.zeros((4, 12), np.float32),
                           np.zeros(1, np.int64))
