"""Pins of the oracle's heap primitives (oracle/oracle.c) that do not restate
them: Python's heapq as an independent heap, the properties the reference's
own test checks (test/kernel/test_operators.py:8-88), and array states derived
by hand from extension/inc/heapq.cuh."""
import heapq
import math

import numpy as np
import pytest

import oracle

INF = float('inf')


def arrays(keys, vals=None):
    k = np.array(keys, np.float32)
    v = np.arange(len(keys), dtype=np.int64) if vals is None else np.array(vals, np.int64)
    return k, v


def is_heap(keys):
    return all(keys[(i - 1) // 2] <= keys[i] for i in range(1, len(keys)))


@pytest.mark.parametrize('size', [1, 2, 7, 33, 512, 1000])
def test_pop_all_leaves_sentinels(size):
    # test_operators.py:11-31
    k, v = arrays(np.zeros(size), np.zeros(size))
    for _ in range(size):
        oracle.heap_pop(k, v)
    assert np.all(np.isposinf(k)) and np.all(v == -1)


@pytest.mark.parametrize('size', [1, 5, 64, 777])
def test_pushpop_ignores_smaller_accepts_larger(size):
    # test_operators.py:33-63
    k, v = arrays(np.zeros(size), np.zeros(size))
    for _ in range(size):
        oracle.heap_pushpop(k, v, -1.0, -1)
    assert np.all(k == 0) and np.all(v == 0)
    for _ in range(size):
        oracle.heap_pushpop(k, v, 1.0, -1)
    assert np.all(k == 1.0) and np.all(v == -1)


@pytest.mark.parametrize('size', [1, 6, 100, 1024])
def test_replace_keeps_heap_order(size):
    # test_operators.py:65-86: heapify is a no-op on the result, root is -1
    k, v = arrays(np.zeros(size), np.zeros(size))
    for _ in range(size):
        oracle.heap_replace(k, v, -1.0, -1)
    assert is_heap(k.tolist())
    assert k[0] == -1


@pytest.mark.parametrize('seed', range(5))
def test_pop_order_equals_heapq(seed):
    rng = np.random.default_rng(seed)
    size = int(rng.integers(2, 300))
    data = rng.normal(size=size).astype(np.float32)
    ref = data.tolist()
    heapq.heapify(ref)
    k, v = arrays(ref, list(range(size)))
    assert is_heap(k.tolist())
    popped = [oracle.heap_pop(k, v)[0] for _ in range(size)]
    assert popped == [heapq.heappop(ref) for _ in range(size)]
    assert np.all(np.isposinf(k))


@pytest.mark.parametrize('seed', range(5))
def test_pushpop_tracks_largest_elements(seed):
    """A min-heap under pushpop keeps exactly the `size` largest keys seen
    (ties aside) — the property the search uses for its result list."""
    rng = np.random.default_rng(100 + seed)
    size = int(rng.integers(1, 64))
    k, v = arrays(np.full(size, -INF), np.full(size, -1))
    stream = rng.permutation(1000)[:400].astype(np.float32)
    for i, x in enumerate(stream):
        oracle.heap_pushpop(k, v, float(x), i)
        assert is_heap(k.tolist())
    assert sorted(k.tolist()) == sorted(stream.tolist())[-size:]
    assert all(stream[i] == key for key, i in zip(k, v))


def test_replace_and_pop_states_derived_by_hand():
    """heapq.cuh:47-77 on a 7-cell heap, step by step: the walk goes to the
    larger child (left on ties), the leaf is overwritten only by a strictly
    smaller key, which then rises past strictly larger parents."""
    k, v = arrays([INF] * 7, [-1] * 7)
    oracle.heap_replace(k, v, 5.0, 1)     # leftmost leaf 3, rises to the root
    assert k.tolist() == [5, INF, INF, INF, INF, INF, INF]
    assert v.tolist() == [1, -1, -1, -1, -1, -1, -1]
    oracle.heap_replace(k, v, 3.0, 2)     # leaf 3 again, rises over 5
    assert k.tolist() == [3, 5, INF, INF, INF, INF, INF]
    assert v.tolist() == [2, 1, -1, -1, -1, -1, -1]
    oracle.heap_replace(k, v, 4.0, 3)     # larger child of the root is cell 2
    assert k.tolist() == [3, 5, 4, INF, INF, INF, INF]
    assert v.tolist() == [2, 1, 3, -1, -1, -1, -1]
    oracle.heap_replace(k, v, 6.0, 4)     # 5 > 4: cell 1, then leaf 3
    assert k.tolist() == [3, 5, 4, 6, INF, INF, INF]
    assert v.tolist() == [2, 1, 3, 4, -1, -1, -1]
    # heapq.cuh:37-45: root out, inf sinks along the smaller child
    key, val = oracle.heap_pop(k, v)
    assert (key, val) == (3.0, 2)
    assert k.tolist() == [4, 5, INF, 6, INF, INF, INF]
    assert v.tolist() == [3, 1, -1, 4, -1, -1, -1]


def test_replace_displaces_a_live_leaf_while_cells_are_free():
    """The walk follows the larger child, not the free cells: in
    [1, 9, 2, 10, 11, inf, inf] it ends on 11.  A smaller key overwrites that
    live entry, a larger one is dropped, although cells 5 and 6 are free."""
    start = [1, 9, 2, 10, 11, INF, INF]
    k, v = arrays(start, [10, 11, 12, 13, 14, -1, -1])
    oracle.heap_replace(k, v, 5.0, 99)
    assert k.tolist() == [1, 5, 2, 10, 9, INF, INF]
    assert v.tolist() == [10, 99, 12, 13, 11, -1, -1]
    k, v = arrays(start, [10, 11, 12, 13, 14, -1, -1])
    oracle.heap_replace(k, v, 12.0, 99)
    assert k.tolist() == start
    k, v = arrays(start, [10, 11, 12, 13, 14, -1, -1])
    oracle.heap_replace(k, v, 11.0, 99)   # ties lose (heapq.cuh:62)
    assert k.tolist() == start
    assert v.tolist() == [10, 11, 12, 13, 14, -1, -1]   # 14 keeps its cell


def test_pop_known_state():
    k, v = arrays([1, 9, 2, 10, 11, INF, INF], [0, 1, 2, 3, 4, -1, -1])
    assert oracle.heap_pop(k, v) == (1.0, 0)
    assert k.tolist() == [2, 9, INF, 10, 11, INF, INF]
    assert v.tolist() == [2, 1, -1, 3, 4, -1, -1]


def test_pushpop_known_state():
    # result list: negated distances, root = worst kept (traverse_cpu.cpp:30)
    k, v = arrays([-9, -5, -7], [0, 1, 2])
    oracle.heap_pushpop(k, v, -10.0, 3)   # not better than the worst: ignored
    assert k.tolist() == [-9, -5, -7]
    oracle.heap_pushpop(k, v, -9.0, 3)    # tie: ignored (heapq.cuh:83)
    assert k.tolist() == [-9, -5, -7]
    assert v.tolist() == [0, 1, 2]        # the root keeps its value
    oracle.heap_pushpop(k, v, -6.0, 3)
    assert k.tolist() == [-7, -5, -6] and v.tolist() == [2, 1, 3]


def test_equal_keys_keep_their_places():
    """The tie rules of heapq.cuh, visible in the values only.  Sinking takes
    the left child when both children are equal (:19-21) and stops on a child
    equal to the sinking key (:22-24); a rising key stops under an equal
    parent (:69-71)."""
    k, v = arrays([1, 5, 5], [0, 1, 2])
    assert oracle.heap_pop(k, v) == (1.0, 0)
    assert k.tolist() == [5, INF, 5] and v.tolist() == [1, -1, 2]
    k, v = arrays([-9, -5, -4], [0, 1, 2])
    oracle.heap_pushpop(k, v, -5.0, 3)    # new root equals its smaller child
    assert k.tolist() == [-5, -5, -4] and v.tolist() == [3, 1, 2]
    k, v = arrays([1, 9, 2, 10, 11, INF, INF], [10, 11, 12, 13, 14, -1, -1])
    oracle.heap_replace(k, v, 9.0, 99)    # leaf 11 overwritten, parent is 9 too
    assert k.tolist() == [1, 9, 2, 10, 9, INF, INF]
    assert v.tolist() == [10, 11, 12, 13, 99, -1, -1]


def test_heap_size_ladder():
    # traverse_cpu.cpp:228-254
    expect = {1: 16, 16: 16, 17: 32, 32: 32, 33: 48, 48: 48, 49: 64, 64: 64,
              65: 96, 96: 96, 97: 128, 128: 128, 129: 192, 192: 192, 193: 256,
              256: 256, 257: 384, 384: 384, 385: 512, 512: 512, 513: 1024,
              1024: 1024, 1025: 2048, 2048: 2048, 2049: -1}
    for ef, h in expect.items():
        assert oracle.heap_size(ef) == h
    assert not math.isnan(INF)
