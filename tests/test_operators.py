"""The operator hooks of the product's host library (`kernels.heapq_pop`,
`heapq_pushpop`, `heapq_replace`, `bitmask_put`, `square_dist`,
`graph_sampling`; pilot_ann/kernels/__init__.py:5-44) against the oracle,
cell for cell, and through the checks of the reference's own operator test
(test/kernel/test_operators.py)."""
import heapq
import random

import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels


@pytest.mark.parametrize('seed', range(6))
def test_heap_hooks_equal_the_oracle_cell_for_cell(seed):
    rng = random.Random(seed)
    n = rng.choice([1, 2, 3, 7, 64, 257, 1024])
    keys = torch.full((n,), float('inf'))
    values = torch.full((n,), -1, dtype=torch.long)
    ok, ov = keys.numpy().copy(), values.numpy().copy()
    for step in range(4 * n + 8):
        op = rng.choice(['replace', 'replace', 'pushpop', 'pop'])
        key, value = rng.choice([0.5, 1.0, 2.0, rng.random() * 4]), rng.randrange(1000)
        if op == 'replace':
            kernels.heapq_replace(keys, values, key, value)
            oracle.heap_replace(ok, ov, key, value)
        elif op == 'pushpop':
            kernels.heapq_pushpop(keys, values, key, value)
            oracle.heap_pushpop(ok, ov, key, value)
        else:
            kernels.heapq_pop(keys, values)
            oracle.heap_pop(ok, ov)
        assert np.array_equal(keys.numpy(), ok) and np.array_equal(values.numpy(), ov), (op, step)


@pytest.mark.parametrize('n', [1, 5, 100, 1024])
def test_heap_hooks_as_the_reference_tests_them(n):
    # test_operators.py:8-30: n pops empty a heap of zeros
    keys, values = torch.zeros(n), torch.zeros(n, dtype=torch.long)
    for _ in range(n):
        kernels.heapq_pop(keys, values)
    assert bool((keys == float('inf')).all()) and bool((values == -1).all())
    # :32-58: smaller keys never enter through pushpop, larger ones take over
    keys, values = torch.zeros(n), torch.zeros(n, dtype=torch.long)
    for _ in range(n):
        kernels.heapq_pushpop(keys, values, key=-1.0, value=-1)
    assert bool((keys == 0).all()) and bool((values == 0).all())
    for _ in range(n):
        kernels.heapq_pushpop(keys, values, key=1.0, value=-1)
    assert bool((keys == 1).all()) and bool((values == -1).all())
    # :60-80: replace keeps the heap order and brings the smallest to the root
    keys, values = torch.zeros(n), torch.zeros(n, dtype=torch.long)
    for _ in range(n):
        kernels.heapq_replace(keys, values, key=-1.0, value=-1)
    as_list = keys.tolist()
    heapified = list(as_list)
    heapq.heapify(heapified)
    assert heapified == as_list and as_list[0] == -1


def test_heap_hook_argument_checks():
    keys, values = torch.zeros(4), torch.zeros(4, dtype=torch.long)
    with pytest.raises(RuntimeError):
        kernels.heapq_pop(keys, values[:3])
    with pytest.raises(RuntimeError):
        kernels.heapq_pop(keys.double(), values)
    with pytest.raises(RuntimeError):
        kernels.heapq_replace(keys, values.int(), 1.0, 1)
    with pytest.raises(RuntimeError):
        kernels.heapq_pushpop(keys.view(2, 2), values.view(2, 2), 1.0, 1)
    kernels.heapq_pop(torch.zeros(0), torch.zeros(0, dtype=torch.long))   # nothing to do


def test_bitmask_put():
    # test_operators.py:86-108
    g = torch.Generator().manual_seed(0)
    keys = torch.randint(16384, (700,), generator=g)
    marks = kernels.bitmask_put(keys, n=16384)
    assert marks.dtype == torch.int32 and marks.shape == (16384,)
    assert int(torch.count_nonzero(marks)) == keys.unique().numel()
    assert bool((marks[keys] == 1).all())
    assert int(kernels.bitmask_put(torch.zeros(0, dtype=torch.long), n=8).abs().sum()) == 0
    with pytest.raises(RuntimeError):
        kernels.bitmask_put(torch.tensor([8]), n=8)
    with pytest.raises(RuntimeError):
        kernels.bitmask_put(torch.tensor([-1]), n=8)
    with pytest.raises(RuntimeError):
        kernels.bitmask_put(keys.int(), n=16384)


@pytest.mark.parametrize('d,n_nodes', [(8, 1), (16, 4), (16, 5), (96, 9), (256, 1000), (200, 3)])
def test_square_dist(d, n_nodes):
    g = torch.Generator().manual_seed(d + n_nodes)
    query = torch.randn(d, generator=g)
    storage = torch.randn(3000, d, generator=g)
    nodelist = torch.randint(3000, (n_nodes,), generator=g)
    out = kernels.square_dist(query, storage, nodelist)
    # bit for bit the oracle's sum (distance.h:31-55: eight lanes, left to right)
    assert np.array_equal(out.numpy(),
                          oracle.square_dist(query.numpy(), storage.numpy(), nodelist.numpy()))
    # test_operators.py:111-131
    exact = torch.cdist(query.unsqueeze(0).double(), storage[nodelist].double()).square()[0]
    assert torch.allclose(out.double(), exact, atol=1e-3)


def test_square_dist_argument_checks():
    query, storage = torch.zeros(16), torch.zeros(10, 16)
    with pytest.raises(RuntimeError):
        kernels.square_dist(query, storage, torch.tensor([10]))
    with pytest.raises(RuntimeError):
        kernels.square_dist(query, storage, torch.tensor([-1]))
    with pytest.raises(RuntimeError):
        kernels.square_dist(torch.zeros(12), torch.zeros(10, 12), torch.tensor([0]))
    with pytest.raises(RuntimeError):
        kernels.square_dist(query, torch.zeros(10, 8), torch.tensor([0]))
    assert kernels.square_dist(query, storage, torch.zeros(0, dtype=torch.long)).shape == (0,)


def test_graph_sampling_hook():
    # a ring: node i -> i + 1; one hop from a seed adds its successor
    n = 50
    indptr = list(range(n + 1))
    indices = [(i + 1) % n for i in range(n)]
    nodelist, mapping = kernels.graph_sampling(indptr, indices, n_samples=20, n_hops=1, seed=3)
    assert nodelist == sorted(set(nodelist)) and len(nodelist) >= 20
    assert len(mapping) == n
    assert [mapping[u] for u in nodelist] == list(range(len(nodelist)))
    assert sum(m == -1 for m in mapping) == n - len(nodelist)
    again = kernels.graph_sampling(indptr, indices, n_samples=20, n_hops=1, seed=3)
    assert again == [nodelist, mapping]
    unseeded = kernels.graph_sampling(torch.tensor(indptr), torch.tensor(indices), 20, 2)
    assert len(unseeded[0]) >= 20
