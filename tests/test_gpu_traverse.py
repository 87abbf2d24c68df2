"""GPU traversal against the CPU oracle on identical graph, entries and
reduced vectors.  Bar: distances bit-identical, ids identical except within
exact distance ties (tests/common.py:assert_same_search)."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import Problem, assert_same_search

pytestmark = pytest.mark.gpu


def run_gpu(p, dp, ef, init_I, init_D, device, counters=False):
    B = p.query.size(0)
    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    cnt = torch.zeros(5, dtype=torch.long, device=device) if counters else None
    storage = p.x[p.nodelist][:, :dp].contiguous().to(device)
    kernels.traverse_cuda(
        output_I=out_I, output_D=out_D,
        indptr=p.sub_indptr.to(device), indices=p.sub_indices.to(device),
        mapping=p.mapping.to(device), storage=storage,
        query=p.query[:, :dp].contiguous().to(device),
        initial_I=init_I.to(device), initial_D=init_D.to(device),
        n_neighbors=p.deg, counters=cnt)
    torch.cuda.synchronize()
    return (out_I.flatten(1).cpu().numpy(), out_D.flatten(1).cpu().numpy(),
            None if cnt is None else cnt.cpu().numpy())


def run_oracle(p, dp, ef, init_I, init_D, counters=None):
    B = p.query.size(0)
    k = 4 * ef
    out_I = np.empty((B, k), np.int64)
    out_D = np.empty((B, k), np.float32)
    oracle.traverse_cpu(
        out_I, out_D, init_I.numpy().copy(), init_D.numpy().copy(),
        p.sub_indptr.numpy(), p.sub_indices.numpy(),
        np.ascontiguousarray(p.x[:, :dp].numpy()),
        np.ascontiguousarray(p.query[:, :dp].numpy()), k, counters)
    return out_I, out_D


CASES = [
    # n, d, dp, deg, graph, ratio, ef, n_init, reference-style padding
    (4000, 32, 32, 32, 'nsw', 0.25, 16, 32, False),
    (4000, 32, 32, 32, 'nsg', 0.25, 64, 32, True),
    (6000, 64, 32, 32, 'nsw', 0.5, 8, 64, False),
    (6000, 96, 64, 48, 'nsg', 0.25, 32, 32, False),
    (8000, 128, 128, 64, 'nsw', 0.25, 64, 64, True),
    (3000, 64, 40, 24, 'nsw', None, 24, 16, False),
    (5000, 64, 64, 64, 'nsw', 0.5, 128, 64, False),
    (5000, 32, 32, 32, 'nsw', 0.5, 512, 32, False),
    # the instantiations the benchmark times, on graphs large enough for the
    # lists to fill: the headline configuration's (128-float rows, 64
    # neighbours, 64 entries, ef 32: traverse_kernel<128, 16>) and those of
    # the 96-dimensional one (64-float rows, 32 neighbours, 32 entries, ef 64
    # and 128: <256, 8> and <512, 8>)
    (24000, 128, 128, 64, 'nsw', 0.25, 32, 64, False),
    (24000, 96, 64, 32, 'nsw', 0.25, 64, 32, False),
    (24000, 96, 64, 32, 'nsw', 0.25, 128, 32, False),
]


@pytest.mark.parametrize('case', CASES, ids=[str(c) for c in CASES])
def test_traverse_matches_oracle(case, device):
    n, d, dp, deg, gtype, ratio, ef, n_init, pad = case
    print('case', case, flush=True)
    p = Problem(n=n, d=d, deg=deg, graph_type=gtype, sample_ratio=ratio,
                seed=n + ef, n_query=96, pad_like_reference=pad)
    init_I, init_D = p.entries(n_init, seed=5, dp=dp)
    I_ref, D_ref = run_oracle(p, dp, ef, init_I, init_D)
    I_gpu, D_gpu, _ = run_gpu(p, dp, ef, init_I, init_D, device)
    assert_same_search(I_gpu, D_gpu, I_ref, D_ref)
    # layout: best first, unused slots -1 / +inf at the end
    finite = np.isfinite(D_gpu)
    assert (D_gpu[:, 1:] >= D_gpu[:, :-1]).all()
    assert ((I_gpu >= 0) == finite).all()


def test_counters_match_oracle(device):
    p = Problem(n=5000, d=64, deg=32, sample_ratio=0.25, seed=11, n_query=128)
    init_I, init_D = p.entries(32, seed=6, dp=32, sampled_only=True)
    ref = np.zeros(5, np.int64)
    I_ref, D_ref = run_oracle(p, 32, 16, init_I, init_D, ref)
    I_gpu, D_gpu, cnt = run_gpu(p, 32, 16, init_I, init_D, device, True)
    assert_same_search(I_gpu, D_gpu, I_ref, D_ref)
    # expansions, distance evaluations and admissions are the same events
    assert cnt[0] == ref[0] and cnt[2] == ref[2] and cnt[3] == ref[3]
    assert cnt[4] == 128 * 64


def test_duplicate_and_unused_entries(device):
    p = Problem(n=3000, d=32, deg=32, sample_ratio=0.5, seed=3, n_query=64)
    init_I, init_D = p.entries(16, seed=7)
    init_I[:, 3] = init_I[:, 2]
    init_D[:, 3] = init_D[:, 2]
    init_I[:, 5] = -1
    I_ref, D_ref = run_oracle(p, 32, 8, init_I, init_D)
    I_gpu, D_gpu, _ = run_gpu(p, 32, 8, init_I, init_D, device)
    assert_same_search(I_gpu, D_gpu, I_ref, D_ref)


def test_repeat_is_deterministic_and_reuses_workspace(device):
    p = Problem(n=4000, d=32, deg=32, sample_ratio=0.25, seed=21, n_query=200)
    init_I, init_D = p.entries(32, seed=8)
    a = run_gpu(p, 32, 32, init_I, init_D, device)
    b = run_gpu(p, 32, 32, init_I, init_D, device)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_argument_errors(device):
    p = Problem(n=2000, d=32, deg=32, sample_ratio=0.5, seed=4, n_query=8)
    init_I, init_D = p.entries(8, seed=1)
    args = dict(
        output_I=torch.empty(8, 4, 16, dtype=torch.long, device=device),
        output_D=torch.empty(8, 4, 16, dtype=torch.float, device=device),
        indptr=p.sub_indptr.to(device), indices=p.sub_indices.to(device),
        mapping=p.mapping.to(device),
        storage=p.x[p.nodelist].contiguous().to(device),
        query=p.query.to(device), initial_I=init_I.to(device),
        initial_D=init_D.to(device), n_neighbors=32)
    kernels.traverse_cuda(**args)
    for key, bad in [
        ('query', args['query'].cpu()),
        ('indices', args['indices'].int()),
        ('output_I', args['output_I'][:, :2]),
        ('output_D', torch.empty(8, 4, 8, dtype=torch.float, device=device)),
        ('storage', args['storage'][:, :24]),
        ('n_neighbors', 65),
        ('initial_I', args['initial_I'][:4]),
    ]:
        with pytest.raises(RuntimeError):
            kernels.traverse_cuda(**{**args, key: bad})
    with pytest.raises(RuntimeError):
        kernels.traverse_cuda(**{
            **args,
            'output_I': torch.empty(8, 4, 1024, dtype=torch.long, device=device),
            'output_D': torch.empty(8, 4, 1024, dtype=torch.float, device=device)})
    # a row longer than n_neighbors is a malformed graph
    with pytest.raises(RuntimeError):
        kernels.traverse_cuda(**{**args, 'n_neighbors': 16})
    torch.cuda.synchronize()


def test_edge_shapes(device):
    """Empty batch, a single query, one result slot per beam, no entries,
    entries that all lack a storage row, degree 1, n_storage not a multiple
    of 32."""
    p = Problem(n=1003, d=16, deg=8, sample_ratio=0.5, seed=13, n_query=5)
    dev_args = dict(indptr=p.sub_indptr.to(device), indices=p.sub_indices.to(device),
                    mapping=p.mapping.to(device),
                    storage=p.x[p.nodelist].contiguous().to(device), n_neighbors=8)

    def run(query, init_I, init_D, ef):
        B = query.size(0)
        out_I = torch.full((B, 4, ef), -7, dtype=torch.long, device=device)
        out_D = torch.full((B, 4, ef), -7.0, dtype=torch.float, device=device)
        kernels.traverse_cuda(output_I=out_I, output_D=out_D, query=query.to(device),
                              initial_I=init_I.to(device), initial_D=init_D.to(device),
                              **dev_args)
        torch.cuda.synchronize()
        ref_I = np.empty((B, 4 * ef), np.int64)
        ref_D = np.empty((B, 4 * ef), np.float32)
        if B:
            oracle.traverse_cpu(ref_I, ref_D, init_I.numpy().copy(), init_D.numpy().copy(),
                                p.sub_indptr.numpy(), p.sub_indices.numpy(), p.x.numpy(),
                                query.numpy(), 4 * ef)
        return out_I.flatten(1).cpu().numpy(), out_D.flatten(1).cpu().numpy(), ref_I, ref_D

    init_I, init_D = p.entries(4, seed=2)
    # empty batch: nothing is launched, nothing is written
    run(p.query[:0], init_I[:0], init_D[:0], 4)
    for B, ef in [(1, 1), (5, 1), (5, 3), (3, 5)]:
        I, D, rI, rD = run(p.query[:B], init_I[:B], init_D[:B], ef)
        assert_same_search(I, D, rI, rD)
    # no entries at all: every slot stays empty
    none_I = torch.empty(5, 0, dtype=torch.long)
    none_D = torch.empty(5, 0)
    I, D, rI, rD = run(p.query, none_I, none_D, 2)
    assert (I == -1).all() and np.isposinf(D).all()
    assert_same_search(I, D, rI, rD)
    # entries without a storage row only: they are popped, expanded to
    # nothing and merged at the end
    outside = torch.nonzero(p.mapping < 0).flatten()[:6]
    lone_I = outside.unsqueeze(0).expand(5, -1).contiguous()
    lone_D = (p.query.unsqueeze(1) - p.x[lone_I]).square().sum(-1).contiguous()
    I, D, rI, rD = run(p.query, lone_I, lone_D, 2)
    assert_same_search(I, D, rI, rD)
    assert sorted(I[0][:6].tolist()) == sorted(outside.tolist())


def test_degree_one_chain(device):
    """A chain with one neighbour per node and the query beyond its end: the
    iteration cap min(1024, 2 * 4 * ef) decides how far the search gets
    (traverse_cpu.cpp:18,82)."""
    n, ef = 300, 8
    indptr = torch.arange(n + 1)
    indices = torch.cat([torch.arange(1, n), torch.tensor([-1])])
    x = torch.zeros(n, 8)
    x[:, 0] = torch.arange(n).float()
    q = torch.zeros(1, 8)
    q[0, 0] = n + 10.0
    out_I = torch.empty(1, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(1, 4, ef, dtype=torch.float, device=device)
    kernels.traverse_cuda(out_I, out_D, indptr.to(device), indices.to(device),
                          torch.arange(n).to(device), x.to(device), q.to(device),
                          torch.zeros(1, 1, dtype=torch.long, device=device),
                          torch.full((1, 1), float((n + 10) ** 2), device=device), 1)
    cap = 2 * 4 * ef
    assert out_I.flatten().tolist() == [cap - i for i in range(4 * ef)]


def test_row_order_does_not_change_results(device):
    """The storage rows may be laid out in any order (``mapping`` says which
    row a node has): same ids, same distances, bit for bit."""
    p = Problem(n=6000, d=64, deg=32, sample_ratio=0.5, seed=31, n_query=80)
    init_I, init_D = p.entries(32, seed=9, dp=64)
    I_a, D_a, _ = run_gpu(p, 64, 32, init_I, init_D, device)
    from pilotann_amd import utils
    rows = p.x[p.nodelist]
    for order in (torch.randperm(rows.size(0), generator=torch.Generator().manual_seed(1)),
                  utils.locality_order(rows, seed=2)):
        place = torch.empty_like(order)
        place[order] = torch.arange(order.numel())
        mapping = p.mapping.clone()
        mapping[p.mapping >= 0] = place[p.mapping[p.mapping >= 0]]
        out_I = torch.empty(80, 4, 32, dtype=torch.long, device=device)
        out_D = torch.empty(80, 4, 32, dtype=torch.float, device=device)
        kernels.traverse_cuda(
            output_I=out_I, output_D=out_D, indptr=p.sub_indptr.to(device),
            indices=p.sub_indices.to(device), mapping=mapping.to(device),
            storage=rows[order].contiguous().to(device),
            query=p.query.contiguous().to(device), initial_I=init_I.to(device),
            initial_D=init_D.to(device), n_neighbors=p.deg)
        torch.cuda.synchronize()
        assert np.array_equal(out_I.flatten(1).cpu().numpy(), I_a)
        assert np.array_equal(out_D.flatten(1).cpu().numpy(), D_a)


def test_rows_outside_indices_are_reported_not_read(device):
    """A row whose start or end lies outside `indices` (a damaged checkpoint)
    sets status bit 8 and is treated as empty; nothing outside the array is
    read."""
    p = Problem(n=2000, d=32, deg=32, sample_ratio=0.5, seed=4, n_query=8)
    n_storage = p.nodelist.numel()
    for damage in ('start beyond the end', 'negative start', 'end beyond the end'):
        print('damaged indptr:', damage, flush=True)
        indptr = p.sub_indptr.clone()
        node = int(p.nodelist[n_storage // 2])
        if damage == 'start beyond the end':
            indptr[node] = indptr[-1] + (1 << 40)
            indptr[node + 1] = indptr[node] + 32
        elif damage == 'negative start':
            indptr[node] = -(1 << 40)
            indptr[node + 1] = indptr[node] + 32
        else:
            node = int(p.nodelist[-1])   # a row that straddles the end
            indptr[node] = p.sub_indices.numel() - 16
            indptr[node + 1:] = indptr[node] + 32
        with pytest.raises(RuntimeError, match='status bits'):
            kernels.PreparedGraph(indptr.to(device), p.sub_indices.to(device),
                                  p.mapping.to(device), n_storage, 32)
    torch.cuda.synchronize()


def hand_built(rows, coords, entries, entry_d, ef_total, device, width=None):
    """A search on a hand-built graph whose nodes sit on the first axis, as in
    tests/test_oracle_traverse.py: returns the device's and the oracle's row."""
    width = width or max(1, max(len(r) for r in rows))
    n = len(rows)
    indptr = torch.arange(n + 1, dtype=torch.long) * width
    indices = torch.full((n * width,), -1, dtype=torch.long)
    for i, r in enumerate(rows):
        indices[i * width:i * width + len(r)] = torch.tensor(r, dtype=torch.long)
    x = torch.zeros(n, 8)
    x[:, 0] = torch.tensor(coords)
    q = torch.zeros(1, 8)
    init_I = torch.tensor([entries], dtype=torch.long)
    init_D = torch.tensor([entry_d], dtype=torch.float)
    ef = ef_total // 4
    out_I = torch.empty(1, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(1, 4, ef, dtype=torch.float, device=device)
    kernels.traverse_cuda(out_I, out_D, indptr.to(device), indices.to(device),
                          torch.arange(n).to(device), x.to(device), q.to(device),
                          init_I.to(device), init_D.to(device), width)
    torch.cuda.synchronize()
    ref_I = np.empty((1, ef_total), np.int64)
    ref_D = np.empty((1, ef_total), np.float32)
    oracle.traverse_cpu(ref_I, ref_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        indptr.numpy(), indices.numpy(), x.numpy(), q.numpy(),
                        ef_total)
    return (out_I.flatten().tolist(), out_D.flatten().tolist(),
            ref_I[0].tolist(), ref_D[0].tolist())


def test_hand_built_rules_on_the_device(device):
    """The hand-derived cases that pin the oracle's rules
    (tests/test_oracle_traverse.py), run on the device with the expected
    outputs stated again: an open list of exactly 2 * 16 cells, the gate in
    front of the open list, and the stop on a key equal to the worst kept."""
    inf = float('inf')
    # open list of 32 cells: the entries with keys 9 and 10 survive, 11 is dropped
    coords = [1, 3, 2, 5, 4, 7, 6, 9, 8, 10, 11]
    rows = [[] for _ in range(14)]
    rows[7], rows[9], rows[10] = [11], [12], [13]
    I, D, rI, rD = hand_built(rows, [float(c) for c in coords] + [0.5, 0.25, 0.125],
                              list(range(11)), [float(c * c) for c in coords], 16, device)
    assert I == [12, 11, 0, 2, 1, 4, 3, 6, 5, 8, 7, 9, 10, -1, -1, -1] == rI
    assert D == [0.0625, 0.25] + [float(c * c) for c in range(1, 12)] + [inf] * 3 == rD
    # a candidate tying with the worst kept stays out of the open list
    a = [40.0] + [float(c) for c in range(30, 21, -1)]
    r = [float(c) for c in range(1, 8)]
    coords = a + r + [-30.0, 10.0, -10.0, 8.0, 0.5]
    rows = [[i + 1] for i in range(9)] + [list(range(10, 17)) + [17, 18, 19, 20]]
    rows += [[] for _ in range(12)]
    rows[18] = [21]
    I, D, rI, rD = hand_built(rows, coords, [0], [1600.0], 16, device)
    assert I[:8] == list(range(10, 17)) + [20] and sorted(I[8:10]) == [18, 19]
    assert I[10:] == [9, 8, 7, 6, 5, 4] and D == rD
    assert sorted(I) == sorted(rI)
    # a popped key equal to the worst kept ends the search
    coords = [1.0, -16.0] + [float(c) for c in range(16, 1, -1)] + [1.5, 0.5]
    rows = [list(range(2, 18)), [18]] + [[] for _ in range(17)]
    I, D, rI, rD = hand_built(rows, coords, [0, 1], [1.0, 256.0], 16, device)
    assert I == [0, 17] + list(range(16, 2, -1)) == rI
    assert D == [1.0, 2.25] + [float(c * c) for c in range(2, 16)] == rD
