"""The wide mode of the traversal (`pa_traverse_wide`): a labelled throughput
mode, not the host search step for step.  What is promised and checked here:
the distance returned for an id is bit for bit the oracle's distance of that
id; rows are best first with -1 / +inf at the end and no id twice; the set of
candidates is as good as the exact mode's (recall of the true nearest
neighbours in the reduced space within a small margin, on average not below);
and, id for id, the search is the one `oracle.traverse_wide` restates on the
CPU (a pool of the best candidates, the `width` best open ones expanded
together)."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels, utils
from common import Problem, assert_same_search

pytestmark = pytest.mark.gpu


def run(p, dp, ef, init_I, init_D, device, mode, width=4, counters=False):
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
        n_neighbors=p.deg, counters=cnt, mode=mode, width=width)
    torch.cuda.synchronize()
    return (out_I.flatten(1).cpu().numpy(), out_D.flatten(1).cpu().numpy(),
            None if cnt is None else cnt.cpu().numpy())


def reduced_recall(p, dp, I, k=10):
    """Share of the k nearest sampled nodes (first dp coordinates) found."""
    rows = p.x[p.nodelist][:, :dp]
    target = p.nodelist[utils.brute_force_topk(p.query[:, :dp], rows, k)]
    return utils.recall(torch.from_numpy(I[:, :k].copy()), target)


CASES = [
    # n, d, dp, deg, graph, ratio, ef, n_init, width
    (4000, 32, 32, 32, 'nsw', 0.25, 16, 32, 4),
    (6000, 64, 32, 32, 'nsw', 0.5, 8, 64, 2),
    (6000, 96, 64, 48, 'nsg', 0.25, 32, 32, 4),
    (8000, 128, 128, 64, 'nsw', 0.25, 64, 64, 4),
    (3000, 64, 40, 24, 'nsw', None, 24, 16, 3),
    (5000, 64, 64, 64, 'nsw', 0.5, 128, 64, 4),
    (5000, 32, 32, 32, 'nsw', 0.5, 512, 32, 4),
    (24000, 128, 128, 64, 'nsw', 0.25, 32, 64, 4),
    (24000, 96, 64, 32, 'nsw', 0.25, 64, 32, 1),
]


@pytest.mark.parametrize('case', CASES, ids=[str(c) for c in CASES])
def test_wide_mode_properties(case, device):
    n, d, dp, deg, gtype, ratio, ef, n_init, width = case
    print('wide case', case, flush=True)
    p = Problem(n=n, d=d, deg=deg, graph_type=gtype, sample_ratio=ratio,
                seed=n + ef, n_query=96)
    init_I, init_D = p.entries(n_init, seed=5, dp=dp)
    I, D, cnt = run(p, dp, ef, init_I, init_D, device, 'wide', width, True)
    xr = np.ascontiguousarray(p.x[:, :dp].numpy())
    qr = np.ascontiguousarray(p.query[:, :dp].numpy())
    for b in range(I.shape[0]):
        real = I[b] >= 0
        # best first, padding at the end only
        assert (D[b][1:] >= D[b][:-1]).all()
        assert real[:real.sum()].all() and np.isinf(D[b][~real]).all()
        # every distance is the oracle's distance of that id, bit for bit
        assert np.array_equal(D[b][real], oracle.square_dist(qr[b], xr, I[b][real].copy()))
        # an id twice only if the entries named it twice
        ids, counts = np.unique(I[b][real], return_counts=True)
        twice = set(ids[counts > 1].tolist())
        assert twice <= set(init_I[b].tolist())
    # id for id the search the oracle restates (ties aside)
    k = 4 * ef
    I_ref = np.empty((I.shape[0], k), np.int64)
    D_ref = np.empty((I.shape[0], k), np.float32)
    ref = np.zeros(5, np.int64)
    oracle.traverse_wide(I_ref, D_ref, init_I.numpy().copy(), init_D.numpy().copy(),
                         p.sub_indptr.numpy(), p.sub_indices.numpy(),
                         p.mapping.numpy(), xr, qr, width, ref)
    assert_same_search(I, D, I_ref, D_ref)
    assert cnt[0] == ref[0] and cnt[2] == ref[2] and cnt[3] == ref[3]
    # the candidates are as good as the exact mode's
    I_exact, D_exact, _ = run(p, dp, ef, init_I, init_D, device, 'exact')
    r_wide, r_exact = reduced_recall(p, dp, I), reduced_recall(p, dp, I_exact)
    print('recall@10 in the reduced space: wide', r_wide, 'exact', r_exact,
          'expansions per query', cnt[0] / I.shape[0], flush=True)
    assert r_wide >= r_exact - 0.01
    assert cnt[4] == I.shape[0] * 4 * ef and cnt[0] > 0


def test_wide_mode_argument_errors(device):
    p = Problem(n=2000, d=32, deg=32, sample_ratio=0.5, seed=4, n_query=8)
    init_I, init_D = p.entries(8, seed=1)
    with pytest.raises(RuntimeError):
        run(p, 32, 16, init_I, init_D, device, 'wide', width=5)
    with pytest.raises(RuntimeError):
        run(p, 32, 16, init_I, init_D, device, 'fast')
    # unused and unsampled entries, an empty batch
    init_I[:, 3] = -1
    I, D, _ = run(p, 32, 16, init_I, init_D, device, 'wide')
    assert (I[:, 0] >= 0).all()
    empty = torch.empty(0, 4, 16, dtype=torch.long, device=device)
    kernels.traverse_cuda(
        empty, torch.empty(0, 4, 16, device=device), p.sub_indptr.to(device),
        p.sub_indices.to(device), p.mapping.to(device),
        p.x[p.nodelist].contiguous().to(device), torch.empty(0, 32, device=device),
        torch.empty(0, 8, dtype=torch.long, device=device),
        torch.empty(0, 8, device=device), 32, mode='wide')
    torch.cuda.synchronize()


@pytest.mark.parametrize('seed', range(60))
def test_wide_mode_on_random_graphs(seed, device):
    """The random graphs of the exact mode's sweep (every pool size, vector
    lengths with and without a specialised kernel, degrees 1..64, ragged
    rows, self loops, repeated and unsampled neighbours and entries, exact
    ties), widths 1..4, against the CPU restatement."""
    from test_gpu_fuzz import make_case
    c = make_case(5000 + seed)
    width = 1 + seed % 4
    print('wide fuzz', {k: c[k] for k in ('seed', 'n_nodes', 'n_rows', 'deg', 'dp', 'ef',
                                          'n_init', 'B', 'tied', 'unsampled_neighbours')},
          'width', width, flush=True)
    B, k = c['B'], 4 * c['ef']
    xn, qn = c['x'].numpy(), c['query'].numpy()
    init_D = np.stack([oracle.square_dist(qn[b].copy(), xn, c['init_I'][b].numpy().copy())
                       for b in range(B)])
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    ref = np.zeros(5, np.int64)
    oracle.traverse_wide(ref_I, ref_D, c['init_I'].numpy().copy(), init_D.copy(),
                         c['indptr'].numpy(), c['indices'].numpy(), c['mapping'].numpy(),
                         xn, qn, width, ref)
    out_I = torch.empty(B, 4, c['ef'], dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, c['ef'], dtype=torch.float, device=device)
    cnt = torch.zeros(5, dtype=torch.long, device=device)
    kernels.traverse_cuda(
        output_I=out_I, output_D=out_D, indptr=c['indptr'].to(device),
        indices=c['indices'].to(device), mapping=c['mapping'].to(device),
        storage=c['x'][c['nodelist']].contiguous().to(device),
        query=c['query'].to(device), initial_I=c['init_I'].to(device),
        initial_D=torch.from_numpy(init_D).to(device), n_neighbors=c['deg'],
        counters=cnt, mode='wide', width=width)
    torch.cuda.synchronize()
    got_I = out_I.flatten(1).cpu().numpy()
    got_D = out_D.flatten(1).cpu().numpy()
    if not c['tied']:
        # a chance tie at the worst kept distance may keep another member
        def at_that_distance(b, ids, dist):
            assert np.array_equal(oracle.square_dist(qn[b].copy(), xn, ids.copy()),
                                  np.full(len(ids), dist, np.float32))
        assert_same_search(got_I, got_D, ref_I, ref_D, worst_tie=at_that_distance)
        cnt = cnt.cpu().numpy()
        assert cnt[2] == ref[2] and cnt[3] == ref[3]
        # An entry named twice sits in the pool twice, and its second copy is
        # expanded too, to no effect; whether that copy is still in the pool
        # when its turn comes can depend on the order inside the tie (the two
        # are equal but for the flag).  Expansions agree up to those copies.
        repeats = sum(len(row) - len(set(row)) for row in c['init_I'].tolist())
        assert abs(int(cnt[0]) - int(ref[0])) <= repeats
        return
    # exact ties: which of several equally distant candidates is expanded or
    # kept first may differ (the order inside a tie is by storage row, and the
    # flag of an expanded entry takes part in it); every id must still carry
    # its own exact distance, best first
    for b in range(B):
        real = got_I[b] >= 0
        assert (got_D[b][1:] >= got_D[b][:-1]).all()
        assert np.array_equal(got_D[b][real],
                              oracle.square_dist(qn[b].copy(), xn, got_I[b][real].copy()))
