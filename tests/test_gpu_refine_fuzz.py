"""Seeded sweep of the device refine over random graphs and shapes: every
heap size of the ladder, row lengths 8..768 with odd and even group counts,
any d_principle, candidate lists / buffers / outputs shorter and longer than
the heap, unused and repeated candidates, ragged rows, self loops, repeats.
Bar: the oracle's `traverse_refine` on the same inputs — completed distances,
buffer and top-k bit-identical, ids up to exact ties."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import assert_same_search

pytestmark = pytest.mark.gpu

EF_SEARCH = [1, 5, 16, 20, 32, 48, 64, 80, 128, 150, 256, 300, 512, 700, 2048]
D = [8, 16, 24, 40, 64, 96, 128, 136, 200, 256, 768]


def random_rows(g, n_rows, n_ids, ids, deg):
    """[n_rows, deg] neighbour lists over `ids` (a sorted id tensor), biased
    to a window so that rows repeat ids and hit their own node; ragged."""
    pos = torch.arange(n_rows).unsqueeze(1) + torch.randint(-20, 21, (n_rows, deg), generator=g)
    far = torch.randint(n_ids, (n_rows, deg), generator=g)
    pick = torch.rand(n_rows, deg, generator=g) < 0.5
    nbr = ids[torch.where(pick, pos.clamp(0, n_ids - 1), far)]
    length = torch.randint(0, deg + 1, (n_rows, 1), generator=g)
    nbr[torch.arange(deg).unsqueeze(0) >= length] = -1
    return nbr


def make_case(seed):
    r = np.random.RandomState(seed)
    g = torch.Generator().manual_seed(seed)
    n = int(r.randint(300, 4000))
    n_sub = max(8, int(n * float(r.choice([0.2, 0.5, 1.0]))))
    d = int(r.choice(D))
    dp = 8 * int(r.randint(1, d // 8 + 1))
    deg_sub = int(r.choice([1, 3, 16, 31, 32, 48, 64]))
    deg_full = int(r.choice([2, 7, 24, 32, 33, 64]))
    ef_search = int(r.choice(EF_SEARCH))
    n_init = int(r.choice([1, 7, 64, 100, 256, 300]))
    n_buffers = n_init if r.rand() < 0.5 else int(r.choice([1, 16, 64, 130, 512]))
    k = int(r.choice([1, 10, 33, 100]))
    B = int(r.randint(1, 60))
    nodelist = torch.randperm(n, generator=g)[:n_sub].sort().values
    mapping = torch.full((n,), -1, dtype=torch.long)
    mapping[nodelist] = torch.arange(n_sub)
    sub = random_rows(g, n_sub, n_sub, nodelist, deg_sub)
    rowlen = torch.zeros(n, dtype=torch.long)
    rowlen[nodelist] = deg_sub
    sub_indptr = torch.zeros(n + 1, dtype=torch.long)
    sub_indptr[1:] = torch.cumsum(rowlen, 0)
    full = random_rows(g, n, n, torch.arange(n), deg_full)
    full_indptr = torch.arange(n + 1, dtype=torch.long) * deg_full
    x = torch.randn(n, d, generator=g)
    query = torch.randn(B, d, generator=g)
    cand = torch.randint(n, (B, n_init), generator=g)
    if r.rand() < 0.5:
        cand = nodelist[torch.randint(n_sub, (B, n_init), generator=g)]
    cand[torch.rand(B, n_init, generator=g) < 0.1] = -1
    return dict(seed=seed, n=n, n_sub=n_sub, d=d, dp=dp, deg_sub=deg_sub,
                deg_full=deg_full, ef_search=ef_search, n_init=n_init,
                n_buffers=n_buffers, k=k, B=B, nodelist=nodelist,
                mapping=mapping, sub_indptr=sub_indptr,
                sub_indices=sub.flatten().contiguous(), full_indptr=full_indptr,
                full_indices=full.flatten().contiguous(), x=x, query=query,
                cand=cand.contiguous())


@pytest.mark.parametrize('seed', range(80))
def test_random_refine(seed, device):
    c = make_case(5000 + seed)
    print('refine fuzz', {k: c[k] for k in ('seed', 'n', 'n_sub', 'd', 'dp',
                                            'deg_sub', 'deg_full', 'ef_search',
                                            'n_init', 'n_buffers', 'k', 'B')},
          flush=True)
    B, d, dp = c['B'], c['d'], c['dp']
    xn, qn = c['x'].numpy(), c['query'].numpy()
    x_dp = np.ascontiguousarray(xn[:, :dp])
    cand_D = torch.from_numpy(np.stack([
        oracle.square_dist(np.ascontiguousarray(qn[b, :dp]), x_dp,
                           c['cand'][b].clamp(min=0).numpy().copy())
        for b in range(B)]))
    alias = c['n_buffers'] == c['n_init']

    ref_init_I, ref_init_D = c['cand'].numpy().copy(), cand_D.numpy().copy()
    if alias:
        ref_buf_I, ref_buf_D = ref_init_I, ref_init_D
    else:
        ref_buf_I = np.empty((B, c['n_buffers']), np.int64)
        ref_buf_D = np.empty((B, c['n_buffers']), np.float32)
    ref_I = np.empty((B, c['k']), np.int64)
    ref_D = np.empty((B, c['k']), np.float32)
    oracle.traverse_refine(
        ref_I, ref_D, ref_buf_I, ref_buf_D, ref_init_I, ref_init_D,
        [c['sub_indptr'].numpy(), c['sub_indices'].numpy()],
        [c['full_indptr'].numpy(), c['full_indices'].numpy()], xn, qn,
        c['ef_search'], dp)

    sub = kernels.prepare_graph(c['sub_indptr'].to(device), c['sub_indices'].to(device),
                                c['mapping'].to(device), c['n_sub'], c['deg_sub'])
    full = kernels.prepare_full_graph(c['full_indptr'].to(device),
                                      c['full_indices'].to(device), c['deg_full'])
    init_I, init_D = c['cand'].to(device), cand_D.to(device)
    if alias:
        buf_I, buf_D = init_I, init_D
    else:
        buf_I = torch.empty(B, c['n_buffers'], dtype=torch.long, device=device)
        buf_D = torch.empty(B, c['n_buffers'], dtype=torch.float, device=device)
    out_I = torch.empty(B, c['k'], dtype=torch.long, device=device)
    out_D = torch.empty(B, c['k'], dtype=torch.float, device=device)
    kernels.traverse_refine_cuda(out_I, out_D, buf_I, buf_D, init_I, init_D, sub,
                                 full, kernels.PreparedRows(c['x'].to(device)),
                                 c['query'].to(device), c['ef_search'], dp)
    torch.cuda.synchronize()
    if not alias:
        assert np.array_equal(init_D.cpu().numpy(), ref_init_D)
    assert_same_search(buf_I.cpu().numpy(), buf_D.cpu().numpy(), ref_buf_I, ref_buf_D)
    assert_same_search(out_I.cpu().numpy(), out_D.cpu().numpy(), ref_I, ref_D)


def test_full_buckets_and_reused_wavefronts(device):
    """Many marks per query on a graph of 50 000 nodes: buckets of the LDS
    visited table fill up and the device bitmask takes over; more queries than
    resident wavefronts, so a wavefront starts its next query after one that
    used its bitmask slice."""
    n, n_sub, d, dp, deg, ef_search, n_init, k, B = 50_000, 20_000, 16, 8, 32, 128, 64, 10, 7000
    g = torch.Generator().manual_seed(77)
    nodelist = torch.randperm(n, generator=g)[:n_sub].sort().values
    mapping = torch.full((n,), -1, dtype=torch.long)
    mapping[nodelist] = torch.arange(n_sub)
    sub = random_rows(g, n_sub, n_sub, nodelist, deg)
    rowlen = torch.zeros(n, dtype=torch.long)
    rowlen[nodelist] = deg
    sub_indptr = torch.zeros(n + 1, dtype=torch.long)
    sub_indptr[1:] = torch.cumsum(rowlen, 0)
    full = random_rows(g, n, n, torch.arange(n), deg)
    full_indptr = torch.arange(n + 1, dtype=torch.long) * deg
    x = torch.randn(n, d, generator=g)
    query = torch.randn(B, d, generator=g)
    cand = nodelist[torch.randint(n_sub, (B, n_init), generator=g)].contiguous()
    xn, qn = x.numpy(), query.numpy()
    cand_D = torch.from_numpy(np.stack([
        oracle.square_dist(np.ascontiguousarray(qn[b, :dp]),
                           np.ascontiguousarray(xn[:, :dp]), cand[b].numpy().copy())
        for b in range(B)]))
    ref_buf_I, ref_buf_D = cand.numpy().copy(), cand_D.numpy().copy()
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_refine(ref_I, ref_D, ref_buf_I, ref_buf_D, ref_buf_I, ref_buf_D,
                           [sub_indptr.numpy(), sub.flatten().numpy()],
                           [full_indptr.numpy(), full.flatten().numpy()], xn, qn,
                           ef_search, dp)
    sub_g = kernels.prepare_graph(sub_indptr.to(device), sub.flatten().contiguous().to(device),
                                  mapping.to(device), n_sub, deg)
    full_g = kernels.prepare_full_graph(full_indptr.to(device),
                                        full.flatten().contiguous().to(device), deg)
    buf_I, buf_D = cand.to(device), cand_D.to(device)
    out_I = torch.empty(B, k, dtype=torch.long, device=device)
    out_D = torch.empty(B, k, dtype=torch.float, device=device)
    counters = torch.zeros(6, dtype=torch.long, device=device)
    kernels.traverse_refine_cuda(out_I, out_D, buf_I, buf_D, buf_I, buf_D, sub_g, full_g,
                                 kernels.PreparedRows(x.to(device)), query.to(device),
                                 ef_search, dp, counters=counters)
    torch.cuda.synchronize()
    assert_same_search(buf_I.cpu().numpy(), buf_D.cpu().numpy(), ref_buf_I, ref_buf_D)
    assert_same_search(out_I.cpu().numpy(), out_D.cpu().numpy(), ref_I, ref_D)
    # far more marks per query than the table's 4096 slots can hold evenly
    assert counters[2].item() / B > 1500
