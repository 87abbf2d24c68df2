"""The fused nearest-neighbour kernel of the graph builder (`pa_knn`,
`kernels.knn_candidates`, the device path of `utils.knn_graph`) against an
exact float64 ranking.  The kernel ranks with half-precision products, so
what is asserted is that the exact neighbours are among its candidates and
that the builder's table, which ranks the candidates again in float32, is
the exact one up to ties."""
import ctypes

import pytest
import torch

from pilotann_amd import _lib, kernels, utils
from pilotann_amd.utils import graphs

pytestmark = pytest.mark.gpu


def exact_neighbours(query, base, k, exclude_self=False):
    d = torch.cdist(query.double(), base.double())
    if exclude_self:
        d.fill_diagonal_(float('inf'))
    return torch.topk(d, k, dim=-1, largest=False)


def overlap(got, want):
    hits = sum(len(set(a) & set(b)) for a, b in zip(got.tolist(), want.tolist()))
    return hits / want.numel()


@pytest.mark.parametrize('n,d,k', [
    (129, 8, 5), (1000, 64, 10), (5000, 72, 47), (5000, 72, 48),
    (20000, 96, 64), (3000, 200, 111), (3000, 200, 127), (12345, 768, 80),
    (9000, 64, 240), (3000, 128, 496), (3000, 128, 497), (2000, 192, 20), (700, 50, 9),
])
def test_knn_table_is_the_exact_one(n, d, k, device):
    print('knn case', n, d, k, flush=True)
    x = utils.gaussian_mixture(n, d, 16, 1.0, seed=n + d, normalize=(d > 100),
                               decay=0.5).to(device)
    ids, d2 = utils.knn_graph(x, k)          # the kernel for n > 128 and k <= 496
    torch.cuda.synchronize()
    assert ids.shape == (n, k) and d2.shape == (n, k)
    assert ids.dtype == torch.long and int(ids.min()) >= 0 and int(ids.max()) < n
    assert not bool((ids == torch.arange(n, device=device).unsqueeze(-1)).any())
    assert bool((d2[:, 1:] >= d2[:, :-1]).all())
    rows = slice(0, min(n, 1500))
    want = exact_neighbours(x[rows], x, k + 1)
    # drop the row itself from the exact ranking (first place, distance 0)
    keep = want.indices != torch.arange(rows.stop, device=device).unsqueeze(-1)
    want_ids = want.indices[keep].view(rows.stop, k)
    want_d = want.values[keep].view(rows.stop, k)
    # the same distances place for place (ids may swap inside exact ties)
    assert torch.allclose(d2[rows].double().sqrt(), want_d, rtol=1e-5, atol=1e-6)
    assert overlap(ids[rows], want_ids) > 0.9999
    # distances are those of the ids returned
    back = (x[ids[:64]] - x[:64].unsqueeze(1)).square().sum(-1)
    assert torch.allclose(back, d2[:64], rtol=1e-5, atol=1e-6)


def test_the_device_table_agrees_with_the_host_path(device):
    x = utils.gaussian_mixture(4000, 64, 8, 1.0, seed=5, decay=0.5)
    host_ids, host_d = utils.knn_graph(x, 20)
    dev_ids, dev_d = utils.knn_graph(x.to(device), 20)
    assert torch.allclose(host_d, dev_d.cpu(), rtol=1e-4, atol=1e-5)
    assert overlap(dev_ids.cpu(), host_ids) > 0.9995


@pytest.mark.parametrize('m,n,d,keep', [
    (1, 130, 64, 64), (300, 20000, 96, 128), (257, 4000, 128, 64), (1000, 1000, 40, 128),
    (200, 9000, 64, 256), (130, 5000, 96, 512),
])
def test_candidates_of_a_few_queries_over_segments(m, n, d, keep, device):
    """Few query rows: the base rows are dealt to several workgroups per tile
    of queries and the lists merged; the exact nearest keep / 2 rows must be
    among the keep candidates."""
    print('knn candidates', m, n, d, keep, flush=True)
    g = torch.Generator().manual_seed(m + n)
    base = torch.randn(n, d, generator=g).to(device)
    query = torch.randn(m, d, generator=g).to(device)
    cand = kernels.knn_candidates(query, base, keep)
    torch.cuda.synchronize()
    assert cand.shape == (m, keep) and int(cand.max()) < n and int(cand.min()) >= 0
    srt = torch.sort(cand, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all())            # no id twice
    want = exact_neighbours(query, base, keep // 2).indices
    assert overlap(cand, want) > 0.9995
    # one segment and many give the same sets when nothing is tied
    one = kernels.knn_candidates(query, base, keep, n_seg=1)
    many = kernels.knn_candidates(query, base, keep, n_seg=min(7, -(-n // 256)))
    assert overlap(one, want) > 0.9995 and overlap(many, want) > 0.9995


def test_a_part_of_a_prepared_set_as_queries(device):
    """Query rows taken from a prepared set (a view that starts on a tile)
    against the whole set."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(3000, 64, generator=g).to(device)
    rows = kernels.HalfRows(x)
    print('knn candidates, rows 512 .. 3000 of a prepared set', flush=True)
    part = kernels.knn_candidates(rows.rows(512, 3000), rows, 64)
    torch.cuda.synchronize()
    assert part.shape == (2488, 64)
    want = exact_neighbours(x[512:], x, 32).indices
    assert overlap(part, want) > 0.9995
    with pytest.raises(RuntimeError):
        rows.rows(100, 3000)


@pytest.mark.parametrize('n,d,m,k,first', [(500, 4, 500, 7, 0), (3000, 768, 1000, 256, 512),
                                           (2000, 100, 333, 65, 1667), (300, 4096, 5, 3, 295)])
def test_exact_distances_to_candidates(n, d, m, k, first, device):
    """pa_knn_rerank: float32 distances from rows first .. first + m to their
    candidates, infinity for -1 and for the row itself."""
    print('knn rerank', n, d, m, k, first, flush=True)
    g = torch.Generator().manual_seed(n + d)
    x = torch.randn(n, d, generator=g)
    cand = torch.randint(0, n, (m, k), generator=g)
    cand[::3, 0] = -1
    cand[1::3, -1] = torch.arange(first, first + m)[1::3]          # the row itself
    got = kernels.knn_rerank(x.to(device), cand.to(device), first).cpu()
    want = (x[cand.clamp(min=0)].double() - x[first:first + m].double().unsqueeze(1)).square().sum(-1)
    skip = (cand < 0) | (cand == torch.arange(first, first + m).unsqueeze(1))
    assert bool(torch.isinf(got[skip]).all()) and bool((got[skip] > 0).all())
    assert torch.allclose(got[~skip].double(), want[~skip], rtol=2e-6, atol=0)
    with pytest.raises(RuntimeError):
        kernels.knn_rerank(x.to(device), cand.to(device), n - m + 1)
    with pytest.raises(RuntimeError):
        kernels.knn_rerank(x[:, :3].contiguous().to(device), cand.to(device), first)


def test_fewer_base_rows_than_candidates(device):
    base = torch.randn(50, 64, generator=torch.Generator().manual_seed(1)).to(device)
    cand = kernels.knn_candidates(base, base, 64)
    torch.cuda.synchronize()
    assert cand.shape == (50, 64)
    assert bool(((cand >= 0).sum(1) == 50).all())             # every row, once, then -1
    assert bool((torch.sort(cand, 1).values[:, 14:] == torch.arange(50, device=device)).all())


def test_repeated_rows_and_large_values(device):
    """Rows that occur twice are each other's nearest neighbour at distance
    zero (only the row itself is dropped); values far outside the half
    range are scaled before the conversion."""
    g = torch.Generator().manual_seed(3)
    x = 1e6 * torch.randn(2000, 64, generator=g)
    x[1000:1100] = x[:100]
    ids, d2 = utils.knn_graph(x.to(device), 8)
    assert bool((ids[:100, 0].cpu() == torch.arange(1000, 1100)).all())
    assert bool((d2[:100, 0] == 0).all())
    # differences first: the product form of cdist cancels at this scale
    exact = (x[:300].double().unsqueeze(1) - x.double().unsqueeze(0)).square().sum(-1)
    exact[torch.arange(300), torch.arange(300)] = float('inf')
    want = torch.topk(exact, 8, dim=-1, largest=False).values
    assert torch.allclose(d2[:300].cpu().double(), want, rtol=1e-5)


def test_a_few_large_coordinates_do_not_spoil_the_table(device):
    """A heavy-tailed column (a few coordinates thousands of times the rest):
    the half-precision copy is scaled by the rows' typical length, not by the
    largest coordinate, so the other coordinates keep their precision and the
    table is still the exact one for the ordinary rows."""
    n, d, k = 20000, 64, 10
    g = torch.Generator().manual_seed(31)
    x = torch.randn(n, d, generator=g)
    wild = torch.arange(0, n, 97)
    x[wild, 5] *= 5000.0
    ids, d2 = utils.knn_graph(x.to(device), k)
    tame = torch.ones(n, dtype=torch.bool)
    tame[wild] = False
    rows = torch.nonzero(tame).flatten()[:2000]
    exact = torch.cdist(x[rows].double(), x.double()).square()
    exact[torch.arange(rows.numel()), rows] = float('inf')
    want = torch.topk(exact, k, dim=-1, largest=False)
    got = ids[rows.to(device)].cpu()
    hit = (got.unsqueeze(-1) == want.indices.unsqueeze(1)).any(1).float().mean()
    print('heavy-tailed column: share of the exact table found', float(hit), flush=True)
    assert float(hit) > 0.999
    assert torch.allclose(d2[rows.to(device)].cpu().double(), want.values, rtol=1e-4)


def test_knn_argument_errors(device):
    lib = _lib.lib()
    buf = torch.zeros(1 << 16, device=device)
    p = ctypes.c_void_p(buf.data_ptr())
    none = ctypes.c_void_p(None)
    def call(m=128, n=128, d=64, keep=64, n_seg=1, q=p):
        return lib.pa_knn(p, p, p, q, p, p, m, n, d, keep, n_seg, none)
    assert call(d=72) == lib.pa_knn(p, p, p, p, p, p, 128, 128, 8, 64, 1, none) != 0   # d % 64
    assert call(keep=100) != 0
    assert call(n=0) != 0
    assert call(n_seg=0) != 0
    assert call(m=-1) != 0
    assert call(q=none) != 0
    assert call(m=0) == 0
    assert lib.pa_knn_tile_rows() == 256
    assert lib.pa_knn_list_capacity(64) == 448 and lib.pa_knn_list_capacity(128) == 512
    assert lib.pa_knn_list_capacity(512) == 896 and lib.pa_knn_list_capacity(100) == 0
    with pytest.raises(RuntimeError):
        kernels.knn_candidates(torch.zeros(4, 64), torch.zeros(200, 64, device=device), 64)
    with pytest.raises(RuntimeError):
        kernels.knn_candidates(torch.zeros(4, 32, device=device),
                               torch.zeros(200, 64, device=device), 64)


@pytest.mark.parametrize('n,k,m_keep,fill', [
    (1, 5, 3, True), (300, 64, 32, True), (300, 64, 32, False), (257, 240, 32, True),
    (100, 512, 48, False), (50, 20, 32, True), (64, 130, 64, False),
])
def test_occlusion_pruning_equals_the_step_by_step_rule(n, k, m_keep, fill, device):
    """`pa_graph_prune` against the rule written out on the host: candidates
    closest first; one is kept unless an earlier kept one is closer to it
    than the node is; `fill` tops up with the closest rejected ones."""
    print('prune case', n, k, m_keep, fill, flush=True)
    g = torch.Generator().manual_seed(n + k)
    pts = torch.randn(n, k, 6, generator=g)
    node = torch.randn(n, 1, 6, generator=g) * 0.3
    d = (pts - node).square().sum(-1)
    order = torch.argsort(d, dim=-1)
    pts = torch.gather(pts, 1, order.unsqueeze(-1).expand(-1, -1, 6))
    d = torch.gather(d, 1, order)
    pair = (pts.unsqueeze(2) - pts.unsqueeze(1)).square().sum(-1).contiguous()
    got = kernels.graph_prune(pair.to(device), d.contiguous().to(device), m_keep, fill).cpu()
    want = torch.full((n, m_keep), -1, dtype=torch.long)
    for i in range(n):
        kept, rejected = [], []
        for j in range(k):
            if len(kept) < m_keep and not any(pair[i, j, r] < d[i, j] for r in kept):
                kept.append(j)
            else:
                rejected.append(j)
        row = kept + (rejected if fill else [])
        row = row[:m_keep]
        want[i, :len(row)] = torch.tensor(row, dtype=torch.long)
    assert torch.equal(got, want)
    with pytest.raises(RuntimeError):
        kernels.graph_prune(pair[:, :, :-1].contiguous().to(device), d.to(device), m_keep, fill)


@pytest.mark.parametrize('n,d,k,m_keep,fill', [
    (3000, 64, 240, 32, True), (2000, 768, 240, 48, False), (1500, 100, 64, 16, True),
    (400, 128, 256, 32, True), (40, 64, 39, 32, True), (300, 192, 9, 4, False),
])
def test_pruning_straight_from_the_rows(n, d, k, m_keep, fill, device):
    """`pa_graph_prune_rows` against `pa_graph_prune` on the float32 table of
    pairwise distances: the same selection, except where a pair's distance and
    the candidate's own differ by less than the two-part products resolve."""
    print('prune rows case', n, d, k, m_keep, fill, flush=True)
    x = utils.gaussian_mixture(n, d, 8, 1.0, seed=n + d, decay=0.3).to(device)
    cand, cand_d = utils.knn_graph(x, k)
    if k == 39:                                   # lists that end in -1
        cand[::2, -5:] = -1
        cand_d[::2, -5:] = float('inf')
    got = kernels.graph_prune_rows(x, cand, cand_d, m_keep, fill)
    v = x[cand.clamp(min=0)].double()
    sq = v.square().sum(-1)                        # float64: the product form is exact enough
    pair = (sq.unsqueeze(-1) + sq.unsqueeze(-2) - 2.0 * (v @ v.mT)).clamp_(min=0.0)
    valid = cand >= 0
    pair[~(valid.unsqueeze(2) & valid.unsqueeze(1))] = float('inf')
    want = kernels.graph_prune(pair.float().contiguous(), cand_d.contiguous(), m_keep, fill)
    if k == 39:
        # candidates behind the end of a list do not exist for the kernel:
        # those rows against the pruning of their first 34 candidates
        short = kernels.graph_prune(pair[::2, :34, :34].float().contiguous(),
                                    cand_d[::2, :34].contiguous(), m_keep, fill)
        want[::2] = short
    same = (got == want).all(-1)
    torch.cuda.synchronize()
    assert int(got.max()) < k and int(got.min()) >= -1
    assert float(same.float().mean()) > 0.995, float(same.float().mean())
    # a row that differs does so at a near-tie
    margin = ((pair - cand_d.double().unsqueeze(-1)).abs() /
              cand_d.double().unsqueeze(-1).clamp(min=1e-30))
    margin[~(valid.unsqueeze(2) & valid.unsqueeze(1))] = float('inf')
    tight = margin.flatten(1).min(-1).values
    assert bool((tight[~same] < 1e-4).all())
    with pytest.raises(RuntimeError):
        kernels.graph_prune_rows(x, cand[:, :1].expand(-1, 300).contiguous(),
                                 cand_d[:, :1].expand(-1, 300).contiguous(), m_keep, fill)


def test_pruning_drops_a_candidate_beyond_the_rows(device):
    """A row number at or beyond the number of rows is no candidate: nothing
    is read for it (it would lie outside the arrays) and the selection is that
    of the same lists ending in -1 there."""
    n, d, k = 3000, 64, 24
    x = utils.gaussian_mixture(n, d, 8, 1.0, seed=77).to(device)
    cand, cand_d = utils.knn_graph(x, k)
    ended = cand.clone()
    ended[::3, -4:] = -1
    beyond = cand.clone()
    beyond[::3, -4:] = torch.tensor([n, n + 1, 1 << 40, (1 << 62) + 5], device=device)
    dist = cand_d.clone()
    dist[::3, -4:] = float('inf')
    want = kernels.graph_prune_rows(x, ended, dist, 12, True)
    got = kernels.graph_prune_rows(x, beyond, dist, 12, True)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert int(got[::3].max()) < k - 4


def test_pruning_of_more_nodes_than_one_launch_takes(device):
    """A launch holds fewer than 2^32 work-items, 2^22 nodes of 512: more nodes
    go in several launches, and the last ones are pruned like the first."""
    n, k, d = (1 << 22) + 1000, 8, 64
    print('prune rows, nodes', n, flush=True)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2000, d, generator=g).to(device)
    cand = torch.stack([torch.randperm(2000, generator=g)[:k] for _ in range(1000)]).to(device)
    cand_d = torch.sort(torch.rand(1000, k, generator=g) * 100 + 60, dim=-1).values.to(device)
    reps = -(-n // 1000)
    got = kernels.graph_prune_rows(x, cand.repeat(reps, 1)[:n].contiguous(),
                                   cand_d.repeat(reps, 1)[:n].contiguous(), 4, True)
    torch.cuda.synchronize()
    assert got.shape == (n, 4)
    assert int(got.min()) >= 0 and int(got.max()) < k
    # node i has the lists of node i % 1000: every block of 1000 nodes alike
    assert torch.equal(got[:1000], got[-1000:].roll(n % 1000, 0))
    assert torch.equal(got[:1000], got[(1 << 22):(1 << 22) + 1000].roll((1 << 22) % 1000, 0))
