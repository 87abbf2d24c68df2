"""Build-time helpers: formats the search path relies on and the properties
the reference's tests state for them (test/kernel/test_routing.py:6-33,
test_svd.py, test_graphs.py)."""
import pytest
import torch

from pilotann_amd import utils


def test_graph_format_and_quality():
    n, d, deg = 3000, 32, 32
    x = utils.gaussian_mixture(n, d, 4, 1.0, seed=1)
    for graph_type in ['nsw', 'nsg']:
        indptr, indices = utils.graph_init(x, graph_type, deg)
        assert indptr.dtype == indices.dtype == torch.int64
        assert indptr.tolist() == [i * deg for i in range(n + 1)]
        rows = indices.view(n, deg)
        assert int(rows.max()) < n and int(rows.min()) >= -1
        assert not (rows == torch.arange(n).unsqueeze(1)).any()      # no self loops
        # padding only at the end of a row, no repeats inside a row
        valid = rows >= 0
        assert (valid[:, :-1] | ~valid[:, 1:]).all()
        srt = torch.sort(torch.where(valid, rows, -torch.arange(1, deg + 1)), 1).values
        assert (srt[:, 1:] != srt[:, :-1]).all()
        # the true nearest neighbour is linked nearly always
        nn = utils.knn_graph(x, 1)[0]
        assert (rows == nn).any(1).float().mean() > 0.95


def test_sampling_is_seeded_and_closed_under_one_hop():
    n, deg = 4000, 16
    x = utils.gaussian_mixture(n, 16, 4, 1.0, seed=2)
    indptr, indices = utils.graph_init(x, 'nsw', deg)
    a = utils.graph_sampling(indptr, indices, n // 4, 1, seed=5)
    b = utils.graph_sampling(indptr, indices, n // 4, 1, seed=5)
    c = utils.graph_sampling(indptr, indices, n // 4, 1, seed=6)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert not torch.equal(a[0], c[0])
    nodelist, mapping = a
    assert n // 4 <= nodelist.numel() <= n // 4 + deg + 1
    assert torch.equal(torch.sort(nodelist).values, nodelist)
    # the checks of test_traverse_cuda.py:36-40
    assert int(mapping.max()) + 1 == nodelist.numel()
    assert (mapping[nodelist] == torch.arange(nodelist.numel())).all()
    assert int((mapping >= 0).sum()) == nodelist.numel()


def test_subgraph_layout():
    n, deg = 3000, 16
    x = utils.gaussian_mixture(n, 16, 4, 1.0, seed=3)
    indptr, indices = utils.graph_init(x, 'nsw', deg)
    sp, si, nodelist, mapping = utils.subgraph_init(indptr, indices, x, 'nsw',
                                                    n // 4, deg, seed=1)
    assert sp.numel() == n + 1 and int(sp[-1]) == si.numel()
    rowlen = sp[1:] - sp[:-1]
    assert (rowlen[mapping < 0] == 0).all() and (rowlen[mapping >= 0] == deg).all()
    assert (mapping[si[si >= 0]] >= 0).all()      # global ids of sampled nodes only


def test_router_init_routes_are_nearest_to_their_own_leaves():
    # test_routing.py:6-33
    # uniform data as in the reference's fuzz loader (utils/loader.py:31-36)
    g = torch.Generator().manual_seed(4)
    x = 2.0 * (torch.rand(40000, 32, generator=g) - 0.5)
    routes, nodes = utils.router_init(x, None, 32, 32, seed=9)
    assert routes.shape == (32, 32) and nodes.shape == (32, 32)
    # rounds draw disjoint node sets: no repeats inside one route's leaves
    assert all(len(set(r)) == 32 for r in nodes.tolist())
    dists = torch.cdist(routes.unsqueeze(0).expand(32, -1, -1), x[nodes]).sum(-1)
    assert torch.equal(torch.argmin(dists, -1), torch.arange(32))
    again = utils.router_init(x, None, 32, 32, seed=9)
    assert torch.equal(again[1], nodes)
    # init_nodes are consumed first (test_routing.py:46-57)
    init = list(range(100, 132))
    _, nodes2 = utils.router_init(x, list(init), 8, 32, seed=1)
    assert set(init) & set(nodes2.flatten().tolist())


def test_svd_rotation():
    # test_svd.py: x V V^T reconstructs x; leading coordinates carry the most
    x = utils.gaussian_mixture(5000, 48, 8, 1.0, seed=5, decay=0.5)
    xr, V = utils.svd(x, max_size=10 ** 7)
    assert torch.allclose(xr @ V.T, x, atol=1e-3)
    assert torch.allclose(V.T @ V, torch.eye(48), atol=1e-4)
    energy = xr.square().sum(0)
    assert (energy[:-1] >= energy[1:] * 0.999).all()
    xs, Vs = utils.svd(x, max_size=1000, seed=3)      # basis from a sample
    assert torch.allclose(xs @ Vs.T, x, atol=1e-3)


def test_recall():
    a = torch.tensor([[1, 2, 3], [4, 5, 6]])
    b = torch.tensor([[3, 2, 9], [7, 8, 9]])
    assert abs(utils.recall(a, b) - (2 / 3 + 0) / 2) < 1e-9


def test_router_init_rejects_a_set_too_small_for_it():
    x = torch.rand(500, 16)
    with pytest.raises(RuntimeError):
        utils.router_init(x, None, 32, 32, seed=1)   # needs 1024 * 32 nodes


def test_locality_order_is_a_permutation_that_groups_neighbours():
    x = utils.gaussian_mixture(6000, 16, 24, 0.2, seed=4)
    order = utils.locality_order(x, n_cells=24, seed=1)
    assert sorted(order.tolist()) == list(range(6000))
    assert torch.equal(order, utils.locality_order(x, n_cells=24, seed=1))
    # rows next to each other in the new order are far closer than rows next
    # to each other in the old one
    y = x[order]
    new_gap = (y[1:] - y[:-1]).norm(dim=1).mean()
    old_gap = (x[1:] - x[:-1]).norm(dim=1).mean()
    assert new_gap < 0.5 * old_gap
    assert utils.locality_order(x[:5]).numel() == 5


def test_sampling_follows_the_reference_rule_on_a_hand_built_graph():
    """extension/sampling_cpu.cpp:38-47: seeds are added, each with all nodes
    within n_hops edges, until the sample has n_samples nodes.  Graph: six
    stars 4k -> {4k+1, 4k+2, 4k+3} whose leaves have no edges, leaves of star
    k also point at the centre of star k+1 through node 4k+3."""
    n = 24
    rows = [[] for _ in range(n)]
    for k in range(6):
        rows[4 * k] = [4 * k + 1, 4 * k + 2, 4 * k + 3]
        rows[4 * k + 3] = [4 * ((k + 1) % 6)]
    indptr = torch.tensor([0] + [len(r) for r in rows]).cumsum(0)
    indices = torch.tensor([v for r in rows for v in r])

    def closure(seeds, hops):
        got = set(seeds)
        for s in seeds:
            frontier = {s}
            for _ in range(hops):
                frontier |= {v for u in frontier for v in rows[u]}
            got |= frontier
        return got

    for hops, want in ((1, 9), (2, 9), (1, 24)):
        for seed in range(5):
            nodelist, mapping, seeds = utils.graph_sampling(
                indptr, indices, want, hops, seed=seed, return_seeds=True)
            seeds = seeds.tolist()
            assert set(nodelist.tolist()) == closure(seeds, hops)
            assert len(nodelist) >= want
            # the last seed was needed: without it the sample is too small
            assert len(closure(seeds[:-1], hops)) < want
            assert (mapping[nodelist] == torch.arange(len(nodelist))).all()
            assert int((mapping >= 0).sum()) == len(nodelist)


def test_connectivity_pass_joins_separated_clusters():
    """Well separated clusters: the neighbour table alone leaves one island
    per cluster; after the pass every node is reachable from every node, the
    row format is intact and the searches of the reference's own graph test
    (test/kernel/test_graphs.py:55-64) find their neighbours from entries in
    another cluster."""
    n, d, deg = 4000, 32, 16
    x = utils.gaussian_mixture(n, d, 16, 0.05, seed=8)
    for graph_type in ['nsw', 'nsg']:
        # every pool from the whole set: the table the pass is there for
        _, loose = utils.graph_init(x, graph_type, deg, connect=False,
                                    insertion_order=False)
        loose = loose.view(n, deg)
        assert not bool(utils.reachable(loose, torch.tensor([0])).all())
        indptr, indices = utils.graph_init(x, graph_type, deg,
                                           insertion_order=False)
        rows = indices.view(n, deg)
        for start in (0, 1234, n - 1):
            assert bool(utils.reachable(rows, torch.tensor([start])).all())
            assert bool(utils.reachable(rows, torch.tensor([start]), reverse=True).all())
        valid = rows >= 0
        assert (valid[:, :-1] | ~valid[:, 1:]).all()
        assert not (rows == torch.arange(n).unsqueeze(1)).any()
        srt = torch.sort(torch.where(valid, rows, -torch.arange(1, deg + 1)), 1).values
        assert (srt[:, 1:] != srt[:, :-1]).all()
        # a search from one fixed entry reaches the neighbours of queries of
        # every cluster
        import numpy as np
        import oracle
        q = utils.gaussian_mixture(64, d, 16, 0.05, seed=9, center_seed=8)
        target = utils.brute_force_topk(q, x, 10)
        init_I = torch.zeros(64, 1, dtype=torch.long)
        init_D = (q - x[0]).square().sum(-1, keepdim=True)
        out_I = np.empty((64, 10), np.int64)
        out_D = np.empty((64, 10), np.float32)
        oracle.traverse_cpu(out_I, out_D, init_I.numpy(), init_D.numpy().copy(),
                            indptr.numpy(), indices.numpy(), x.numpy(), q.numpy(), 64)
        # (0.08 on the table without the pass: one cluster of sixteen; the
        # bridges are few, so a greedy search does not always find them)
        assert utils.recall(torch.from_numpy(out_I), target) > 0.5


def test_insertion_order_makes_the_graph_navigable_across_clusters():
    """Pools taken in insertion order (a node's nearest among the nodes
    before it in a seeded random order): the early nodes' long edges join the
    clusters without the connectivity pass, and a search from one fixed entry
    finds the neighbours of queries of every cluster far better than on the
    table of nearest neighbours in the whole set with its few bridges."""
    import numpy as np
    import oracle
    n, d, deg = 4000, 32, 16
    x = utils.gaussian_mixture(n, d, 16, 0.05, seed=8)
    q = utils.gaussian_mixture(64, d, 16, 0.05, seed=9, center_seed=8)
    target = utils.brute_force_topk(q, x, 10)
    init_I = torch.zeros(64, 1, dtype=torch.long)
    init_D = (q - x[0]).square().sum(-1, keepdim=True)
    score = {}
    for ordered in (False, True):
        indptr, indices = utils.graph_init(x, 'nsw', deg, connect=not ordered,
                                           insertion_order=ordered, seed=3)
        rows = indices.view(n, deg)
        for start in (0, 1234, n - 1):
            assert bool(utils.reachable(rows, torch.tensor([start])).all())
            assert bool(utils.reachable(rows, torch.tensor([start]), reverse=True).all())
        valid = rows >= 0
        assert (valid[:, :-1] | ~valid[:, 1:]).all()
        assert not (rows == torch.arange(n).unsqueeze(1)).any()
        srt = torch.sort(torch.where(valid, rows, -torch.arange(1, deg + 1)), 1).values
        assert (srt[:, 1:] != srt[:, :-1]).all()
        out_I = np.empty((64, 10), np.int64)
        out_D = np.empty((64, 10), np.float32)
        oracle.traverse_cpu(out_I, out_D, init_I.numpy(), init_D.numpy().copy(),
                            indptr.numpy(), indices.numpy(), x.numpy(), q.numpy(), 64)
        score[ordered] = utils.recall(torch.from_numpy(out_I), target)
    print('recall@10 from one entry, whole-set pools / insertion order:', score)
    assert score[True] > 0.9 and score[True] > score[False]
    # same seed, same graph
    again = utils.graph_init(x, 'nsw', deg, connect=False, seed=3)[1]
    assert torch.equal(again, indices)
