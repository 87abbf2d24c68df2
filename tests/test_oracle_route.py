"""The oracle's router (`orc_route`, after extension/routing_cuda.cu:70-113)
against what fixes it without a device: the route of a query is the float64
argmin of its distances to the route vectors (the reference asks libtorch's
cdist / argmin for it, routing_cuda.cu:93-95, and its own test compares with
exactly that, test/kernel/test_routing.py:69-85), and the distances returned
are those of the pinned distance function to the chosen route's leaves."""
import numpy as np
import pytest
import torch

import oracle


@pytest.mark.parametrize('B,R,L,d', [(257, 8, 32, 64), (100, 16, 64, 128),
                                     (1, 3, 32, 8), (64, 64, 64, 40)])
def test_route_is_the_float64_argmin_and_leaf_distances_are_the_pinned_ones(B, R, L, d):
    g = torch.Generator().manual_seed(B + R + L + d)
    q = torch.randn(B, d, generator=g)
    routes = torch.randn(R, d, generator=g)
    leaves = torch.randn(R, L, d, generator=g)
    router, dist = oracle.route(q.numpy(), routes.numpy(), leaves.numpy())
    all_d = torch.cdist(q.double(), routes.double())
    want = all_d.argmin(-1).numpy()
    # a float32 sum may turn a float64 near-tie round: accept either then
    ok = router == want
    for b in np.flatnonzero(~ok):
        gap = all_d[b, router[b]] - all_d[b, want[b]]
        assert float(gap) <= 1e-5 * float(all_d[b, want[b]]), (b, float(gap))
    assert ok.mean() > 0.99
    flat = leaves.reshape(R * L, d).numpy()
    for b in range(B):
        nodes = np.arange(L, dtype=np.int64) + router[b] * L
        assert np.array_equal(dist[b], oracle.square_dist(q[b].numpy(), flat, nodes))
    ref = torch.cdist(q.double().unsqueeze(1), leaves[torch.from_numpy(router)].double()).square()
    assert np.allclose(dist, ref.squeeze(1).numpy(), rtol=1e-5, atol=1e-6)


def test_route_ties_go_to_the_first_route():
    """Two identical route vectors: the lower index wins, as argmin does."""
    q = np.zeros((4, 8), np.float32)
    routes = np.ones((3, 8), np.float32)
    routes[2] = 0.5          # the nearest
    routes[1] = 0.5          # ... and its twin before it
    leaves = np.zeros((3, 32, 8), np.float32)
    router, _ = oracle.route(q, routes, leaves)
    assert (router == 1).all()
