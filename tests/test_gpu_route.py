"""Router against the oracle: route ids equal to the exact argmin except on
float ties, leaf distances bit-identical."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels, utils

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('R,L,d,B', [(8, 32, 64, 1), (16, 64, 200, 777),
                                     (32, 32, 64, 1023), (64, 64, 128, 2500),
                                     (40, 96, 32, 333)])
def test_routing_matches_oracle(R, L, d, B, device):
    n = max(20000, 2 * min(1024, R * R) * L)
    x = utils.gaussian_mixture(n, d, 32, 0.5, seed=R + L)
    q = utils.gaussian_mixture(B, d, 32, 0.5, seed=99, center_seed=R + L)
    route_vectors, entry_nodes = utils.router_init(x, None, R, L, seed=1)
    entry_vectors = x[entry_nodes].contiguous()
    router, dist = kernels.routing_cuda(
        q.to(device), route_vectors.contiguous().to(device),
        entry_nodes.to(device), entry_vectors.to(device))
    router, dist = router.cpu().numpy(), dist.cpu().numpy()
    ref_router, _ = oracle.route(q.numpy(), route_vectors.contiguous().numpy(),
                                 entry_vectors.numpy())
    # the chosen route is the nearest one up to float rounding
    exact = torch.cdist(q.double(), route_vectors.double()).square().numpy()
    chosen = exact[np.arange(B), router]
    assert (chosen <= exact.min(-1) * (1 + 1e-5) + 1e-6).all()
    assert (router == ref_router).mean() > 0.999
    # distances to the leaves of the chosen route: bit-identical
    ref = np.stack([
        oracle.square_dist(q[b].numpy(), x.numpy(),
                           entry_nodes[router[b]].numpy().copy())
        for b in range(B)])
    assert np.array_equal(dist, ref)
    # the reference's own check (test_routing.py:69-85)
    target = torch.cdist(q.unsqueeze(1), x[entry_nodes[router]]).square()
    assert torch.allclose(torch.from_numpy(dist), target.squeeze(1), atol=1e-3)
    # the same launch can hand back the chosen route's entry ids
    r2, d2, ids = kernels.routing_cuda(
        q.to(device), route_vectors.contiguous().to(device),
        entry_nodes.to(device), entry_vectors.to(device), return_entries=True)
    assert np.array_equal(r2.cpu().numpy(), router)
    assert np.array_equal(d2.cpu().numpy(), dist)
    assert torch.equal(ids.cpu(), entry_nodes[torch.from_numpy(router)])


def test_entry_distances(device):
    x = utils.gaussian_mixture(5000, 96, 8, 0.5, seed=5)
    q = utils.gaussian_mixture(300, 96, 8, 0.5, seed=6, center_seed=5)
    nodes = torch.randint(high=5000, size=[48],
                          generator=torch.Generator().manual_seed(0))
    dist = kernels.entry_distances(q.to(device), x[nodes].contiguous().to(device))
    ref = np.stack([oracle.square_dist(q[b].numpy(), x.numpy(),
                                       nodes.numpy().copy())
                    for b in range(300)])
    assert np.array_equal(dist.cpu().numpy(), ref)


def test_routing_argument_errors(device):
    q = torch.randn(4, 64, device=device)
    rv = torch.randn(8, 64, device=device)
    en = torch.zeros(8, 32, dtype=torch.long, device=device)
    ev = torch.randn(8, 32, 64, device=device)
    kernels.routing_cuda(q, rv, en, ev)
    with pytest.raises(RuntimeError):
        kernels.routing_cuda(q.cpu(), rv, en, ev)
    with pytest.raises(RuntimeError):
        kernels.routing_cuda(q, rv[:, :32], en, ev)
    with pytest.raises(RuntimeError):
        kernels.routing_cuda(q, rv, en[:, :24].contiguous(),
                             ev[:, :24].contiguous())
    with pytest.raises(RuntimeError):
        kernels.routing_cuda(q, rv, en.int(), ev)


@pytest.mark.parametrize('seed', range(24))
def test_routing_random_shapes(seed, device):
    r = np.random.RandomState(500 + seed)
    R = int(r.choice([1, 2, 5, 31, 32, 33, 64, 100, 257]))
    L = int(r.choice([32, 64, 128]))
    d = int(r.choice([8, 24, 40, 64, 128, 256]))
    B = int(r.randint(1, 1500))
    print('route', dict(R=R, L=L, d=d, B=B), flush=True)
    g = torch.Generator().manual_seed(seed)
    q = torch.rand(B, d, generator=g)
    route_vectors = torch.rand(R, d, generator=g)
    entry_vectors = torch.rand(R, L, d, generator=g)
    entry_nodes = torch.arange(R * L).view(R, L)
    router, dist = kernels.routing_cuda(
        q.to(device), route_vectors.to(device), entry_nodes.to(device),
        entry_vectors.to(device))
    router, dist = router.cpu().numpy(), dist.cpu().numpy()
    assert router.min() >= 0 and router.max() < R
    exact = torch.cdist(q.double(), route_vectors.double()).square().numpy()
    chosen = exact[np.arange(B), router]
    assert (chosen <= exact.min(-1) * (1 + 1e-5) + 1e-6).all()
    flat = entry_vectors.view(R * L, d).numpy()
    ref = np.stack([
        oracle.square_dist(q[b].numpy(), flat, entry_nodes[router[b]].numpy().copy())
        for b in range(B)])
    assert np.array_equal(dist, ref)


@pytest.mark.parametrize('B,d,n_out', [
    (1, 8, 8), (31, 64, 32), (64, 96, 64), (100, 200, 40), (1000, 768, 128),
    (257, 768, 768), (65, 72, 1),
    # enough workgroups for the 64 x 128 and the 128 x 128 tiles, with ragged
    # edges in all three dimensions
    (3300, 1000, 1000), (6437, 1000, 1000),
])
def test_rotation_matches_float64_matmul(B, d, n_out, device):
    """`pa_rotate` (query @ VT.T, first n_out columns) against a float64
    product of the same float32 inputs.  Tolerance: float32 accumulation of d
    products, |error| <= 4 d eps |q| |v| (eps = 2^-24), far inside the 1e-5
    relative the search's distances are held to."""
    print('rotate case', B, d, n_out, flush=True)
    g = torch.Generator().manual_seed(B + d)
    query = torch.randn(B, d, generator=g)
    basis, _ = torch.linalg.qr(torch.randn(d, d, generator=g))
    VT = basis.T.contiguous()
    out = kernels.rotate(query.to(device), VT.to(device), n_out)
    torch.cuda.synchronize()
    assert out.shape == (B, n_out)
    ref = (query.to(device).double() @ VT.to(device).double().T)[:, :n_out].cpu()
    bound = 4 * d * 2.0 ** -24 * query.double().norm(dim=1, keepdim=True) \
        * VT.double().norm(dim=1)[:n_out].unsqueeze(0)
    assert bool(((out.cpu().double() - ref).abs() <= bound).all())
    # the rotation preserves lengths when all columns are kept
    if n_out == d:
        assert torch.allclose(out.cpu().norm(dim=1), query.norm(dim=1), rtol=1e-5)
    with pytest.raises(RuntimeError):
        kernels.rotate(query.to(device), VT.to(device), d + 1)
    with pytest.raises(RuntimeError):
        kernels.rotate(query, VT.to(device))
