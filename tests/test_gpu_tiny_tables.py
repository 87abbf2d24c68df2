"""The visited-set paths that a normal-size test never reaches, on a build of
the library whose LDS tables are one word / one bucket wide
(`tests/libpilotann_tiny_tables.so`: -DPA_SEEN_LOG2=0 -DPA_REFINE_SEEN_LOG2=0,
compiled by `__graft_entry__.build()`): with more than 65 535 rows the 16-bit
tags no longer fit and both kernels work on the bitmask alone (in the
shipped build that takes 67 M rows for the traversal, 33 M nodes for the
refine); below that the tiny tables displace or overflow on every step.  Same
bar: the oracle's distances bit for bit, its ids up to exact ties."""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import _lib, kernels, utils
from common import Problem, assert_same_search

pytestmark = pytest.mark.gpu

VARIANT = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                       'libpilotann_tiny_tables.so')


@pytest.fixture
def tiny_tables():
    if not os.path.exists(VARIANT):
        pytest.fail(f'{VARIANT} has not been built (__graft_entry__.build())')
    handle = ctypes.CDLL(VARIANT)
    for name, (restype, argtypes) in _lib._SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype, fn.argtypes = restype, argtypes
    shipped = _lib.lib()
    _lib._lib = handle
    yield
    _lib._lib = shipped


def traverse_case(p, dp, ef, n_init, device):
    init_I, init_D = p.entries(n_init, seed=5, dp=dp)
    B, k = p.query.size(0), 4 * ef
    ref_I, ref_D = np.empty((B, k), np.int64), np.empty((B, k), np.float32)
    oracle.traverse_cpu(ref_I, ref_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        p.sub_indptr.numpy(), p.sub_indices.numpy(),
                        np.ascontiguousarray(p.x[:, :dp].numpy()),
                        np.ascontiguousarray(p.query[:, :dp].numpy()), k)
    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    # not through the wrappers' caches: those belong to the shipped library
    graph = kernels.PreparedGraph(p.sub_indptr.to(device), p.sub_indices.to(device),
                                  p.mapping.to(device), p.nodelist.numel(), p.deg)
    rows = kernels.PreparedRows(p.x[p.nodelist][:, :dp].contiguous().to(device))
    kernels.traverse_prepared(out_I, out_D, graph, rows,
                              p.query[:, :dp].contiguous().to(device),
                              init_I.to(device), init_D.to(device))
    torch.cuda.synchronize()
    assert_same_search(out_I.flatten(1).cpu().numpy(), out_D.flatten(1).cpu().numpy(),
                       ref_I, ref_D)
    return out_I.flatten(1), out_D.flatten(1), graph


def refine_case(p, dp, ef_search, k, cand_I, cand_D, sub, device):
    B = p.query.size(0)
    ref_init_I, ref_init_D = cand_I.cpu().numpy().copy(), cand_D.cpu().numpy().copy()
    ref_I, ref_D = np.empty((B, k), np.int64), np.empty((B, k), np.float32)
    oracle.traverse_refine(ref_I, ref_D, ref_init_I, ref_init_D, ref_init_I, ref_init_D,
                           [p.sub_indptr.numpy(), p.sub_indices.numpy()],
                           [p.indptr.numpy(), p.indices.numpy()], p.x.numpy(),
                           p.query.numpy(), ef_search, dp)
    ident = torch.arange(p.n, device=device)
    full = kernels.PreparedGraph(p.indptr.to(device), p.indices.to(device), ident,
                                 p.n, p.deg)
    init_I, init_D = cand_I.clone(), cand_D.clone()
    out_I = torch.empty(B, k, dtype=torch.long, device=device)
    out_D = torch.empty(B, k, dtype=torch.float, device=device)
    kernels.traverse_refine_cuda(out_I, out_D, init_I, init_D, init_I, init_D, sub,
                                 full, kernels.PreparedRows(p.x.to(device)),
                                 p.query.to(device), ef_search, dp)
    torch.cuda.synchronize()
    assert_same_search(init_I.cpu().numpy(), init_D.cpu().numpy(), ref_init_I, ref_init_D)
    assert_same_search(out_I.cpu().numpy(), out_D.cpu().numpy(), ref_I, ref_D)


@pytest.mark.parametrize('n,ratio', [(6000, 0.5), (140_000, 0.5), (70_000, None)])
def test_both_kernels_with_one_word_tables(n, ratio, tiny_tables, device):
    """6000 nodes: tags fit, a one-word table that loses nearly every row it
    is told (traversal) and a single bucket that is full after eight marks
    (refine).  140 000 nodes, half of them stored (70 000 rows), and 70 000
    nodes all stored: more than 65 535 rows and nodes, no table at all."""
    print('tiny tables: nodes', n, 'sampled', ratio, flush=True)
    d, dp, deg = 32, 16, 32
    if n <= 10_000:
        p = Problem(n=n, d=d, deg=deg, sample_ratio=ratio, seed=n, n_query=64)
    else:
        # the neighbour tables of this size are built on the device
        p = Problem.__new__(Problem)
        p.n, p.d, p.deg = n, d, deg
        x = utils.gaussian_mixture(n, d, 32, 0.8, seed=n, device=device)
        p.query = utils.gaussian_mixture(64, d, 32, 0.8, seed=n + 1, center_seed=n)
        p.indptr, p.indices = utils.graph_init(x, 'nsw', deg)
        if ratio is None:
            p.sub_indptr, p.sub_indices = p.indptr, p.indices
            p.nodelist = torch.arange(n)
            p.mapping = torch.arange(n)
        else:
            sub = utils.subgraph_init(p.indptr, p.indices, x, 'nsw',
                                      round(ratio * n), deg, seed=n + 2)
            p.sub_indptr, p.sub_indices, p.nodelist, p.mapping = sub
        p.x = x.cpu().contiguous()
        assert p.nodelist.numel() > 0xffff
    cand_I, cand_D, graph = traverse_case(p, dp, 16, 32, device)
    refine_case(p, dp, 64, 10, cand_I.contiguous(), cand_D.contiguous(), graph, device)
