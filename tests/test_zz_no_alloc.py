"""pa_traverse_static — the traversal for callers that cannot allocate device
memory, scratch in a static device array — against pa_traverse on the same
inputs, through the C ABI: two calls in a row, the second on a smaller index
with fewer queries and shorter lists, so that whatever the first call left in
the shared array is still there.  Ids and distances must be equal bit for bit
(both entry points run the same search)."""
import ctypes

import numpy as np
import pytest
import torch

from pilotann_amd import _lib, kernels
from common import Problem

pytestmark = pytest.mark.gpu


def both_entry_points(p, dp, ef, n_init, seed, device):
    B = p.query.size(0)
    init_I, init_D = p.entries(n_init, seed=seed, dp=dp)
    graph = kernels.prepare_graph(p.sub_indptr.to(device), p.sub_indices.to(device),
                                  p.mapping.to(device), p.nodelist.numel(), p.deg)
    rows = kernels.prepare_rows(p.x[p.nodelist][:, :dp].contiguous().to(device))
    query = p.query[:, :dp].contiguous().to(device)
    init_I, init_D = init_I.to(device), init_D.to(device)
    out = []
    for static in (False, True):
        out_I = torch.full((B, 4, ef), -7, dtype=torch.long, device=device)
        out_D = torch.full((B, 4, ef), -7.0, dtype=torch.float, device=device)
        cnt = torch.zeros(5, dtype=torch.long, device=device)
        if static:
            lib = _lib.lib()
            vp = ctypes.c_void_p
            stream = vp(torch.cuda.current_stream().cuda_stream)
            rc = lib.pa_traverse_static(
                vp(out_I.data_ptr()), vp(out_D.data_ptr()),
                vp(graph.adj.data_ptr()), vp(graph.gid.data_ptr()),
                vp(graph.mapping.data_ptr()), vp(rows.rows.data_ptr()),
                vp(query.data_ptr()), vp(init_I.data_ptr()),
                vp(init_D.data_ptr()), B, graph.n_nodes, graph.n_storage, dp,
                n_init, 4, ef, p.deg, vp(cnt.data_ptr()), stream)
            assert rc == 0, _lib.lib().pa_error_string(rc)
        else:
            kernels.traverse_prepared(out_I, out_D, graph, rows, query, init_I,
                                      init_D, counters=cnt)
        torch.cuda.synchronize()
        out.append((out_I.cpu().numpy(), out_D.cpu().numpy(), cnt.cpu().numpy()))
    return out


def test_static_scratch_entry_point_equals_pa_traverse(device):
    big = Problem(n=9000, d=64, deg=48, sample_ratio=0.5, seed=61, n_query=700)
    small = Problem(n=2500, d=32, deg=16, sample_ratio=0.25, seed=62, n_query=37)
    # the third call with the longest lists (ef 512: 4096 cells, whose last
    # two levels live in the array as well)
    for name, p, dp, ef, n_init in (('first call', big, 64, 96, 48),
                                    ('second, smaller call', small, 32, 8, 8),
                                    ('third call, longest lists', small, 32, 512, 8)):
        print('static scratch:', name, flush=True)
        (I_a, D_a, c_a), (I_b, D_b, c_b) = both_entry_points(p, dp, ef, n_init, 3, device)
        assert (I_a != -7).all() and (I_b != -7).all()
        assert np.array_equal(I_a, I_b)
        assert np.array_equal(D_a, D_b)
        assert np.array_equal(c_a, c_b) and c_a[0] > 0


def test_static_scratch_limits(device):
    """Argument errors are the same as pa_traverse's; an index whose visited
    slices do not fit the array often enough is refused, nothing is launched."""
    lib = _lib.lib()
    none = ctypes.c_void_p(None)
    args = [none] * 9
    # 200 M rows: 25 MB per wavefront, five fit, 256 are asked for
    assert lib.pa_traverse_static(*args, 1000, 300_000_000, 200_000_000, 128, 64,
                                  4, 64, 64, none, none) == -1      # null pointers first
    x = torch.zeros(1024, device=device)
    ptr = ctypes.c_void_p(x.data_ptr())
    assert lib.pa_traverse_static(*([ptr] * 9), 1000, 300_000_000, 200_000_000,
                                  128, 64, 4, 64, 64, none, none) == -11
    assert b'static scratch' in lib.pa_error_string(-11)
    assert lib.pa_traverse_static(*([ptr] * 9), 10, 1000, 500, 60, 8, 4, 8, 16,
                                  none, none) == -3
    assert lib.pa_traverse_static(*([ptr] * 9), 0, 1000, 500, 64, 8, 4, 8, 16,
                                  none, none) == 0
