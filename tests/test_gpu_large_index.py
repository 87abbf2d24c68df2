"""Traversal parity on an index of the memory-bounded configuration's shape:
2.5M reduced rows of 128 floats behind a sparse mapping, out-degree 48 with
ragged rows, ef = 128.  The graph is random (a proximity graph of this size
takes too long to build inside a test); the search rules do not care.  Same
bar as the small cases: distances bit-identical to the oracle, ids identical
except inside exact ties."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import assert_same_search

pytestmark = pytest.mark.gpu


def test_two_and_a_half_million_rows(device):
    n_nodes, n_rows, deg, dp, ef, n_init, B = 2_700_000, 2_500_000, 48, 128, 128, 64, 48
    g = torch.Generator().manual_seed(77)
    print('large index: nodes', n_nodes, 'rows', n_rows, flush=True)
    nodelist = torch.randperm(n_nodes, generator=g)[:n_rows].sort().values
    mapping = torch.full((n_nodes,), -1, dtype=torch.long)
    mapping[nodelist] = torch.arange(n_rows)
    nbr = nodelist[torch.randint(n_rows, (n_rows, deg), generator=g)]
    length = torch.randint(deg // 2, deg + 1, (n_rows, 1), generator=g)
    nbr[torch.arange(deg).unsqueeze(0) >= length] = -1
    rowlen = torch.zeros(n_nodes, dtype=torch.long)
    rowlen[nodelist] = deg
    indptr = torch.zeros(n_nodes + 1, dtype=torch.long)
    indptr[1:] = torch.cumsum(rowlen, 0)
    indices = nbr.flatten().contiguous()
    del nbr, length, rowlen

    x = torch.randn(n_nodes, dp, generator=g)
    query = torch.randn(B, dp, generator=g)
    init_I = nodelist[torch.randint(n_rows, (B, n_init), generator=g)].contiguous()
    xn, qn = x.numpy(), query.numpy()
    init_D = torch.from_numpy(np.stack([
        oracle.square_dist(qn[b].copy(), xn, init_I[b].numpy().copy())
        for b in range(B)]))

    k = 4 * ef
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_cpu(ref_I, ref_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        indptr.numpy(), indices.numpy(), xn, qn, k)

    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    storage = x[nodelist].contiguous().to(device)
    kernels.traverse_cuda(
        output_I=out_I, output_D=out_D, indptr=indptr.to(device),
        indices=indices.to(device), mapping=mapping.to(device),
        storage=storage, query=query.to(device), initial_I=init_I.to(device),
        initial_D=init_D.to(device), n_neighbors=deg)
    torch.cuda.synchronize()
    assert_same_search(out_I.flatten(1).cpu().numpy(),
                       out_D.flatten(1).cpu().numpy(), ref_I, ref_D)
    assert (ref_I >= 0).sum() > B * k // 2   # the searches did go somewhere
