"""Device refine on rows that span more than 4 GiB (1.5M x 768 floats): row
offsets beyond 32 bits, a visited slice of 1.5M bits, random graphs of the
memory-bounded configuration's degrees.  Same bar as the small cases."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import assert_same_search

pytestmark = pytest.mark.gpu


def test_rows_beyond_four_gib(device):
    n, n_sub, d, dp, deg, ef_search, B, n_cand, k = 1_500_000, 400_000, 768, 128, 48, 64, 32, 256, 10
    g = torch.Generator().manual_seed(91)
    print('large refine: nodes', n, 'row bytes', n * d * 4, flush=True)
    x = torch.randn(n, d, generator=g)
    query = torch.randn(B, d, generator=g)
    nodelist = torch.randperm(n, generator=g)[:n_sub].sort().values
    mapping = torch.full((n,), -1, dtype=torch.long)
    mapping[nodelist] = torch.arange(n_sub)
    sub = nodelist[torch.randint(n_sub, (n_sub, deg), generator=g)]
    rowlen = torch.zeros(n, dtype=torch.long)
    rowlen[nodelist] = deg
    sub_indptr = torch.zeros(n + 1, dtype=torch.long)
    sub_indptr[1:] = torch.cumsum(rowlen, 0)
    full = torch.randint(n, (n, deg), generator=g)
    full[torch.arange(deg).unsqueeze(0) >= torch.randint(deg // 2, deg + 1, (n, 1), generator=g)] = -1
    full_indptr = torch.arange(n + 1, dtype=torch.long) * deg
    # candidates biased to the upper part of the table (offsets > 4 GiB)
    cand = nodelist[torch.randint(n_sub * 3 // 4, n_sub, (B, n_cand), generator=g)].contiguous()
    xn, qn = x.numpy(), query.numpy()
    x_dp = np.ascontiguousarray(xn[:, :dp])
    cand_D = torch.from_numpy(np.stack([
        oracle.square_dist(np.ascontiguousarray(qn[b, :dp]), x_dp, cand[b].numpy().copy())
        for b in range(B)]))
    del x_dp

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
    rows = kernels.PreparedRows(x.to(device))
    buf_I, buf_D = cand.to(device), cand_D.to(device)
    out_I = torch.empty(B, k, dtype=torch.long, device=device)
    out_D = torch.empty(B, k, dtype=torch.float, device=device)
    kernels.traverse_refine_cuda(out_I, out_D, buf_I, buf_D, buf_I, buf_D, sub_g, full_g,
                                 rows, query.to(device), ef_search, dp)
    torch.cuda.synchronize()
    assert_same_search(buf_I.cpu().numpy(), buf_D.cpu().numpy(), ref_buf_I, ref_buf_D)
    assert_same_search(out_I.cpu().numpy(), out_D.cpu().numpy(), ref_I, ref_D)
    assert (ref_I >= n // 2).any()
