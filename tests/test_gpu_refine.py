"""Device refine against the oracle's `traverse_refine` on the same inputs
(extension/traverse_cpu.cpp:261-369): the buffer of the first search, the
completed candidate distances and the final top-k must be the host's, distances
bit for bit, ids up to exact ties; the invariants of the reference's own test
(test/kernel/test_traverse_refine.py) hold on top."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import Problem, assert_same_search

pytestmark = pytest.mark.gpu


def candidates(p, dp, ef, n_init, device, seed=9):
    """Stage-1 output of the device traversal: [B, 4 * ef] ids and distances
    over the first dp coordinates."""
    B = p.query.size(0)
    init_I, init_D = p.entries(n_init, seed=seed, dp=dp)
    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    kernels.traverse_cuda(out_I, out_D, p.sub_indptr.to(device),
                          p.sub_indices.to(device), p.mapping.to(device),
                          p.x[p.nodelist][:, :dp].contiguous().to(device),
                          p.query[:, :dp].contiguous().to(device),
                          init_I.to(device), init_D.to(device), p.deg)
    return out_I.flatten(1).contiguous(), out_D.flatten(1).contiguous()


def run_both(p, dp, ef_search, k, cand_I, cand_D, device, n_buffers=None,
             alias=True):
    B = p.query.size(0)
    n_buffers = n_buffers or cand_I.size(1)
    # oracle
    ref_init_I = cand_I.cpu().numpy().copy()
    ref_init_D = cand_D.cpu().numpy().copy()
    if alias:
        ref_buf_I, ref_buf_D = ref_init_I, ref_init_D
    else:
        ref_buf_I = np.empty((B, n_buffers), np.int64)
        ref_buf_D = np.empty((B, n_buffers), np.float32)
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_refine(ref_I, ref_D, ref_buf_I, ref_buf_D, ref_init_I,
                           ref_init_D,
                           [p.sub_indptr.numpy(), p.sub_indices.numpy()],
                           [p.indptr.numpy(), p.indices.numpy()], p.x.numpy(),
                           p.query.numpy(), ef_search, dp)
    # device
    sub = kernels.prepare_graph(p.sub_indptr.to(device), p.sub_indices.to(device),
                                p.mapping.to(device), p.nodelist.numel(), p.deg)
    full = kernels.prepare_full_graph(p.indptr.to(device), p.indices.to(device))
    init_I, init_D = cand_I.clone(), cand_D.clone()
    if alias:
        buf_I, buf_D = init_I, init_D
    else:
        buf_I = torch.empty(B, n_buffers, dtype=torch.long, device=device)
        buf_D = torch.empty(B, n_buffers, dtype=torch.float, device=device)
    out_I = torch.empty(B, k, dtype=torch.long, device=device)
    out_D = torch.empty(B, k, dtype=torch.float, device=device)
    counters = torch.zeros(6, dtype=torch.long, device=device)
    kernels.traverse_refine_cuda(out_I, out_D, buf_I, buf_D, init_I, init_D,
                                 sub, full, kernels.prepare_rows(p.x.to(device)),
                                 p.query.to(device), ef_search, dp,
                                 counters=counters)
    torch.cuda.synchronize()
    got = dict(out_I=out_I.cpu().numpy(), out_D=out_D.cpu().numpy(),
               buf_I=buf_I.cpu().numpy(), buf_D=buf_D.cpu().numpy(),
               init_D=init_D.cpu().numpy(), counters=counters.cpu().numpy())
    ref = dict(out_I=ref_I, out_D=ref_D, buf_I=ref_buf_I, buf_D=ref_buf_D,
               init_D=ref_init_D)
    return got, ref


@pytest.mark.parametrize('d,dp,deg,ef,ef_search,k,graph', [
    (64, 32, 32, 16, 16, 10, 'nsw'),      # the pipeline's shape: n_buffers = 4 ef_search > H
    (64, 64, 32, 8, 32, 10, 'nsw'),       # nothing to complete
    (128, 32, 24, 32, 64, 20, 'nsw'),
    (96, 40, 32, 16, 100, 100, 'nsg'),    # odd number of groups before the tail
    (768, 128, 32, 16, 64, 10, 'nsw'),    # long rows
    (256, 40, 32, 16, 32, 10, 'nsw'),     # odd first group, batched loads, rest
    (64, 16, 48, 64, 300, 10, 'nsw'),     # heap tail in LDS
])
def test_refine_matches_oracle(d, dp, deg, ef, ef_search, k, graph, device):
    print('refine case', d, dp, deg, ef, ef_search, k, graph, flush=True)
    n = 3000 if d == 768 else 6000
    p = Problem(n=n, d=d, deg=deg, graph_type=graph, sample_ratio=0.25,
                seed=41, n_query=96)
    cand_I, cand_D = candidates(p, dp, ef, 32, device)
    got, ref = run_both(p, dp, ef_search, k, cand_I, cand_D, device)
    # buffer: the first search's result (aliases the candidates, as in
    # pipeline_cpu.cpp:110-114)
    assert_same_search(got['buf_I'], got['buf_D'], ref['buf_I'], ref['buf_D'])
    assert_same_search(got['out_I'], got['out_D'], ref['out_I'], ref['out_D'])
    # test_traverse_refine.py: D is the full-dimension distance of I
    top_I = torch.from_numpy(got['out_I'])
    ok = top_I >= 0
    target = torch.cdist(p.query.unsqueeze(1),
                         p.x[top_I.clamp(min=0)]).squeeze(1).square()
    assert torch.allclose(torch.from_numpy(got['out_D'])[ok], target[ok],
                          atol=1e-3)
    c = got['counters']
    assert c[0] <= 2 * 96 and c[1] > 0 and c[2] > 0
    assert c[4] == (0 if dp == d else int((cand_I >= 0).sum()))


def test_separate_buffer_and_completed_distances(device):
    """Buffer of another width than the candidates; initial_D ends up as the
    full-dimension distance of initial_I (traverse_cpu.cpp:42-62)."""
    p = Problem(n=5000, d=64, deg=32, sample_ratio=0.3, seed=43, n_query=64)
    cand_I, cand_D = candidates(p, 32, 16, 32, device)
    for n_buffers in (24, 64, 200):
        got, ref = run_both(p, 32, 48, 10, cand_I, cand_D, device,
                            n_buffers=n_buffers, alias=False)
        assert np.array_equal(got['init_D'], ref['init_D'])
        assert_same_search(got['buf_I'], got['buf_D'], ref['buf_I'], ref['buf_D'])
        assert_same_search(got['out_I'], got['out_D'], ref['out_I'], ref['out_D'])
    ids = cand_I.cpu()
    ok = ids >= 0
    target = torch.cdist(p.query.unsqueeze(1),
                         p.x[ids.clamp(min=0)]).squeeze(1).square()
    assert torch.allclose(torch.from_numpy(got['init_D'])[ok], target[ok],
                          atol=1e-3)


def test_unused_candidates_and_small_batches(device):
    """Negative ids among the candidates are skipped; batches smaller than the
    number of resident wavefronts; an empty batch."""
    p = Problem(n=4000, d=64, deg=32, sample_ratio=0.25, seed=47, n_query=7)
    cand_I, cand_D = candidates(p, 32, 16, 32, device)
    cand_I[:, ::3] = -1
    cand_I[2] = -1                       # a query without any candidate
    got, ref = run_both(p, 32, 32, 10, cand_I, cand_D, device)
    assert_same_search(got['buf_I'], got['buf_D'], ref['buf_I'], ref['buf_D'])
    assert_same_search(got['out_I'], got['out_D'], ref['out_I'], ref['out_D'])
    assert (got['out_I'][2] == -1).all()
    sub = kernels.prepare_graph(p.sub_indptr.to(device), p.sub_indices.to(device),
                                p.mapping.to(device), p.nodelist.numel(), p.deg)
    full = kernels.prepare_full_graph(p.indptr.to(device), p.indices.to(device))
    rows = kernels.prepare_rows(p.x.to(device))
    empty_I = torch.empty(0, 10, dtype=torch.long, device=device)
    empty_D = torch.empty(0, 10, dtype=torch.float, device=device)
    kernels.traverse_refine_cuda(
        empty_I, empty_D, empty_I.clone(), empty_D.clone(), empty_I.clone(),
        empty_D.clone(), sub, full, rows,
        torch.empty(0, 64, device=device), 32, 32)
    with pytest.raises(RuntimeError):    # host tensors are refused
        kernels.traverse_refine_cuda(
            empty_I.cpu(), empty_D, empty_I, empty_D, empty_I, empty_D, sub,
            full, rows, torch.empty(0, 64, device=device), 32, 32)
    with pytest.raises(RuntimeError):    # plain rows are refused
        kernels.traverse_refine_cuda(
            empty_I, empty_D, empty_I, empty_D, empty_I, empty_D, sub,
            full, p.x.to(device), torch.empty(0, 64, device=device), 32, 32)


@pytest.mark.parametrize('d', [8, 16, 24, 40, 768])
def test_row_layout(d, device):
    """pa_rows_prepare: within every 16 floats the pairs of the two groups of
    eight are interleaved by lane; a last group without a partner stays."""
    x = torch.arange(5 * d, dtype=torch.float32).reshape(5, d)
    got = kernels.prepare_rows(x.to(device)).rows.cpu()
    blocks = d // 16
    want = x.clone()
    if blocks:
        head = x[:, :blocks * 16].reshape(5, blocks, 2, 4, 2)   # block, group, lane, pair
        want[:, :blocks * 16] = head.permute(0, 1, 3, 2, 4).reshape(5, blocks * 16)
    assert torch.equal(got, want)
