"""Parity at the shape of the top-100 configuration: 128-float reduced rows,
out-degree 64, half of the nodes sampled, 64 entries, result lists of 1024
(ef = 256) and 2048 (ef = 512) cells on a proximity graph large enough that
a search runs into the cap of 1024 expansions and fills its open list, so that
the large-leaf rule of the open list (extension/inc/heapq.cuh:47-77) displaces
live entries.  Then the refine with top-100 and ef_search = 256 on the same
index.  Bar as everywhere: distances bit-identical to the oracle, ids
identical except inside exact ties; the work counters are the oracle's."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels, utils
from common import assert_same_search

pytestmark = pytest.mark.gpu

N, D, DP, DEG, N_INIT, B = 120_000, 256, 128, 64, 64, 48


class LongListIndex:
    def __init__(self, device):
        x = utils.gaussian_mixture(N, D, 64, 1.0, seed=401, device=device,
                                   decay=0.5)
        self.query = utils.gaussian_mixture(B, D, 64, 1.0, seed=402,
                                            center_seed=401, decay=0.5)
        self.indptr, self.indices = utils.graph_init(x, 'nsw', DEG)
        sub = utils.subgraph_init(self.indptr, self.indices, x, 'nsw',
                                  N // 2, DEG, seed=403)
        self.sub_indptr, self.sub_indices, self.nodelist, self.mapping = sub
        self.x = x.cpu()
        g = torch.Generator().manual_seed(404)
        pick = torch.randint(self.nodelist.numel(), (B, N_INIT), generator=g)
        self.init_I = self.nodelist[pick].contiguous()
        xr = np.ascontiguousarray(self.x[:, :DP].numpy())
        qr = np.ascontiguousarray(self.query[:, :DP].numpy())
        self.xr, self.qr = xr, qr
        self.init_D = torch.from_numpy(np.stack([
            oracle.square_dist(qr[b].copy(), xr, self.init_I[b].numpy().copy())
            for b in range(B)]))


@pytest.fixture(scope='module')
def index(device):
    print('building the 120k-node index', flush=True)
    return LongListIndex(device)


def traverse_both(ix, ef, device):
    k = 4 * ef
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    ref_cnt = np.zeros(5, np.int64)
    oracle.traverse_cpu(ref_I, ref_D, ix.init_I.numpy().copy(),
                        ix.init_D.numpy().copy(), ix.sub_indptr.numpy(),
                        ix.sub_indices.numpy(), ix.xr, ix.qr, k, ref_cnt)
    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    cnt = torch.zeros(5, dtype=torch.long, device=device)
    storage = torch.from_numpy(ix.xr)[ix.nodelist].contiguous().to(device)
    kernels.traverse_cuda(
        out_I, out_D, ix.sub_indptr.to(device), ix.sub_indices.to(device),
        ix.mapping.to(device), storage, torch.from_numpy(ix.qr).to(device),
        ix.init_I.to(device), ix.init_D.to(device), DEG, counters=cnt)
    torch.cuda.synchronize()
    return (out_I.flatten(1), out_D.flatten(1), cnt.cpu().numpy(),
            ref_I, ref_D, ref_cnt)


@pytest.mark.parametrize('ef', [256, 512])
def test_long_result_lists_match_oracle(ef, index, device):
    print('long lists: ef', ef, 'heap', oracle.heap_size(4 * ef), flush=True)
    out_I, out_D, cnt, ref_I, ref_D, ref_cnt = traverse_both(index, ef, device)
    assert_same_search(out_I.cpu().numpy(), out_D.cpu().numpy(), ref_I, ref_D)
    # the regime this test is for: (nearly) every search is ended by the cap
    # of 1024 expansions, and the open list's large-leaf rule has displaced
    # live entries
    assert ref_cnt[0] >= 0.85 * B * 1024
    assert ref_cnt[4] > 0
    assert cnt[0] == ref_cnt[0] and cnt[2] == ref_cnt[2] and cnt[3] == ref_cnt[3]
    assert (ref_I >= 0).all()


def test_refine_top_100_matches_oracle(index, device):
    ix = index
    ef, ef_search, k = 256, 256, 100
    cand_I, cand_D, _, _, _, _ = traverse_both(ix, ef, device)
    cand_I, cand_D = cand_I.contiguous(), cand_D.contiguous()
    ref_init_I = cand_I.cpu().numpy().copy()
    ref_init_D = cand_D.cpu().numpy().copy()
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_refine(ref_I, ref_D, ref_init_I, ref_init_D, ref_init_I,
                           ref_init_D,
                           [ix.sub_indptr.numpy(), ix.sub_indices.numpy()],
                           [ix.indptr.numpy(), ix.indices.numpy()],
                           ix.x.numpy(), ix.query.numpy(), ef_search, DP)
    sub = kernels.prepare_graph(ix.sub_indptr.to(device),
                                ix.sub_indices.to(device),
                                ix.mapping.to(device), ix.nodelist.numel(), DEG)
    full = kernels.prepare_full_graph(ix.indptr.to(device),
                                      ix.indices.to(device), DEG)
    init_I, init_D = cand_I.clone(), cand_D.clone()
    out_I = torch.empty(B, k, dtype=torch.long, device=device)
    out_D = torch.empty(B, k, dtype=torch.float, device=device)
    kernels.traverse_refine_cuda(out_I, out_D, init_I, init_D, init_I, init_D,
                                 sub, full, kernels.prepare_rows(ix.x.to(device)),
                                 ix.query.to(device), ef_search, DP)
    torch.cuda.synchronize()
    assert_same_search(init_I.cpu().numpy(), init_D.cpu().numpy(),
                       ref_init_I, ref_init_D)
    assert_same_search(out_I.cpu().numpy(), out_D.cpu().numpy(), ref_I, ref_D)


def test_longest_lists_when_wavefronts_take_a_second_query(index, device):
    """More queries than a launch has wavefronts (9 per compute unit with the
    lists of 4096 cells), so that a wavefront starts a query on the log whose
    head the last query's two-part sort has rewritten: the 48 queries 60 times
    over, every copy equal to the oracle's answer for its query."""
    ef, reps = 512, 60
    k = 4 * ef
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_cpu(ref_I, ref_D, index.init_I.numpy().copy(),
                        index.init_D.numpy().copy(), index.sub_indptr.numpy(),
                        index.sub_indices.numpy(), index.xr, index.qr, k)
    n = B * reps
    out_I = torch.empty(n, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(n, 4, ef, dtype=torch.float, device=device)
    storage = torch.from_numpy(index.xr)[index.nodelist].contiguous().to(device)
    kernels.traverse_cuda(
        out_I, out_D, index.sub_indptr.to(device), index.sub_indices.to(device),
        index.mapping.to(device), storage,
        torch.from_numpy(index.qr).to(device).repeat(reps, 1).contiguous(),
        index.init_I.to(device).repeat(reps, 1).contiguous(),
        index.init_D.to(device).repeat(reps, 1).contiguous(), DEG)
    torch.cuda.synchronize()
    got_I = out_I.flatten(1).cpu().numpy().reshape(reps, B, k)
    got_D = out_D.flatten(1).cpu().numpy().reshape(reps, B, k)
    assert_same_search(got_I[0], got_D[0], ref_I, ref_D)
    for r in range(1, reps):
        assert np.array_equal(got_D[r], got_D[0]), f'copy {r}: distances'
        assert np.array_equal(got_I[r], got_I[0]), f'copy {r}: ids'
