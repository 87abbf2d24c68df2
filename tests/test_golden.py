"""The committed fixture (tests/golden/) against the oracle, the host stages
and, on a GPU, the device kernels."""
import os

import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import assert_same_search

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope='module')
def fx():
    z = np.load(os.path.join(HERE, 'golden', 'traverse_small.npz'))
    out = {k: z[k] for k in z.files}
    for k in ['indptr', 'indices', 'sub_indptr', 'sub_indices', 'nodelist',
              'mapping', 'init_I', 'cand_I', 'stage2_I', 'top_I']:
        out[k] = out[k].astype(np.int64)
    for k in ['dp', 'ef', 'k', 'deg']:
        out[k] = int(out[k])
    return out


def test_oracle_reproduces_the_fixture(fx):
    dp, ef = fx['dp'], fx['ef']
    B = fx['query'].shape[0]
    cand_I = np.empty((B, 4 * ef), np.int64)
    cand_D = np.empty((B, 4 * ef), np.float32)
    oracle.traverse_cpu(cand_I, cand_D, fx['init_I'].copy(), fx['init_D'].copy(),
                        fx['sub_indptr'], fx['sub_indices'],
                        np.ascontiguousarray(fx['x'][:, :dp]),
                        np.ascontiguousarray(fx['query'][:, :dp]), 4 * ef)
    assert np.array_equal(cand_I, fx['cand_I']) and np.array_equal(cand_D, fx['cand_D'])


def test_host_stages_reproduce_the_fixture(fx):
    dp, ef, k = fx['dp'], fx['ef'], fx['k']
    B = fx['query'].shape[0]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    top_I = torch.empty(B, k, dtype=torch.long)
    top_D = torch.empty(B, k)
    buf_I, buf_D = t(fx['cand_I'].copy()), t(fx['cand_D'].copy())
    kernels.traverse_refine(top_I, top_D, buf_I, buf_D, buf_I, buf_D,
                            [t(fx['sub_indptr']), t(fx['sub_indices'])],
                            [t(fx['indptr']), t(fx['indices'])], t(fx['x']),
                            t(fx['query']), ef, dp)
    assert np.array_equal(top_I.numpy(), fx['top_I'])
    assert np.array_equal(top_D.numpy(), fx['top_D'])
    assert np.array_equal(buf_I.numpy(), fx['stage2_I'])
    assert np.array_equal(buf_D.numpy(), fx['stage2_D'])


@pytest.mark.gpu
def test_device_kernels_reproduce_the_fixture(fx, device):
    dp, ef, k = fx['dp'], fx['ef'], fx['k']
    B = fx['query'].shape[0]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    storage_cuda = t(fx['x'][fx['nodelist']][:, :dp]).to(device)
    query_cuda = t(fx['query'][:, :dp]).to(device)
    sub_cuda = [t(fx['sub_indptr']).to(device), t(fx['sub_indices']).to(device),
                t(fx['mapping']).to(device)]
    kernels.traverse_cuda(out_I, out_D, sub_cuda[0], sub_cuda[1], sub_cuda[2],
                          storage_cuda, query_cuda, t(fx['init_I']).to(device),
                          t(fx['init_D']).to(device), fx['deg'])
    assert_same_search(out_I.flatten(1).cpu().numpy(), out_D.flatten(1).cpu().numpy(),
                       fx['cand_I'], fx['cand_D'])
    top_I, top_D = kernels.pipeline(
        graph=[t(fx['indptr']), t(fx['indices'])],
        subgraph=[t(fx['sub_indptr']), t(fx['sub_indices'])],
        subgraph_cuda=sub_cuda, storage=t(fx['x']), storage_cuda=storage_cuda,
        query=t(fx['query']), query_cuda=query_cuda,
        initial_I=t(fx['init_I']).to(device), initial_D=t(fx['init_D']).to(device),
        n_neighbors=fx['deg'], k=k, ef_search=ef, d_principle=dp, chunk_size=8)
    assert np.array_equal(top_I.numpy(), fx['top_I'])
    assert np.array_equal(top_D.numpy(), fx['top_D'])
