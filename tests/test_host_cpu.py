"""The product's host stages (csrc/host_search.cpp through the C ABI and the
`kernels` wrappers) against the oracle: bit-identical outputs, plus the
argument checks of the reference's CHECK_CPU / TORCH_CHECK lines."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels
from common import Problem


@pytest.fixture(scope='module')
def problem():
    return Problem(n=5000, d=64, deg=32, sample_ratio=0.25, seed=5, n_query=100)


@pytest.mark.parametrize('ef,k', [(10, 10), (64, 10), (100, 100), (16, 40), (700, 10)])
def test_traverse_cpu_equals_oracle(problem, ef, k):
    p = problem
    B = p.query.size(0)
    init_I, init_D = p.entries(32, seed=ef)
    out_I = torch.empty(B, k, dtype=torch.long)
    out_D = torch.empty(B, k)
    kernels.traverse_cpu(out_I, out_D, init_I.clone(), init_D.clone(),
                         p.indptr, p.indices, p.x, p.query, ef)
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_cpu(ref_I, ref_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        p.indptr.numpy(), p.indices.numpy(), p.x.numpy(),
                        p.query.numpy(), ef)
    assert np.array_equal(out_I.numpy(), ref_I)
    assert np.array_equal(out_D.numpy(), ref_D)


@pytest.mark.parametrize('ef,dp,n_init', [(8, 32, 32), (32, 16, 128), (64, 64, 256)])
def test_traverse_refine_equals_oracle(problem, ef, dp, n_init):
    p = problem
    B, k = p.query.size(0), 10
    init_I, init_D = p.entries(n_init, seed=ef, dp=dp)
    sub = [p.sub_indptr, p.sub_indices]
    full = [p.indptr, p.indices]
    out = [torch.empty(B, k, dtype=torch.long), torch.empty(B, k),
           torch.empty(B, n_init, dtype=torch.long), torch.empty(B, n_init)]
    entry_D = init_D.clone()
    kernels.traverse_refine(out[0], out[1], out[2], out[3], init_I.clone(),
                            entry_D, sub, full, p.x, p.query, ef, dp)
    ref = [np.empty((B, k), np.int64), np.empty((B, k), np.float32),
           np.empty((B, n_init), np.int64), np.empty((B, n_init), np.float32)]
    ref_entry_D = init_D.numpy().copy()
    oracle.traverse_refine(ref[0], ref[1], ref[2], ref[3], init_I.numpy().copy(),
                           ref_entry_D, [g.numpy() for g in sub],
                           [g.numpy() for g in full], p.x.numpy(),
                           p.query.numpy(), ef, dp)
    for a, b in zip(out, ref):
        assert np.array_equal(a.numpy(), b)
    assert np.array_equal(entry_D.numpy(), ref_entry_D)
    # the pipeline's aliased form (pipeline_cpu.cpp:110-114)
    hI, hD = init_I.clone(), init_D.clone()
    kernels.traverse_refine(out[0], out[1], hI, hD, hI, hD, sub, full, p.x,
                            p.query, ef, dp)
    assert np.array_equal(out[0].numpy(), ref[0])
    assert np.array_equal(hI.numpy(), ref[2]) and np.array_equal(hD.numpy(), ref[3])


def test_long_rows():
    """Rows of 400 floats (the small cases have 64): host stages bit-identical
    to the oracle."""
    p = Problem(n=3000, d=400, n_centers=12, deg=32, sample_ratio=0.5, seed=17,
                n_query=60)
    B, k, ef, dp, n_init = 60, 10, 24, 32, 64
    init_I, init_D = p.entries(32, seed=3)
    out_I = torch.empty(B, k, dtype=torch.long)
    out_D = torch.empty(B, k)
    kernels.traverse_cpu(out_I, out_D, init_I.clone(), init_D.clone(),
                         p.indptr, p.indices, p.x, p.query, ef)
    ref_I = np.empty((B, k), np.int64)
    ref_D = np.empty((B, k), np.float32)
    oracle.traverse_cpu(ref_I, ref_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        p.indptr.numpy(), p.indices.numpy(), p.x.numpy(),
                        p.query.numpy(), ef)
    assert np.array_equal(out_I.numpy(), ref_I) and np.array_equal(out_D.numpy(), ref_D)
    init_I, init_D = p.entries(n_init, seed=4, dp=dp, sampled_only=True)
    sub, full = [p.sub_indptr, p.sub_indices], [p.indptr, p.indices]
    out = [torch.empty(B, k, dtype=torch.long), torch.empty(B, k),
           torch.empty(B, n_init, dtype=torch.long), torch.empty(B, n_init)]
    kernels.traverse_refine(out[0], out[1], out[2], out[3], init_I.clone(),
                            init_D.clone(), sub, full, p.x, p.query, ef, dp)
    ref = [np.empty((B, k), np.int64), np.empty((B, k), np.float32),
           np.empty((B, n_init), np.int64), np.empty((B, n_init), np.float32)]
    oracle.traverse_refine(ref[0], ref[1], ref[2], ref[3], init_I.numpy().copy(),
                           init_D.numpy().copy(), [g.numpy() for g in sub],
                           [g.numpy() for g in full], p.x.numpy(),
                           p.query.numpy(), ef, dp)
    for a, b in zip(out, ref):
        assert np.array_equal(a.numpy(), b)


def test_host_argument_errors(problem):
    p = problem
    B = p.query.size(0)
    init_I, init_D = p.entries(8, seed=1)
    good = dict(output_I=torch.empty(B, 10, dtype=torch.long),
                output_D=torch.empty(B, 10), initial_I=init_I, initial_D=init_D,
                indptr=p.indptr, indices=p.indices, storage=p.x, query=p.query,
                ef_search=16)
    kernels.traverse_cpu(**good)
    for key, bad in [('query', p.query.double()), ('indices', p.indices.int()),
                     ('output_D', torch.empty(B, 9)),
                     ('initial_I', init_I[:, :4]), ('storage', p.x[:, :32]),
                     ('ef_search', 4096), ('output_I', torch.empty(B + 1, 10, dtype=torch.long))]:
        with pytest.raises(RuntimeError):
            kernels.traverse_cpu(**{**good, key: bad})
    with pytest.raises(RuntimeError):
        kernels.traverse_refine(good['output_I'], good['output_D'], init_I, init_D,
                                init_I, init_D, [p.sub_indptr], [p.indptr, p.indices],
                                p.x, p.query, 16, 32)
    with pytest.raises(RuntimeError):      # d_principle must be a multiple of 8
        kernels.traverse_refine(good['output_I'], good['output_D'], init_I.clone(),
                                init_D.clone(), init_I.clone(), init_D.clone(),
                                [p.sub_indptr, p.sub_indices], [p.indptr, p.indices],
                                p.x, p.query, 16, 12)
