"""Chunk pipeline and index modules on the GPU.

`pipeline` must equal the unchunked composition traverse_cuda ->
traverse_refine bit for bit (every piece is deterministic); the invariants of
the reference's own tests hold on top (test/kernel/test_pipeline.py:60-92,
test/module/test_entry.py, test_staged.py:42-50)."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import kernels, layers, utils
from common import Problem, assert_same_search

pytestmark = pytest.mark.gpu


def compose(p, dp, ef, k, init_I, init_D, device):
    B = p.query.size(0)
    out_I = torch.empty(B, 4, ef, dtype=torch.long, device=device)
    out_D = torch.empty(B, 4, ef, dtype=torch.float, device=device)
    kernels.traverse_cuda(out_I, out_D, p.sub_indptr.to(device),
                          p.sub_indices.to(device), p.mapping.to(device),
                          p.x[p.nodelist][:, :dp].contiguous().to(device),
                          p.query[:, :dp].contiguous().to(device),
                          init_I.to(device), init_D.to(device), p.deg)
    buf_I, buf_D = out_I.flatten(1).cpu(), out_D.flatten(1).cpu()
    top_I = np.empty((B, k), np.int64)
    top_D = np.empty((B, k), np.float32)
    bI, bD = buf_I.numpy().copy(), buf_D.numpy().copy()
    oracle.traverse_refine(top_I, top_D, bI, bD, bI, bD,
                           [p.sub_indptr.numpy(), p.sub_indices.numpy()],
                           [p.indptr.numpy(), p.indices.numpy()], p.x.numpy(),
                           p.query.numpy(), ef, dp)
    return top_I, top_D


@pytest.mark.parametrize('dp,ef,chunk', [(64, 16, 32), (32, 64, 128), (64, 8, 256)])
def test_pipeline_equals_unchunked_composition(dp, ef, chunk, device):
    p = Problem(n=6000, d=64, deg=32, sample_ratio=0.25, seed=31, n_query=256)
    k = 10
    init_I, init_D = p.entries(32, seed=9, dp=dp)
    ref_I, ref_D = compose(p, dp, ef, k, init_I, init_D, device)
    args = dict(
        graph=[p.indptr, p.indices], subgraph=[p.sub_indptr, p.sub_indices],
        subgraph_cuda=[p.sub_indptr.to(device), p.sub_indices.to(device),
                       p.mapping.to(device)],
        storage=p.x, storage_cuda=p.x[p.nodelist][:, :dp].contiguous().to(device),
        query=p.query, query_cuda=p.query[:, :dp].contiguous().to(device),
        initial_I=init_I.to(device), initial_D=init_D.to(device),
        n_neighbors=p.deg, k=k, ef_search=ef, d_principle=dp, chunk_size=chunk)
    for _ in range(2):                      # second call reuses the buffers
        top_I, top_D = kernels.pipeline(**args)
        assert not top_I.is_cuda and top_I.shape == (256, k)
        assert np.array_equal(top_I.numpy(), ref_I)
        assert np.array_equal(top_D.numpy(), ref_D)
    # test_pipeline.py:86-92: returned D is the full-dimension distance
    target = torch.cdist(p.query.unsqueeze(1), p.x[top_I]).squeeze(1).square()
    assert torch.allclose(top_D, target, atol=1e-3)
    with pytest.raises(RuntimeError):       # pipeline_cpu.cpp:58
        kernels.pipeline(**{**args, 'chunk_size': 100})
    with pytest.raises(RuntimeError):
        kernels.pipeline(**{**args, 'query': p.query.to(device)})


def test_index_entry_on_gpu(device):
    # test_entry.py:5-42
    x = utils.gaussian_mixture(70000, 64, 16, 1.0, seed=1)
    q = utils.gaussian_mixture(300, 64, 16, 1.0, seed=2, center_seed=1)
    target = utils.brute_force_topk(q, x, 64)
    for method in ['random32', 'router16x32', 'router32x32']:
        index = layers.IndexEntry(d_model=64, method=method, seed=5).train(x)
        index = index.to(device)
        EP_I, EP_D = index.search(q.to(device))
        EP_I, EP_D = EP_I.cpu(), EP_D.cpu()
        assert EP_I.shape == EP_D.shape and EP_I.size(0) == 300
        assert utils.recall(EP_I, target[:, :EP_I.size(-1)]) != 0.0
        ref = torch.cdist(q.unsqueeze(1), x[EP_I]).squeeze(1).square()
        assert torch.allclose(EP_D, ref, atol=1e-3)


def test_index_staged_end_to_end(device):
    # test_staged.py:19-50, on a seeded mixture instead of deep-64k
    n, d, dp, k = 30000, 64, 32, 10
    x = utils.gaussian_mixture(n, d, 32, 1.0, seed=41, decay=0.5)
    q = utils.gaussian_mixture(512, d, 32, 1.0, seed=42, center_seed=41, decay=0.5)
    target = utils.brute_force_topk(q, x, k)
    index = layers.IndexStaged(d_model=d, d_principle=dp, sample_ratio=0.25,
                               graph_method='nsw32', entry_method='router16x32',
                               seed=3, build_device=str(device))
    index.train(x)
    index.to(device)
    top_I, top_D = index.search(q, k=k, ef_search=32, chunk_size=128)
    assert utils.recall(top_I, target) > 0.90
    ref = torch.cdist(q.unsqueeze(1), x[top_I]).squeeze(1).square()
    assert torch.allclose(top_D, ref, atol=1e-3)
    # chunking does not change the answer
    again_I, again_D = index.search(q, k=k, ef_search=32, chunk_size=512)
    assert torch.equal(again_I, top_I) and torch.equal(again_D, top_D)
    # the refine on the device gives the host refine's answer (same rotated
    # query: both rotate it on the device)
    dev_I, dev_D = index.search(q, k=k, ef_search=32, refine='device')
    assert not dev_I.is_cuda
    assert_same_search(dev_I.numpy(), dev_D.numpy(), top_I.numpy(), top_D.numpy())
    # a large batch runs as two halves on two streams: same rows
    big_I, big_D = index.search(q.repeat(5, 1), k=k, ef_search=32, refine='device')
    for i in range(5):
        assert torch.equal(big_I[512 * i:512 * (i + 1)], dev_I)
        assert torch.equal(big_D[512 * i:512 * (i + 1)], dev_D)
    # a query that is already on the device: same rotation, same answer
    gpu_I, gpu_D = index.search(q.to(device), k=k, ef_search=32, refine='device')
    assert torch.equal(gpu_I, dev_I) and torch.equal(gpu_D, dev_D)
    # candidates from the wide mode of the traversal: a search of the same
    # quality (its ids are not promised to be the exact mode's)
    wide_I, wide_D = index.search(q, k=k, ef_search=32, refine='device',
                                  traversal='wide')
    assert abs(utils.recall(wide_I, target) - utils.recall(dev_I, target)) <= 0.002
    ref = torch.cdist(q.unsqueeze(1), x[wide_I]).squeeze(1).square()
    assert torch.allclose(wide_D, ref, atol=1e-3)
    # the reference's host matmul instead: another summation order, results
    # of the same quality
    host_I, host_D = index.search(q, k=k, ef_search=32, chunk_size=128,
                                  rotate='host')
    assert abs(utils.recall(host_I, target) - utils.recall(top_I, target)) < 0.005
    assert float((host_I == top_I).float().mean()) > 0.99
    # a reloaded checkpoint searches identically
    import io
    blob = io.BytesIO()
    torch.save(index.dump(), blob)
    blob.seek(0)
    clone = layers.IndexStaged.load(blob)
    clone.to(device)
    clone_I, clone_D = clone.search(q, k=k, ef_search=32, chunk_size=128)
    assert torch.equal(clone_I, top_I) and torch.equal(clone_D, top_D)


def test_command_line_benchmark_prints_the_reference_lines(device, capsys):
    """script/bench_1.py:57-60: one `method: recall=…, duration=…ms` line per
    ef_search and method, then the records."""
    import re
    from pilotann_amd import cli
    records = cli.main(['--dataset', 'synth:20000x64:16:0.5', '--d_principle', '32',
                        '--n_neighbors', '32', '--router', 'router16x32',
                        '--ef_search', '16,32', '--n_queries', '256',
                        '--n_repeats', '3', '--device', str(device)])
    out = capsys.readouterr().out
    lines = re.findall(r'^(search-pilot|host-cpu): recall=(\d\.\d{3}), '
                       r'duration=(\d+\.\d{3})ms$', out, flags=re.M)
    assert [m for m, _, _ in lines] == ['search-pilot'] * 2 + ['host-cpu'] * 2
    assert all(0.5 < float(r) <= 1.0 for _, r, _ in lines)
    assert set(records) == {'search-pilot', 'host-cpu'}
    assert [r['ef_search'] for r in records['search-pilot']] == [16, 32]
    # more effort, better recall
    assert records['search-pilot'][1]['recall'] >= records['search-pilot'][0]['recall']
    # the labelled wide traversal: device refine only, recall within a point
    wide = cli.main(['--dataset', 'synth:20000x64:16:0.5', '--d_principle', '32',
                     '--n_neighbors', '32', '--router', 'router16x32',
                     '--ef_search', '32', '--n_queries', '256', '--n_repeats', '3',
                     '--refine', 'device', '--traversal', 'wide',
                     '--methods', 'search-pilot', '--device', str(device)])
    assert abs(wide['search-pilot'][0]['recall']
               - records['search-pilot'][1]['recall']) < 0.02
    with pytest.raises(SystemExit):
        cli.main(['--traversal', 'wide', '--device', str(device)])


def test_command_line_benchmark_reads_the_reference_dataset_layout(device, capsys, tmp_path):
    """`--dataset deep-1m` as script/bench_1.py:32-34 passes it on: base,
    queries and ground truth in the .fbin / .ibin layout of
    pilot_ann/utils/loader.py:43-50,92-148 under the data root."""
    import os
    import re
    import numpy as np
    from pilotann_amd import cli, utils
    from pilotann_amd.utils.loader import write_bins
    base = utils.gaussian_mixture(20000, 64, 16, 1.0, seed=3, normalize=True, decay=0.5)
    query = utils.gaussian_mixture(512, 64, 16, 1.0, seed=4, center_seed=3,
                                   normalize=True, decay=0.5)
    truth = utils.brute_force_topk(query, base, 100)
    folder = tmp_path / 'deep-1m'
    os.makedirs(folder)
    write_bins(folder / 'base.fbin', base.numpy())
    write_bins(folder / 'query.fbin', query.numpy())
    write_bins(folder / 'groundtruth.ibin', truth.numpy().astype(np.int32))
    records = cli.main(['--dataset', 'deep-1m', '--data_root', str(tmp_path),
                        '--d_principle', '32', '--n_neighbors', '32',
                        '--router', 'router16x32', '--ef_search', '32',
                        '--n_queries', '256', '--n_repeats', '2',
                        '--methods', 'search-pilot', '--device', str(device)])
    out = capsys.readouterr().out
    assert '[hnsw] dataset: deep-1m, d_model: 64' in out
    assert re.search(r'^search-pilot: recall=\d\.\d{3}, duration=\d+\.\d{3}ms$', out, flags=re.M)
    assert records['search-pilot'][0]['recall'] > 0.7
    with pytest.raises(SystemExit):
        cli.main(['--dataset', 'sift-1m', '--device', str(device)])
