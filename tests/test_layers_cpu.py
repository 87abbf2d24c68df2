"""Index modules on the CPU: the parts of pilot_ann/layers that need no GPU
(test/module/test_entry.py:44-49, test_dump.py)."""
import io

import pytest
import torch

from pilotann_amd import layers, utils


def test_index_entry_random_on_cpu():
    x = utils.gaussian_mixture(5000, 32, 4, 1.0, seed=1)
    q = utils.gaussian_mixture(40, 32, 4, 1.0, seed=2, center_seed=1)
    for method in ['random32', 'random64']:
        index = layers.IndexEntry(d_model=32, method=method, seed=7)
        assert index.train(x) is index
        EP_I, EP_D = index.search(q)
        n = int(method.removeprefix('random'))
        assert EP_I.shape == EP_D.shape == (40, n)
        assert index.nodes() == EP_I[0].tolist()
        target = torch.cdist(q.unsqueeze(1), x[EP_I]).squeeze(1).square()
        assert torch.allclose(EP_D, target, atol=1e-3)
    with pytest.raises(RuntimeError):
        layers.IndexEntry(d_model=16).train(x)
    with pytest.raises(NotImplementedError):
        layers.IndexEntry(d_model=32, method='grid8').train(x)


def test_index_staged_train_dump_load():
    x = utils.gaussian_mixture(3000, 32, 4, 1.0, seed=3, decay=0.5)
    index = layers.IndexStaged(d_model=32, d_principle=16, sample_ratio=0.25,
                               graph_method='nsw16', entry_method='router8x32',
                               seed=11)
    index.train(x)
    assert index.n_neighbors == 16 and index.graph_type == 'nsw'
    assert index.storage.shape == (3000, 32) and index.VT.shape == (32, 32)
    assert torch.allclose(index.storage @ index.VT, x, atol=1e-3)
    assert index.entry.entry_vectors.shape == (8, 32, 16)
    assert index.entry.route_vectors.shape == (8, 16)
    ckpt = index.dump()
    assert set(ckpt['config']) == {'d_model', 'd_principle', 'graph_method',
                                   'entry_method'}
    keys = set(ckpt['state_dict'])
    assert {'VT', 'storage', 'mapping', 'nodelist', 'subgraph.indptr',
            'subgraph.indices', 'fullgraph.indptr', 'fullgraph.indices',
            'entry.entry_nodes', 'entry.entry_vectors',
            'entry.route_vectors'} == keys
    blob = io.BytesIO()
    torch.save(ckpt, blob)
    blob.seek(0)
    clone = layers.IndexStaged.load(blob)
    for name in keys:
        a = ckpt['state_dict'][name]
        b = clone.state_dict()[name]
        assert torch.equal(a, b), name
    assert clone.n_neighbors == 16 and clone.d_principle == 16


def test_search_cpu_is_the_whole_search_on_the_host():
    """`IndexStaged.search_cpu`: rotation, router entries, host search on the
    full graph — finds the true neighbours and reports full-dimension
    distances (a rotation keeps them)."""
    x = utils.gaussian_mixture(6000, 64, 16, 1.0, seed=1, decay=0.5)
    q = utils.gaussian_mixture(100, 64, 16, 1.0, seed=2, center_seed=1, decay=0.5)
    target = utils.brute_force_topk(q, x, 10)
    for entry_method in ('router8x32', 'random32'):
        index = layers.IndexStaged(64, 32, 0.25, 'nsw32', entry_method, seed=3)
        index.train(x)
        top_I, top_D = index.search_cpu(q, 10, 64)
        assert utils.recall(top_I, target) > 0.95
        ref = (q.unsqueeze(1) - x[top_I]).square().sum(-1)
        assert torch.allclose(top_D, ref, atol=1e-3)
