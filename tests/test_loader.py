"""`utils.DataLoader` on the reference's dataset names and file layouts
(pilot_ann/utils/loader.py, test/module/test_loader.py), with small files
written into a temporary directory, and `utils.search_simple` on a built
graph (test/kernel/test_graphs.py)."""
import os
import random

import numpy as np
import pytest
import torch

from pilotann_amd import utils
from pilotann_amd.utils import loader as L


def brute(query, storage, k):
    return torch.topk(torch.cdist(query.double(), storage.double()), k, dim=-1,
                      largest=False).indices


def test_bins_round_trip(tmp_path):
    a = np.arange(35, dtype=np.float32).reshape(7, 5)
    L.write_bins(tmp_path / 'a.fbin', a)
    raw = np.fromfile(tmp_path / 'a.fbin', dtype=np.int32)
    assert raw[0] == 7 and raw[1] == 5 and raw.size == 2 + 35
    assert np.array_equal(L.read_bins(str(tmp_path / 'a.fbin'), np.float32), a)
    ids = np.arange(12, dtype=np.int32).reshape(3, 4)
    L.write_bins(tmp_path / 'g.ibin', ids)
    assert np.array_equal(L.read_bins(str(tmp_path / 'g.ibin'), np.int32), ids)
    with open(tmp_path / 'short.fbin', 'wb') as f:
        np.asarray([7, 5], dtype=np.int32).tofile(f)
        a[:3].tofile(f)
    with pytest.raises(ValueError):
        L.read_bins(str(tmp_path / 'short.fbin'), np.float32)


def test_search_target_is_exact_and_ordered():
    g = torch.Generator().manual_seed(1)
    q, x = torch.randn(50, 16, generator=g), torch.randn(3000, 16, generator=g)
    # pieces smaller than the base: the running top-k is merged across them
    got = L.search_target(q, x, top_k=20, chunk_size=1 << 20)
    assert torch.equal(got, brute(q, x, 20))
    assert torch.equal(L.search_target(q, x, top_k=20, chunk_size=16), brute(q, x, 20))
    assert L.search_target(q, x[:5], top_k=20).shape == (50, 5)


def test_fuzz_names():
    for name, around in (('fuzz-16k', 16384), ('fuzz-64k', 65536)):
        if around == 65536:
            continue          # the 64k ground truth is half a minute of host time
        a = utils.DataLoader(name, seed=5)
        assert a.d_model in L.FUZZ_WIDTHS
        assert around // 2 <= a.n_storage <= 2 * around
        assert a.query.shape == (4096, a.d_model) and a.target.shape == (4096, 100)
        assert float(a.storage.min()) >= -1.0 and float(a.storage.max()) < 1.0
        assert torch.equal(a.target[:16, :10], brute(a.query[:16], a.storage, 10))
        query, target = a.load_query(1024, k=10)
        assert query.shape == (1024, a.d_model) and target.shape == (1024, 10)
        with pytest.raises(RuntimeError):
            a.load_query(4, k=101)
        b = utils.DataLoader(name, seed=5)
        assert torch.equal(a.storage, b.storage) and torch.equal(a.target, b.target)
    with pytest.raises(NotImplementedError):
        utils.DataLoader('fuzz-1m')
    with pytest.raises(NotImplementedError):
        utils.DataLoader('sift-1m')


def test_bin_families(tmp_path):
    g = torch.Generator().manual_seed(2)
    base = torch.randn(70000, 8, generator=g)
    query = torch.randn(64, 8, generator=g)
    folder = tmp_path / 'deep-1m'
    os.makedirs(folder)
    L.write_bins(folder / 'base.fbin', base.numpy())
    L.write_bins(folder / 'query.fbin', query.numpy())
    L.write_bins(folder / 'groundtruth.ibin', brute(query, base, 100).numpy().astype(np.int32))
    # the file holds fewer rows than the name asks for: taken as it is
    whole = utils.DataLoader('deep-1m', root=str(tmp_path))
    assert whole.n_storage == 70000 and whole.d_model == 8
    assert torch.equal(whole.storage, base)
    assert whole.target.dtype == torch.long
    assert torch.equal(whole.target, brute(query, base, 100))
    # more rows than the name asks for: a subset without repeats and its own
    # ground truth
    cut = utils.DataLoader('deep-64k', root=str(tmp_path), seed=1)
    assert cut.n_storage == 65536
    assert torch.unique(cut.storage, dim=0).size(0) == 65536
    assert torch.equal(cut.target[:, :10], brute(query, cut.storage, 10))
    again = utils.DataLoader('deep-64k', root=str(tmp_path), seed=1)
    assert torch.equal(cut.storage, again.storage)
    q, t = cut.load_query(1024, k=10)
    assert q.shape == (1024, 8) and t.shape == (1024, 10)
    # queries without a base file (loader.py:137-138)
    os.makedirs(tmp_path / 'text2img-10m')
    L.write_bins(tmp_path / 'text2img-10m' / 'query.fbin', query.numpy())
    L.write_bins(tmp_path / 'text2img-10m' / 'groundtruth.ibin',
                 np.zeros((64, 100), dtype=np.int32))
    only = utils.DataLoader('text2img-10m', root=str(tmp_path))
    assert only.storage is None and only.query.shape == (64, 8)


def test_numpy_families(tmp_path):
    g = torch.Generator().manual_seed(3)
    base = torch.randn(66000, 8, generator=g)
    query = torch.randn(32, 8, generator=g)
    folder = tmp_path / 'laion-1m'
    os.makedirs(folder)
    np.save(folder / 'query.npy', query.numpy())
    np.save(folder / 'groundtruth.npy', brute(query, base, 100).numpy())
    np.save(folder / 'img_emb_0.npy', base[:30000].numpy())
    np.save(folder / 'img_emb_1.npy', base[30000:].numpy())
    whole = utils.DataLoader('laion-1m', root=str(tmp_path))
    assert torch.equal(whole.storage, base)
    cut = utils.DataLoader('laion-64k', root=str(tmp_path), seed=4)
    assert cut.n_storage == 65536
    assert torch.equal(cut.target[:, :10], brute(query, cut.storage, 10))
    # every kept row is a row of the files
    rows = {row.tobytes() for row in base.numpy()}
    assert all(row.tobytes() in rows for row in cut.storage.numpy())
    assert len({row.tobytes() for row in cut.storage.numpy()}) == 65536


def test_search_simple_on_a_built_graph():
    """The recall floor of the reference's graph test for this width
    (test_graphs.py:55-64: 0.60 for d <= 128) with its parameters: 64
    neighbours, ef_search 32, top-10."""
    g = torch.Generator().manual_seed(7)
    n, d, k = 4096, 64, 10
    x = 2.0 * (torch.rand(n, d, generator=g) - 0.5)
    q = 2.0 * (torch.rand(32, d, generator=g) - 0.5)
    indptr, indices = utils.graph_init(x, 'nsw', n_neighbors=64)
    indptr, indices = indptr.tolist(), indices.tolist()
    rng = random.Random(0)
    found = []
    for i in range(q.size(0)):
        out = utils.search_simple(indptr, indices, list(range(n)), x, q[i], k=k,
                                  ef_search=32, rng=rng)
        assert len(out['topk']) == k and len(set(out['topk'])) == k
        assert out['n_visited'] == len(out['visited']) >= out['n_computed']
        assert out['n_steps'] < 64
        found.append(out['topk'])
    score = utils.recall(torch.tensor(found), brute(q, x, k))
    assert score >= 0.60, score
    # given entries are used before random ones; closed nodes are never returned
    target = brute(q[:1], x, 1)[0].tolist()
    out = utils.search_simple(indptr, indices, list(range(n)), x, q[0], k=1,
                              ef_search=32, ep=list(target), rng=rng)
    assert out['topk'] == target
    out = utils.search_simple(indptr, indices, list(range(n)), x, q[0], k=5,
                              ef_search=32, closedlist=list(target), rng=rng)
    assert target[0] not in out['topk']
