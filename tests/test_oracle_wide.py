"""`oracle.traverse_wide`, the CPU restatement of the library's wide mode (no
counterpart in the reference), against what fixes it: brute force where the
pool holds every node, and graphs built by hand for the stop rule, the cap on
expansions and the grouping of a step."""
import numpy as np
import torch

import oracle
from pilotann_amd import utils


def padded(rows, deg):
    """CSR with `deg` slots a row, -1 filled, from lists of neighbours."""
    n = len(rows)
    indices = np.full((n, deg), -1, np.int64)
    for i, r in enumerate(rows):
        indices[i, :len(r)] = r
    return np.arange(n + 1, dtype=np.int64) * deg, indices.reshape(-1)


def points(coord):
    """8-dimensional points with the given first coordinate (the others
    zero): squared distance from the origin = coord², exactly."""
    x = np.zeros((len(coord), 8), np.float32)
    x[:, 0] = np.asarray(coord, np.float32)
    return x


def search(x, rows, entries, k, width, deg=4, mapping=None):
    indptr, indices = padded(rows, deg)
    n = len(x)
    if mapping is None:
        mapping = np.arange(n, dtype=np.int64)
    q = np.zeros((1, 8), np.float32)
    init_I = np.asarray([entries], np.int64)
    init_D = (x[init_I[0]] ** 2).sum(-1)[None].astype(np.float32)
    out_I = np.empty((1, k), np.int64)
    out_D = np.empty((1, k), np.float32)
    cnt = np.zeros(5, np.int64)
    oracle.traverse_wide(out_I, out_D, init_I, init_D, indptr, indices, mapping,
                         x, q, width, cnt)
    return out_I[0], out_D[0], cnt


def test_brute_force_when_the_pool_holds_every_node():
    n, d, k = 120, 16, 128
    x = utils.gaussian_mixture(n, d, 4, 0.8, seed=2)
    q = utils.gaussian_mixture(16, d, 4, 0.8, seed=3, center_seed=2)
    indptr, indices = utils.graph_init(x, 'nsw', 8)
    assert bool(utils.reachable(indices.view(n, 8), torch.tensor([5])).all())
    target = torch.cdist(q.double(), x.double()).square()
    order = torch.argsort(target, dim=-1).numpy()
    init_I = np.full((16, 1), 5, np.int64)
    init_D = ((q - x[5]) ** 2).sum(-1, keepdim=True).numpy().astype(np.float32)
    for width in (1, 2, 4):
        out_I = np.empty((16, k), np.int64)
        out_D = np.empty((16, k), np.float32)
        oracle.traverse_wide(out_I, out_D, init_I, init_D, indptr.numpy(),
                             indices.numpy(), np.arange(n, dtype=np.int64),
                             x.numpy(), q.numpy(), width)
        assert np.array_equal(out_I[:, :n], order)
        assert (out_I[:, n:] == -1).all() and np.isinf(out_D[:, n:]).all()
        assert np.allclose(out_D[:, :n], np.take_along_axis(target.numpy(), order, 1),
                           rtol=1e-5)


def chain(n):
    rows = [[i + 1] if i + 1 < n else [] for i in range(n)]
    return points(np.arange(n, dtype=np.float32) + 1.0), rows


def test_the_search_ends_when_nothing_in_the_pool_is_left_to_expand():
    """A chain of nodes ever farther away: the pool of 64 takes the first 64,
    the 65th is not below its last key, and with every candidate of the pool
    expanded the search stops, well below the cap of 128."""
    x, rows = chain(300)
    for width in (1, 4):
        I, D, cnt = search(x, rows, [0], 64, width)
        assert cnt[0] == 64 and cnt[2] == 64        # node 64 was looked at, not taken
        assert np.array_equal(I, np.arange(64))
        assert np.array_equal(D, (np.arange(64, dtype=np.float32) + 1.0) ** 2)


def test_the_cap_on_expansions():
    """min(1024, 2k) expansions: k = 16 stops the chain after 32, the pool
    then holds nodes 0..32 and the 16 best are returned."""
    x, rows = chain(300)
    I, D, cnt = search(x, rows, [0], 16, 3)
    assert cnt[0] == 32
    assert np.array_equal(I, np.arange(16))


def test_a_step_expands_its_candidates_together():
    """Two entries h1, h2 with one child each (a, b) and one grandchild each
    (a2, b2, the nearest nodes); k = 2 allows four expansions.  Width 2: h1
    and h2, then a and b — both grandchildren found.  Width 1 follows the
    best candidate alone: h1, a, a2, then h2 — b2 is never reached."""
    #           h1  h2   a    b    a2   b2
    x = points([5., 6., 1.0, 2.0, 0.5, 0.25])
    rows = [[2], [3], [4], [5], [], []]
    I, D, cnt = search(x, rows, [0, 1], 2, 2)
    assert cnt[0] == 4 and I.tolist() == [5, 4]
    I, D, cnt = search(x, rows, [0, 1], 2, 1)
    assert cnt[0] == 4 and I.tolist() == [4, 2]


def test_entries_without_a_row_unused_entries_and_row_ends():
    """An entry outside the sample keeps its global id, is returned with its
    given distance and is never expanded; a negative entry is skipped; a row
    of neighbours ends at its first negative id."""
    x = points([3., 1., 2., 0.5, 0.25])      # squared distances 9, 1, 4, 0.25, 0.0625
    rows = [[1, -1, 4], [2], [], [4], []]          # node 4 sits behind a -1 in row 0
    mapping = np.asarray([0, 1, 2, -1, 3], np.int64)   # node 3 has no storage row
    indptr, indices = padded(rows, 4)
    q = np.zeros((1, 8), np.float32)
    init_I = np.asarray([[0, 3, -1]], np.int64)
    init_D = np.asarray([[9., 0.25, 81.]], np.float32)
    out_I = np.empty((1, 4), np.int64)
    out_D = np.empty((1, 4), np.float32)
    cnt = np.zeros(5, np.int64)
    oracle.traverse_wide(out_I, out_D, init_I, init_D, indptr, indices, mapping,
                         x, q, 4, cnt)
    assert out_I[0].tolist() == [3, 1, 2, 0]
    assert out_D[0].tolist() == [0.25, 1.0, 4.0, 9.0]
    assert cnt[0] == 3            # nodes 0, 1, 2; node 3 cannot be expanded, 4 is never seen
