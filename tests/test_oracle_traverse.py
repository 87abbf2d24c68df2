"""Pins of the oracle's search (oracle/oracle.c, after
extension/traverse_cpu.cpp:12-369).  None of them restates the algorithm:
brute force on small graphs where the search must be exhaustive, hand-built
graphs that isolate one rule each with the expected output worked out on
paper, and the invariants the reference's own tests check
(test/kernel/test_traverse_cpu.py:60-84, test_traverse_refine.py:68-95)."""
import numpy as np
import pytest
import torch

import oracle
from pilotann_amd import utils

D = 8            # smallest legal row length (distance.h:35-36)
INF = np.inf


def csr(rows, width=None):
    """Padded CSR with -1 fill from a list of neighbour lists."""
    width = width or max(1, max(len(r) for r in rows))
    indptr = np.arange(len(rows) + 1, dtype=np.int64) * width
    indices = np.full(len(rows) * width, -1, np.int64)
    for i, r in enumerate(rows):
        indices[i * width:i * width + len(r)] = r
    return indptr, indices


def points_on_axis(coords):
    x = np.zeros((len(coords), D), np.float32)
    x[:, 0] = coords
    return x


def search(rows, x, q, entries, entry_d, ef, k, width=None):
    indptr, indices = csr(rows, width)
    out_I = np.empty((1, k), np.int64)
    out_D = np.empty((1, k), np.float32)
    oracle.traverse_cpu(out_I, out_D, np.array([entries], np.int64),
                        np.array([entry_d], np.float32), indptr, indices, x,
                        q.reshape(1, -1).astype(np.float32), ef)
    return out_I[0].tolist(), out_D[0].tolist()


@pytest.mark.parametrize('ef,cap', [(16, 32), (40, 80), (600, 1024)])
def test_iteration_cap_on_a_chain(ef, cap):
    """Node i of a chain lies at coordinate i and links to i + 1 only; the
    query lies beyond the end, so every pop finds one closer node and the
    search never stops on its own.  After min(1024, 2 ef) expansions
    (traverse_cpu.cpp:18,82) the nodes 1..cap are known and nothing else."""
    n = cap + 50
    rows = [[i + 1] if i + 1 < n else [] for i in range(n)]
    x = points_on_axis(np.arange(n))
    q = points_on_axis([n + 10.0])[0]
    k = 8
    I, Dk = search(rows, x, q, [0], [(n + 10.0) ** 2], ef, k)
    assert I == [cap - i for i in range(k)]
    assert Dk == [float((n + 10 - (cap - i)) ** 2) for i in range(k)]


def test_scan_of_a_row_ends_at_the_first_negative():
    """traverse_cpu.cpp:107-109: `break`, not `continue`.  Node 0 lists
    [1, -1, 2, 3]; 2 is the true neighbour of the query but sits after -1."""
    rows = [[1, -1, 2, 3], [], [], []]
    x = points_on_axis([0.0, 5.0, 9.0, 8.0])
    q = points_on_axis([9.0])[0]
    I, Dk = search(rows, x, q, [0], [81.0], 16, 4, width=4)
    assert I == [1, 0, -1, -1]
    assert Dk == [16.0, 81.0, INF, INF]


def test_entries_join_the_results_only_after_the_loop():
    """traverse_cpu.cpp:69-79,138-148.  Heap of 16.  Entry a (distance 1)
    links to 15 nodes r_1..r_15 at distances 4..256; entry b (distance 900)
    links to z, the true nearest node.  The result heap holds discovered
    nodes only, so after a's expansion it has 15 of 16 cells, its threshold is
    still +inf, every r and finally b is popped and z is found.  Were the
    entries in the heap from the start (as traverse_cuda.cu:96-111 does) it
    would be full after r_14, b would be displaced by r_15 and the search
    would stop at r_15 with b unexpanded and z unknown.  After the loop a
    takes the cell of the worst r, b loses against it."""
    # nodes: 0 = a, 1 = b, 2..16 = r_1..r_15, 17 = z
    coords = [1.0, 30.0] + [float(i) for i in range(2, 17)] + [0.5]
    # a lists the r's farthest first: rising keys would run into the leaf rule
    # of heap_replace (next test) and push b out of the open heap
    rows = [list(range(16, 1, -1)), [17]] + [[] for _ in range(16)]
    x = points_on_axis(coords)
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, [0, 1], [1.0, 900.0], 16, 16)
    assert I == [17, 0] + list(range(2, 16))
    assert Dk == [0.25, 1.0] + [float(i * i) for i in range(2, 16)]


def test_entries_in_rising_order_can_be_lost():
    """A consequence of heapq.cuh:47-77 that a restatement must keep: pushing
    entries with rising keys into the empty 32-cell open heap sends every
    walk down the same branch; from the tenth on it ends on the finite leaf
    81 and the entry is dropped, with half of the heap still empty.  Entry 15
    (distance 256), the only link to z, is one of them."""
    coords = [float(i) for i in range(1, 17)] + [0.5]
    rows = [[] for _ in range(17)]
    rows[15] = [16]
    x = points_on_axis(coords)
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, list(range(16)), [c * c for c in coords[:16]],
                   16, 16)
    assert I == list(range(16))          # z (node 16) was never reached


def test_open_list_has_twice_the_heap_size_cells():
    """traverse_cpu.cpp:21-24: HEAP_SIZE = 16 result cells, 2 * 16 = 32 open
    cells: five full levels (cells 0..30) and the lone cell 31 under cell 15.
    Eleven entries arrive with the keys (coordinates, squared)
    1 3 2 5 4 7 6 9 8 10 11.  Stepping heapq.cuh:47-77 by hand, every walk
    goes left at the root and below it, because the left child is the larger
    finite one there:
      1 -> root; 3 -> down the empty left spine to cell 31, rises to cell 1;
      2 -> right of the root (inf beats 3), rises to cell 2;
      5 -> cell 1 (3 > 2), empty below: cell 31, rises to cell 3;
      4 -> cell 1, then right (inf beats 5): rises to cell 4;
      7 -> 1, 3 (5 > 4), empty below: rises to cell 7;   6 -> 1, 3, right: cell 8;
      9 -> 1, 3, 7 (7 > 6), cell 15, cell 31: rises to cell 15;
      8 -> 1, 3, 7, right (inf beats 9): cell 16, a leaf;
      10 -> 1, 3, 7, 15 (9 > 8), its only child 31 is free: stays in cell 31;
      11 -> 1, 3, 7, 15, 31: a leaf holding 10 <= 11: dropped.
    With 33 cells or more cell 15 has a second, free child and 11 is kept;
    with 31 cells or fewer cell 15 is a leaf and 10 is dropped against 9; with
    16 cells 8 overwrites 9 in cell 15 and 10, 11 are dropped.  The entries
    with the keys 9, 10 and 11 are the only links to the three nodes nearest
    to the query: the first two must be found, the third must not.  All
    entries are merged after the loop whether they were expanded or not."""
    coords = [1, 3, 2, 5, 4, 7, 6, 9, 8, 10, 11]
    # nodes 0..10 = the entries in this order; 11, 12, 13 = the near nodes
    rows = [[] for _ in range(14)]
    rows[7] = [11]            # key 9
    rows[9] = [12]            # key 10
    rows[10] = [13]           # key 11, dropped from the open list
    x = points_on_axis([float(c) for c in coords] + [0.5, 0.25, 0.125])
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, list(range(11)),
                   [float(c * c) for c in coords], 16, 16)
    by_key = [0, 2, 1, 4, 3, 6, 5, 8, 7, 9, 10]      # entries, nearest first
    assert I == [12, 11] + by_key + [-1] * 3
    assert Dk == ([0.0625, 0.25] + [float(c * c) for c in range(1, 12)]
                  + [INF] * 3)


def test_candidates_not_better_than_the_worst_kept_stay_out_of_the_open_list():
    """traverse_cpu.cpp:25-39: a distance >= the worst kept result skips the
    result heap *and* the open list.  Such a node could never be expanded (a
    popped key >= worst kept ends the search), so the rule shows only through
    the cell the node would occupy.  Heap of 16, open list of 32 cells.
    A chain a0 -> a1 -> ... -> a9 at coordinates 40, 30, 29, ..., 22 puts nine
    results into the result heap and leaves the open list empty when a9 is
    popped.  a9's row is  r1..r7 (coordinates 1..7), D (-30), Y (10), Z (-10),
    W (8):
      r1..r7 have rising keys: cells 0, 1, 2, 5, 6, 13, 14 (each walk follows
      the larger child, the right spine); the result heap is now full and its
      worst is a1 with 900;
      D has 900 >= 900: skipped.  Y (100): walk 0, 2, 6, 14, both children
      free: cell 29.  Z (100): cell 29 holds Y, 30 is free: cell 30.
      W (64): at cell 14 the children tie (100, 100), the left one is taken:
      W overwrites Y, the only link to the nearest node z.
    The search then pops r1..r7, W, Z and runs dry: z is never seen.
    Were D inserted, it would sit in cell 29, Y would go to 30, Z would
    overwrite D in 29, W would overwrite Z, Y would be expanded and z found."""
    a = [40.0] + [float(c) for c in range(30, 21, -1)]          # nodes 0..9
    r = [float(c) for c in range(1, 8)]                         # nodes 10..16
    coords = a + r + [-30.0, 10.0, -10.0, 8.0, 0.5]
    D_, Y, Z, W, z = 17, 18, 19, 20, 21
    rows = [[i + 1] for i in range(9)] + [list(range(10, 17)) + [D_, Y, Z, W]]
    rows += [[] for _ in range(12)]
    rows[Y] = [z]
    x = points_on_axis(coords)
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, [0], [1600.0], 16, 16)
    assert I[:8] == list(range(10, 17)) + [W]
    assert sorted(I[8:10]) == [Y, Z]
    assert I[10:] == [9, 8, 7, 6, 5, 4]
    assert Dk == ([float(c * c) for c in range(1, 8)] + [64.0, 100.0, 100.0]
                  + [float(c * c) for c in range(22, 28)])


def test_a_popped_key_equal_to_the_worst_kept_ends_the_search():
    """traverse_cpu.cpp:88-90: `u.key >= -buffer_D[0]` stops, equality
    included.  Entries a (coordinate 1) and t (-16, key 256).  a's row holds
    16 nodes at 16, 15, ..., 2 and 1.5 (falling keys: the 32-cell open list
    keeps all of them); they fill the result heap, whose worst is then the
    node at 16 with key 256.  The fifteen nearer ones are popped and expanded
    (empty rows); the next pop returns a key of 256 (t or the node at 16),
    which is not smaller than the worst kept: the search ends and t's only
    neighbour z, the node nearest to the query, is never seen.  After the loop
    a takes the place of the node at 16 and t loses the tie against the new
    worst (heapq.cuh:83)."""
    coords = [1.0, -16.0] + [float(c) for c in range(16, 1, -1)] + [1.5, 0.5]
    z = len(coords) - 1
    rows = [list(range(2, 18)), [z]] + [[] for _ in range(17)]
    x = points_on_axis(coords)
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, [0, 1], [1.0, 256.0], 16, 16)
    assert I == [0, 17] + list(range(16, 2, -1))
    assert Dk == [1.0, 2.25] + [float(c * c) for c in range(2, 16)]


def test_front_padding_when_k_exceeds_the_heap():
    """traverse_cpu.cpp:150-162 with k > HEAP_SIZE: the pops past the heap's
    16 cells return (inf, -1) and land, sign flipped, in front."""
    rows = [[1, 2], [], []]
    x = points_on_axis([3.0, 2.0, 1.0])
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, [0], [9.0], 16, 20, width=2)
    assert I[:4] == [-1] * 4 and Dk[:4] == [-INF] * 4
    assert I[4:7] == [2, 1, 0] and Dk[4:7] == [1.0, 4.0, 9.0]
    assert I[7:] == [-1] * 13 and Dk[7:] == [INF] * 13


def test_unused_and_repeated_entries():
    """Negative entries are skipped (traverse_cpu.cpp:71-73); an entry given
    twice is pushed and merged twice (no de-duplication anywhere)."""
    rows = [[], [], []]
    x = points_on_axis([1.0, 2.0, 3.0])
    q = points_on_axis([0.0])[0]
    I, Dk = search(rows, x, q, [2, -1, 0, 0], [9.0, 123.0, 1.0, 1.0], 16, 4)
    assert I == [0, 0, 2, -1]
    assert Dk == [1.0, 1.0, 9.0, INF]


def test_empty_batch_and_bad_arguments():
    indptr, indices = csr([[]])
    x = points_on_axis([0.0])
    e = np.empty((0, 4), np.int64)
    oracle.traverse_cpu(e, np.empty((0, 4), np.float32), np.empty((0, 1), np.int64),
                        np.empty((0, 1), np.float32), indptr, indices, x,
                        np.empty((0, D), np.float32), 16)
    with pytest.raises(RuntimeError):          # ef_search above the ladder
        oracle.traverse_cpu(np.empty((1, 4), np.int64), np.empty((1, 4), np.float32),
                            np.zeros((1, 1), np.int64), np.zeros((1, 1), np.float32),
                            indptr, indices, x, np.zeros((1, D), np.float32), 4096)


def connected_knn(n, d, deg, seed):
    x = utils.gaussian_mixture(n, d, 4, 0.8, seed=seed)
    ids, _ = utils.knn_graph(x, deg - 2)
    ring = torch.stack([(torch.arange(n) + 1) % n, (torch.arange(n) - 1) % n], 1)
    rows = torch.cat([ids, ring], 1)            # ring edges: one component
    indptr = torch.arange(n + 1) * deg
    return x, indptr.numpy(), rows.flatten().numpy()


@pytest.mark.parametrize('seed,n,d', [(0, 150, 8), (1, 200, 16), (2, 240, 32)])
def test_exhaustive_search_equals_brute_force(seed, n, d):
    """With a heap at least as large as a connected graph and an iteration
    cap above its size the search visits every node: the result must be the
    exact top-k, distances included."""
    x, indptr, indices = connected_knn(n, d, 12, seed)
    q = utils.gaussian_mixture(20, d, 4, 0.8, seed=seed + 50, center_seed=seed)
    k = 10
    g = torch.Generator().manual_seed(seed)
    init_I = torch.randint(high=n, size=[20, 3], generator=g)
    init_D = (q.unsqueeze(1) - x[init_I]).square().sum(-1)
    out_I = np.empty((20, k), np.int64)
    out_D = np.empty((20, k), np.float32)
    cnt = np.zeros(5, np.int64)
    oracle.traverse_cpu(out_I, out_D, init_I.numpy().copy(),
                        init_D.numpy().copy(), indptr, indices, x.numpy(),
                        q.numpy(), 256, cnt)
    exact = torch.cdist(q.double(), x.double()).square()
    top = torch.topk(exact, k, largest=False)
    # a repeated entry would show twice; draw is without repeats here or the
    # set comparison below would say so
    assert [sorted(r) for r in out_I.tolist()] == [sorted(r) for r in top.indices.tolist()]
    assert np.allclose(out_D, top.values.numpy(), rtol=1e-5)
    assert (np.diff(out_D, axis=1) >= 0).all()


@pytest.mark.parametrize('graph_type,ratio', [('nsw', None), ('nsg', None), ('nsw', 0.25)])
def test_reference_invariants_traverse_cpu(graph_type, ratio):
    """test_traverse_cpu.py:60-84: a recall floor and returned D == squared
    distance of returned I (atol 1e-3), here also best-first order."""
    n, d, deg, ef, k, B = 6000, 64, 32, 128, 10, 128
    x = utils.gaussian_mixture(n, d, 8, 1.0, seed=7)
    q = utils.gaussian_mixture(B, d, 8, 1.0, seed=8, center_seed=7)
    target = utils.brute_force_topk(q, x, k)
    indptr, indices = utils.graph_init(x, graph_type, deg)
    if ratio:
        indptr, indices, nodelist, mapping = utils.subgraph_init(
            indptr, indices, x, graph_type, round(ratio * n), deg, seed=1)
    g = torch.Generator().manual_seed(3)
    init_I = torch.randint(high=n, size=[B, ef], generator=g)
    dist = torch.cdist(q, x).square()
    init_D = torch.gather(dist, 1, init_I).contiguous()
    out_I = np.empty((B, k), np.int64)
    out_D = np.empty((B, k), np.float32)
    oracle.traverse_cpu(out_I, out_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        indptr.numpy(), indices.numpy(), x.numpy(), q.numpy(), ef)
    score = utils.recall(torch.from_numpy(out_I), target)
    assert score >= (0.60 / 4 if ratio else 0.60)
    got = torch.gather(dist, 1, torch.from_numpy(out_I))
    assert torch.allclose(torch.from_numpy(out_D), got, atol=1e-3)
    assert (np.diff(out_D, axis=1) >= 0).all()


def test_reference_invariants_traverse_refine():
    """test_traverse_refine.py:68-95: final D and the stage-2 buffer D equal
    the full-dimension squared distances of their ids; recall floor."""
    n, d, deg, ef, k, B = 6000, 64, 64, 32, 10, 128
    dp = 8 * (d // 16)
    x = utils.gaussian_mixture(n, d, 8, 1.0, seed=17)
    q = utils.gaussian_mixture(B, d, 8, 1.0, seed=18, center_seed=17)
    target = utils.brute_force_topk(q, x, k)
    graph = utils.graph_init(x, 'nsw', deg)
    sub = utils.subgraph_init(graph[0], graph[1], x, 'nsw', n // 4, deg, seed=2)
    g = torch.Generator().manual_seed(5)
    init_I = torch.randint(high=n, size=[B, ef], generator=g)
    init_D = torch.gather(torch.cdist(q[:, :dp], x[:, :dp]).square(), 1, init_I)
    out_I, out_D = np.empty((B, k), np.int64), np.empty((B, k), np.float32)
    buf_I, buf_D = np.empty((B, ef), np.int64), np.empty((B, ef), np.float32)
    entry_D = init_D.numpy().copy()
    oracle.traverse_refine(out_I, out_D, buf_I, buf_D, init_I.numpy().copy(),
                           entry_D, [sub[0].numpy(), sub[1].numpy()],
                           [graph[0].numpy(), graph[1].numpy()], x.numpy(),
                           q.numpy(), ef, dp)
    assert utils.recall(torch.from_numpy(out_I), target) >= 0.50
    full = torch.cdist(q, x).square()
    assert torch.allclose(torch.from_numpy(out_D),
                          torch.gather(full, 1, torch.from_numpy(out_I)), atol=1e-3)
    assert (buf_I >= 0).all()
    assert torch.allclose(torch.from_numpy(buf_D),
                          torch.gather(full, 1, torch.from_numpy(buf_I)), atol=1e-3)
    # the entries' distances were completed in place (traverse_cpu.cpp:42-62)
    assert torch.allclose(torch.from_numpy(entry_D),
                          torch.gather(full, 1, init_I), atol=1e-3)


def test_refine_stages_share_the_visited_marks():
    """traverse_cpu.cpp:317-336: stage 3 runs with stage 2's marker.  Node 2
    is evaluated in stage 2 (it enters the buffer); in stage 3 it is reachable
    again from node 3 but already marked, so it is not admitted a second
    time.  With separate marks it would show up twice in the output."""
    # subgraph: 0 -> 2.   full graph: 0 -> 3, 3 -> 2, 1 isolated.
    sub = csr([[2], [], [], []])
    full = csr([[3], [], [], [2]])
    x = points_on_axis([4.0, 9.0, 1.0, 2.0])
    q = points_on_axis([0.0]).astype(np.float32)
    out_I, out_D = np.empty((1, 4), np.int64), np.empty((1, 4), np.float32)
    buf_I, buf_D = np.empty((1, 16), np.int64), np.empty((1, 16), np.float32)
    oracle.traverse_refine(out_I, out_D, buf_I, buf_D,
                           np.array([[0]], np.int64), np.array([[16.0]], np.float32),
                           list(sub), list(full), x, q, 16, D)
    assert buf_I[0].tolist() == [2, 0] + [-1] * 14
    assert out_I[0].tolist() == [2, 3, 0, -1]
    assert out_D[0].tolist() == [1.0, 4.0, 16.0, INF]


def test_refine_expands_two_nodes_on_the_subgraph():
    """traverse_cpu.cpp:9,317-326: stage 2 runs with max_iterations =
    REFINE_STEP = 2.  The subgraph is a chain 0 -> 1 -> 2 -> 3 -> 4 towards
    the query: two expansions (of 0 and of 1) reach node 2 and no further, so
    the buffer is exactly [2, 1, 0].  The full graph has no edges, stage 3 adds
    nothing and returns the buffer's three nodes."""
    sub = csr([[1], [2], [3], [4], []])
    full = csr([[], [], [], [], []])
    x = points_on_axis([5.0, 4.0, 3.0, 2.0, 1.0])
    q = points_on_axis([0.0]).astype(np.float32)
    out_I, out_D = np.empty((1, 4), np.int64), np.empty((1, 4), np.float32)
    buf_I, buf_D = np.empty((1, 16), np.int64), np.empty((1, 16), np.float32)
    oracle.traverse_refine(out_I, out_D, buf_I, buf_D,
                           np.array([[0]], np.int64), np.array([[25.0]], np.float32),
                           list(sub), list(full), x, q, 16, D)
    assert buf_I[0].tolist() == [2, 1, 0] + [-1] * 13
    assert buf_D[0].tolist() == [9.0, 16.0, 25.0] + [INF] * 13
    assert out_I[0].tolist() == [2, 1, 0, -1]
    assert out_D[0].tolist() == [9.0, 16.0, 25.0, INF]


def test_stage_three_skips_what_stage_two_has_marked():
    """traverse_cpu.cpp:317-336, the case the buffer cannot hide: with a
    buffer of one slot stage 2 hands over node 2 only, but it has also
    evaluated (and marked) node 3.  Stage 3 expands 2, whose row is [3, 4]:
    3 carries the shared mark and is skipped although it is nearer than 4.
    With a mark of its own stage 3 would return [2, 3, 4]."""
    sub = csr([[2, 3], [], [], [], []])
    full = csr([[], [], [3, 4], [], []])
    x = points_on_axis([5.0, 9.0, 1.0, 2.0, 3.0])
    q = points_on_axis([0.0]).astype(np.float32)
    out_I, out_D = np.empty((1, 3), np.int64), np.empty((1, 3), np.float32)
    buf_I, buf_D = np.empty((1, 1), np.int64), np.empty((1, 1), np.float32)
    oracle.traverse_refine(out_I, out_D, buf_I, buf_D,
                           np.array([[0]], np.int64), np.array([[25.0]], np.float32),
                           list(sub), list(full), x, q, 16, D)
    assert buf_I[0].tolist() == [2] and buf_D[0].tolist() == [1.0]
    assert out_I[0].tolist() == [2, 4, -1]
    assert out_D[0].tolist() == [1.0, 9.0, INF]
