"""Operator API with the call signatures of ``pilot_ann/kernels/__init__.py``.

Every function validates its tensors the way the reference's ``CHECK_CPU`` /
``CHECK_CUDA`` macros do (``extension/inc/common.h:15-29``: device, rank,
dtype, contiguity; ``RuntimeError`` on violation) and then calls the C ABI of
``csrc/libpilotann.so``.  Device work is enqueued on torch's current stream
and not synchronised, like the reference (``traverse_cuda.cu:284``,
``routing_cuda.cu:103``).
"""
import ctypes
from collections import OrderedDict

import torch

from .. import _lib

BEAM_WIDTH = 4


# ---- argument checks --------------------------------------------------------

def _check(x, name, dim, dtype, cuda):
    if not isinstance(x, torch.Tensor):
        raise RuntimeError(f'{name} must be a tensor')
    if cuda and not x.is_cuda:
        raise RuntimeError(f'{name} must be a CUDA tensor')
    if not cuda and x.is_cuda:
        raise RuntimeError(f'{name} must be a CPU tensor')
    if x.dim() != dim:
        raise RuntimeError(f'{name} must be of dim {dim}')
    if x.dtype != dtype:
        raise RuntimeError(f'{name} must be type of {dtype}')
    if not x.is_contiguous():
        raise RuntimeError(f'{name} custom kernel requires contiguous tensor')


def _require(cond, text):
    if not cond:
        raise RuntimeError(f'Expected {text} to be true, but got false.')


def _ptr(x):
    return ctypes.c_void_p(x.data_ptr() if x is not None else None)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


# ---- device graph -----------------------------------------------------------

class PreparedGraph:
    """Device-resident search form of a subgraph (see ``pa_graph_prepare``):
    ``adj[n_storage, n_neighbors]`` int32 storage rows, ``gid[n_storage]``
    int32 global ids, plus the int64 ``mapping`` the caller supplied."""

    def __init__(self, indptr, indices, mapping, n_storage, n_neighbors):
        _check(indptr, 'indptr', 1, torch.int64, True)
        _check(indices, 'indices', 1, torch.int64, True)
        _check(mapping, 'mapping', 1, torch.int64, True)
        n_nodes = indptr.size(0) - 1
        _require(mapping.size(0) == n_nodes, 'mapping.size(0) == n_nodes')
        self.n_nodes = n_nodes
        self.n_storage = int(n_storage)
        self.n_neighbors = int(n_neighbors)
        self.mapping = mapping
        self._sources = (indptr, indices)
        dev = indptr.device
        self.adj = torch.empty(self.n_storage * self.n_neighbors,
                               dtype=torch.int32, device=dev)
        self.gid = torch.empty(self.n_storage, dtype=torch.int32, device=dev)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)
        with torch.cuda.device(dev):
            rc = _lib.lib().pa_graph_prepare(
                _ptr(indptr), _ptr(indices), _ptr(mapping), n_nodes,
                self.n_storage, indices.numel(), self.n_neighbors,
                _ptr(self.adj),
                _ptr(self.gid), _ptr(self.status), _stream())
        if rc == -7:
            raise RuntimeError(
                'pa_graph_prepare: malformed graph, status bits '
                f'{int(self.status.item())} (1 mapping not a bijection, '
                '2 row longer than n_neighbors, 4 id out of range, '
                '8 row outside indices)')
        _lib.check(rc, 'pa_graph_prepare')


_graph_cache = OrderedDict()
_GRAPH_CACHE_SIZE = 4


def prepare_graph(indptr, indices, mapping, n_storage, n_neighbors):
    """Cached :class:`PreparedGraph` for these three tensors.  The cache holds
    the tensors themselves, so an address cannot come back with other
    content; an in-place change bumps the tensor's version and misses."""
    key = (indptr.data_ptr(), indices.data_ptr(), mapping.data_ptr(),
           indptr._version, indices._version, mapping._version,
           indptr.numel(), indices.numel(), int(n_storage), int(n_neighbors),
           str(indptr.device))
    hit = _graph_cache.get(key)
    if hit is not None:
        _graph_cache.move_to_end(key)
        return hit
    graph = PreparedGraph(indptr, indices, mapping, n_storage, n_neighbors)
    _graph_cache[key] = graph
    while len(_graph_cache) > _GRAPH_CACHE_SIZE:
        _graph_cache.popitem(last=False)
    return graph


_workspaces = {}


def _workspace(device, nbytes):
    """Scratch memory for one traversal call, one buffer per (device,
    stream): calls on different streams may overlap and must not share it."""
    key = (str(device), torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8,
                          device=device)
        _workspaces[key] = buf
    return buf


# ---- traversal --------------------------------------------------------------

def traverse_cuda(output_I: torch.Tensor,
                  output_D: torch.Tensor,
                  indptr: torch.Tensor,
                  indices: torch.Tensor,
                  mapping: torch.Tensor,
                  storage: torch.Tensor,
                  query: torch.Tensor,
                  initial_I: torch.Tensor,
                  initial_D: torch.Tensor,
                  n_neighbors: int,
                  counters: torch.Tensor = None,
                  mode: str = 'exact', width: int = 4):
    """Same arguments as ``kernels.traverse_cuda``
    (``pilot_ann/kernels/__init__.py:62-75``; checks of
    ``traverse_cuda.cu:256-281``).  ``output_*`` are ``[B, 4, ef]``; row b,
    flattened, receives the ``4·ef`` best candidates of the host search
    (``traverse_cpu.cpp:12-163`` with ``ef_search = k = 4·ef``) best first,
    ``-1`` / ``+inf`` in unused slots.  ``n_neighbors`` may be any value up
    to 64.  ``counters`` (5 int64 on the device) is an optional work tally.
    ``mode='wide'`` runs the labelled throughput mode instead
    (:func:`traverse_wide_prepared`): not the host search step for step.
    """
    _check(indptr, 'indptr', 1, torch.int64, True)
    _check(indices, 'indices', 1, torch.int64, True)
    _check(mapping, 'mapping', 1, torch.int64, True)
    _check(storage, 'storage', 2, torch.float32, True)
    _check(query, 'query', 2, torch.float32, True)
    _check(initial_I, 'initial_I', 2, torch.int64, True)
    _check(initial_D, 'initial_D', 2, torch.float32, True)
    _check(output_I, 'output_I', 3, torch.int64, True)
    _check(output_D, 'output_D', 3, torch.float32, True)
    d_model = query.size(-1)
    batch_size = query.size(0)
    n_nodes = indptr.size(0) - 1
    n_storage = storage.size(0)
    ef_search = output_I.size(-1)
    _require(mapping.size(0) == n_nodes, 'mapping.size(0) == n_nodes')
    _require(storage.size(-1) == d_model, 'storage.size(-1) == d_model')
    _require(output_I.size(0) == batch_size, 'output_I.size(0) == batch_size')
    _require(output_I.size(1) == BEAM_WIDTH, 'output_I.size(1) == BEAM_WIDTH')
    _require(initial_I.size(0) == batch_size,
             'initial_I.size(0) == batch_size')
    _require(output_I.size() == output_D.size(),
             'output_I.sizes() == output_D.sizes()')
    _require(initial_I.size() == initial_D.size(),
             'initial_I.sizes() == initial_D.sizes()')
    _require(1 <= n_neighbors <= 64, '1 <= n_neighbors <= 64')
    _require(BEAM_WIDTH * ef_search <= 2048, 'heapq_size supported')
    _require(d_model % 8 == 0, 'd_model % 8 == 0')
    if counters is not None:
        _check(counters, 'counters', 1, torch.int64, True)
        _require(counters.numel() >= 5, 'counters.numel() >= 5')

    _require(mode in ('exact', 'wide'), "mode in ('exact', 'wide')")
    graph = prepare_graph(indptr, indices, mapping, n_storage, n_neighbors)
    if mode == 'wide':
        _require(1 <= width <= 4, '1 <= width <= 4')
        traverse_wide_prepared(output_I, output_D, graph, storage, query,
                               initial_I, initial_D, counters, width)
        return
    traverse_prepared(output_I, output_D, graph, storage, query, initial_I,
                      initial_D, counters)


def traverse_prepared(output_I, output_D, graph: PreparedGraph, storage,
                      query, initial_I, initial_D, counters=None):
    """:func:`traverse_cuda` on an already prepared graph (no checks beyond
    the C ABI's own).  ``storage``: plain rows (their device layout is made
    once and cached) or :class:`PreparedRows`."""
    lib = _lib.lib()
    storage = prepare_rows(storage).rows
    batch_size, d_model = query.shape
    ef_search = output_I.size(-1)
    beam = output_I.size(1)
    with torch.cuda.device(query.device):
        nbytes = ctypes.c_size_t()
        _lib.check(lib.pa_traverse_plan(
            graph.n_storage, batch_size, d_model, beam * ef_search, None,
            ctypes.byref(nbytes)), 'pa_traverse_plan')
        ws = _workspace(query.device, nbytes.value)
        _lib.check(lib.pa_traverse(
            _ptr(output_I), _ptr(output_D), _ptr(graph.adj), _ptr(graph.gid),
            _ptr(graph.mapping), _ptr(storage), _ptr(query), _ptr(initial_I),
            _ptr(initial_D), batch_size, graph.n_nodes, graph.n_storage,
            d_model, initial_I.size(-1), beam, ef_search, graph.n_neighbors,
            _ptr(ws), ws.numel(), _ptr(counters), _stream()), 'pa_traverse')


def traverse_wide_prepared(output_I, output_D, graph: PreparedGraph, storage,
                           query, initial_I, initial_D, counters=None,
                           width: int = 4):
    """The wide mode of the traversal (``pa_traverse_wide``), a labelled
    throughput mode beside :func:`traverse_prepared`, never the default: same
    arguments and output layout, the ``width`` (1..4) best open candidates
    expanded together per step, result list and open list one sorted pool.
    Distances of returned ids are the exact mode's, bit for bit; the ids are
    not promised to be the host search's (``traverse_cpu``)."""
    lib = _lib.lib()
    storage = prepare_rows(storage).rows
    batch_size, d_model = query.shape
    ef_search = output_I.size(-1)
    beam = output_I.size(1)
    with torch.cuda.device(query.device):
        nbytes = ctypes.c_size_t()
        _lib.check(lib.pa_traverse_wide_plan(
            graph.n_storage, batch_size, d_model, beam * ef_search, None,
            ctypes.byref(nbytes)), 'pa_traverse_wide_plan')
        ws = _workspace(query.device, nbytes.value)
        _lib.check(lib.pa_traverse_wide(
            _ptr(output_I), _ptr(output_D), _ptr(graph.adj), _ptr(graph.gid),
            _ptr(graph.mapping), _ptr(storage), _ptr(query), _ptr(initial_I),
            _ptr(initial_D), batch_size, graph.n_nodes, graph.n_storage,
            d_model, initial_I.size(-1), beam, ef_search, graph.n_neighbors,
            int(width), _ptr(ws), ws.numel(), _ptr(counters), _stream()),
            'pa_traverse_wide')


# ---- entry router -----------------------------------------------------------

def routing_cuda(query: torch.Tensor,
                 route_vectors: torch.Tensor,
                 entry_nodes: torch.Tensor,
                 entry_vectors: torch.Tensor,
                 return_entries: bool = False):
    """``kernels.routing_cuda`` (``pilot_ann/kernels/__init__.py:97-103``,
    checks of ``routing_cuda.cu:76-90``): returns ``(router[B] int64,
    distances[B, n_leaves] float32)``.  With ``return_entries`` the ids of the
    chosen route's leaves, ``entry_nodes[router]`` ``[B, n_leaves]``, are
    written by the same launch and returned as a third tensor (the
    ``index_select`` of ``layers/entry.py:86``)."""
    _check(query, 'query', 2, torch.float32, True)
    _check(route_vectors, 'route_vectors', 2, torch.float32, True)
    _check(entry_vectors, 'entry_vectors', 3, torch.float32, True)
    _check(entry_nodes, 'entry_nodes', 2, torch.int64, True)
    d_model = query.size(-1)
    batch_size = query.size(0)
    n_leaves = entry_nodes.size(-1)
    n_routers = route_vectors.size(0)
    _require(route_vectors.size(-1) == d_model,
             'route_vectors.size(-1) == d_model')
    _require(entry_vectors.size(-1) == d_model,
             'entry_vectors.size(-1) == d_model')
    _require(entry_vectors.size(0) == n_routers,
             'entry_vectors.size(0) == n_routers')
    _require(entry_vectors.size(1) == n_leaves,
             'entry_vectors.size(1) == n_leaves')
    _require(n_leaves % 32 == 0, 'n_leaves % BLOCK_SIZE == 0')
    _require(d_model % 8 == 0, 'd_model % 8 == 0')
    _require(entry_nodes.size(0) == n_routers,
             'entry_nodes.size(0) == n_routers')
    router = torch.empty(batch_size, dtype=torch.int64, device=query.device)
    distances = torch.empty(batch_size, n_leaves, dtype=torch.float32,
                            device=query.device)
    entries = None
    if return_entries:
        entries = torch.empty(batch_size, n_leaves, dtype=torch.int64,
                              device=query.device)
    with torch.cuda.device(query.device):
        _lib.check(_lib.lib().pa_route(
            _ptr(router), _ptr(distances), _ptr(query), _ptr(route_vectors),
            _ptr(entry_vectors), batch_size, n_routers, n_leaves, d_model,
            _ptr(entry_nodes) if return_entries else None, _ptr(entries),
            _stream()), 'pa_route')
    if return_entries:
        return router, distances, entries
    return router, distances


def rotate(query: torch.Tensor, VT: torch.Tensor, n_out: int = None):
    """``query @ VT.T`` restricted to its first ``n_out`` columns (all of them
    by default): the rotation of ``IndexStaged.search``
    (``pilot_ann/layers/staged.py:198-201``) on the device's matrix cores.
    ``query[B, d]`` and ``VT[d, d]`` are device tensors; returns ``[B, n_out]``
    on the current stream."""
    _check(query, 'query', 2, torch.float32, True)
    _check(VT, 'VT', 2, torch.float32, True)
    d_model = query.size(-1)
    _require(VT.size(0) == d_model and VT.size(1) == d_model,
             'VT.sizes() == {d_model, d_model}')
    _require(d_model % 8 == 0, 'd_model % 8 == 0')
    n_out = d_model if n_out is None else int(n_out)
    _require(1 <= n_out <= d_model, '1 <= n_out <= d_model')
    out = torch.empty(query.size(0), n_out, dtype=torch.float32,
                      device=query.device)
    with torch.cuda.device(query.device):
        _lib.check(_lib.lib().pa_rotate(
            _ptr(out), _ptr(query), _ptr(VT), query.size(0), d_model, n_out,
            _stream()), 'pa_rotate')
    return out


def entry_distances(query: torch.Tensor, entry_vectors: torch.Tensor):
    """Squared L2 from every query to a fixed list of entry vectors
    ``[n_entries, d]`` — what ``IndexEntry.search`` computes with
    ``cdist().square()`` in its random mode (``layers/entry.py:70-74``),
    here with the traversal's own distance kernel."""
    _check(query, 'query', 2, torch.float32, True)
    _check(entry_vectors, 'entry_vectors', 2, torch.float32, True)
    _require(entry_vectors.size(-1) == query.size(-1),
             'entry_vectors.size(-1) == d_model')
    _require(query.size(-1) % 8 == 0, 'd_model % 8 == 0')
    distances = torch.empty(query.size(0), entry_vectors.size(0),
                            dtype=torch.float32, device=query.device)
    with torch.cuda.device(query.device):
        _lib.check(_lib.lib().pa_route(
            None, _ptr(distances), _ptr(query), None, _ptr(entry_vectors),
            query.size(0), 0, entry_vectors.size(0), query.size(-1), None,
            None, _stream()), 'pa_route')
    return distances


# ---- nearest-neighbour candidates for the graph builder -----------------------

class HalfRows:
    """Rows prepared for :func:`knn_candidates`: a half-precision copy, scaled
    so that a row is about one unit long (root mean square over the set) and
    clamped to the half range, padded with zeros to whole tiles of the kernel
    (``pa_knn_tile_rows()`` rows, 64 columns: what it reads without bounds
    checks), and the squared lengths of the scaled rows.  (Scaling by the
    largest coordinate instead would push a set with a few large coordinates
    — outliers, unnormalised embeddings — into the half subnormals.)"""

    HALF_MAX = 60000.0

    def __init__(self, rows: torch.Tensor, scale: float = None):
        _check(rows, 'rows', 2, torch.float32, True)
        n, d = rows.shape
        if scale is None:
            rms = float(rows.square().sum(-1).mean().sqrt()) if n else 1.0
            scale = 1.0 / max(rms, 1e-30)
        self.n, self.d, self.scale = n, d, scale
        self.tile = int(_lib.lib().pa_knn_tile_rows())
        n_pad, d_pad = -(-max(n, 1) // self.tile) * self.tile, -(-d // 64) * 64
        self.half = torch.zeros(n_pad, d_pad, dtype=torch.float16, device=rows.device)
        self.norm = torch.zeros(n_pad, dtype=torch.float32, device=rows.device)
        for lo in range(0, n, 1 << 20):     # in pieces: no second copy of a large set
            piece = (rows[lo:lo + (1 << 20)] * scale).clamp_(-self.HALF_MAX, self.HALF_MAX)
            self.half[lo:lo + piece.size(0), :d] = piece
            self.norm[lo:lo + piece.size(0)] = piece.square().sum(-1)

    def low(self, rows: torch.Tensor) -> torch.Tensor:
        """The second half-precision part of ``rows`` (the tensor this set was
        made from): ``rows * scale - half``, same shape and padding as
        ``half``, so that ``half + low`` is the scaled row to about 22 bits."""
        low = torch.zeros_like(self.half)
        for lo in range(0, self.n, 1 << 20):
            hi = min(self.n, lo + (1 << 20))
            piece = (rows[lo:hi] * self.scale).clamp_(-self.HALF_MAX, self.HALF_MAX)
            low[lo:hi, :self.d] = piece - self.half[lo:hi, :self.d].float()
        return low

    def rows(self, lo: int, hi: int) -> 'HalfRows':
        """Rows ``lo .. hi`` as a set of their own (a view; ``lo`` a multiple
        of the tile, so that the padding still reaches a whole tile)."""
        _require(lo % self.tile == 0 and 0 <= lo < hi <= self.n,
                 'lo a multiple of the tile rows, lo < hi <= n')
        part = HalfRows.__new__(HalfRows)
        part.n, part.d, part.scale, part.tile = hi - lo, self.d, self.scale, self.tile
        part.half, part.norm = self.half[lo:], self.norm[lo:]
        return part


# workgroups the device runs at a time: one per compute unit
_KNN_RESIDENT = 256


def knn_candidates(query, base, keep: int, n_seg: int = None):
    """For every row of ``query`` the ``keep`` (64, 128, 256 or 512) rows of ``base``
    that are closest by half-precision products (``pa_knn``; the step the
    reference leaves to faiss, ``pilot_ann/utils/graphs.py:15-20``).
    ``query`` / ``base``: float32 device tensors or :class:`HalfRows` (pass the
    same object for both to rank a set against itself).  Returns ids
    ``[m, keep]`` (int64, ``-1`` where ``base`` has fewer rows) in no
    particular order; rank them with exact distances."""
    if not isinstance(base, HalfRows):
        base = HalfRows(base)
    if not isinstance(query, HalfRows):
        query = HalfRows(query, scale=base.scale)
    _require(query.d == base.d, 'query.size(-1) == base.size(-1)')
    _require(query.half.device == base.half.device, 'query.device == base.device')
    _require(base.n >= 1, 'base.size(0) >= 1')
    m, n, device = query.n, base.n, base.half.device
    if m == 0:
        return torch.empty(0, keep, dtype=torch.long, device=device)
    tile = query.tile
    blocks, tiles = -(-m // tile), -(-n // tile)
    if n_seg is None:
        # enough workgroups for one per compute unit
        n_seg = max(1, min(tiles, _KNN_RESIDENT // blocks))
    cap = int(_lib.lib().pa_knn_list_capacity(int(keep)))
    _require(cap > 0, 'keep is 64, 128, 256 or 512')
    score = torch.empty(n_seg, m, cap, dtype=torch.float32, device=device)
    ids = torch.empty(n_seg, m, cap, dtype=torch.int32, device=device)
    count = torch.empty(n_seg, m, dtype=torch.int32, device=device)
    with torch.cuda.device(device):
        _lib.check(_lib.lib().pa_knn(
            _ptr(score), _ptr(ids), _ptr(count), _ptr(query.half), _ptr(base.half),
            _ptr(base.norm), m, n, base.half.size(1), int(keep), n_seg, _stream()),
            'pa_knn')
    score, ids = score[:, :, :keep], ids[:, :, :keep]
    valid = torch.arange(keep, device=device).view(1, 1, keep) < count.unsqueeze(-1)
    ids = torch.where(valid, ids.long(), torch.full_like(ids, -1, dtype=torch.long))
    if n_seg == 1:
        return ids[0]
    score = torch.where(valid, score, torch.full_like(score, float('inf')))
    score = score.permute(1, 0, 2).reshape(m, n_seg * keep)
    ids = ids.permute(1, 0, 2).reshape(m, n_seg * keep)
    top = torch.topk(score, min(keep, score.size(1)), dim=-1, largest=False)
    return torch.gather(ids, 1, top.indices)


def knn_rerank(rows: torch.Tensor, cand: torch.Tensor, first: int = 0):
    """Exact squared float32 distances ``[m, k]`` from rows ``first ..
    first + m`` of ``rows`` to their candidates ``cand`` ``[m, k]`` (int64 row
    numbers; ``pa_knn_rerank``): infinity where a candidate is ``-1`` or the
    row itself.  The ranking step after :func:`knn_candidates`."""
    _check(rows, 'rows', 2, torch.float32, True)
    _check(cand, 'cand', 2, torch.int64, True)
    _require(cand.device == rows.device, 'cand.device == rows.device')
    m, k = cand.shape
    n, d = rows.shape
    _require(0 <= first and first + m <= n, 'first + cand.size(0) <= rows.size(0)')
    dist = torch.empty(m, k, dtype=torch.float32, device=rows.device)
    with torch.cuda.device(rows.device):
        _lib.check(_lib.lib().pa_knn_rerank(
            _ptr(dist), _ptr(rows), _ptr(cand), m, int(first), n, d, k, _stream()),
            'pa_knn_rerank')
    return dist


def graph_prune(pair: torch.Tensor, cand_dist: torch.Tensor, m_keep: int, fill: bool):
    """Occlusion pruning of candidate lists (``pa_graph_prune``): ``pair``
    ``[n, k, k]`` distances between a node's candidates, ``cand_dist``
    ``[n, k]`` their distances to the node, closest first.  Returns the
    positions ``[n, m_keep]`` (int64, ``-1`` padded) of the candidates kept, in
    order, topped up with the closest rejected ones when ``fill``."""
    _check(pair, 'pair', 3, torch.float32, True)
    _check(cand_dist, 'cand_dist', 2, torch.float32, True)
    n, k = cand_dist.shape
    _require(pair.shape == (n, k, k), 'pair.shape == (n, k, k)')
    selected = torch.empty(n, int(m_keep), dtype=torch.int32, device=pair.device)
    with torch.cuda.device(pair.device):
        _lib.check(_lib.lib().pa_graph_prune(
            _ptr(selected), _ptr(pair), _ptr(cand_dist), n, k, int(m_keep),
            int(bool(fill)), _stream()), 'pa_graph_prune')
    return selected.long()


def graph_prune_rows(rows: torch.Tensor, cand: torch.Tensor, cand_dist: torch.Tensor,
                     m_keep: int, fill: bool):
    """:func:`graph_prune` without the table of pairwise distances
    (``pa_graph_prune_rows``): ``rows`` ``[N, d]`` float32, ``cand`` ``[n, k]``
    int64 row numbers (closest first, ``-1`` after the last, ``k <= 256``; a
    number beyond the rows counts as ``-1``),
    ``cand_dist`` ``[n, k]`` their squared distances to the node.  Returns the
    positions ``[n, m_keep]`` as :func:`graph_prune` does."""
    _check(rows, 'rows', 2, torch.float32, True)
    _check(cand, 'cand', 2, torch.int64, True)
    _check(cand_dist, 'cand_dist', 2, torch.float32, True)
    _require(cand.shape == cand_dist.shape, 'cand.shape == cand_dist.shape')
    _require(cand.device == rows.device == cand_dist.device, 'one device')
    n, k = cand.shape
    _require(1 <= k <= 256, '1 <= k <= 256')
    if n == 0:
        return torch.empty(0, int(m_keep), dtype=torch.long, device=rows.device)
    parts = HalfRows(rows)
    low = parts.low(rows)
    selected = torch.empty(n, int(m_keep), dtype=torch.int32, device=rows.device)
    with torch.cuda.device(rows.device):
        _lib.check(_lib.lib().pa_graph_prune_rows(
            _ptr(selected), _ptr(parts.half), _ptr(low), _ptr(parts.norm), _ptr(cand),
            _ptr(cand_dist), n, rows.size(0), parts.half.size(1), k, int(m_keep),
            int(bool(fill)),
            float(parts.scale) ** 2, _stream()), 'pa_graph_prune_rows')
    return selected.long()


# ---- the reference's operator hooks ------------------------------------------

def _heap(keys, values):
    _check(keys, 'keys', 1, torch.float32, False)
    _check(values, 'values', 1, torch.int64, False)
    _require(keys.numel() == values.numel(), 'keys.numel() == values.numel()')


def heapq_pop(keys: torch.Tensor, values: torch.Tensor):
    """``kernels.heapq_pop`` (``pilot_ann/kernels/__init__.py:5-7``,
    ``ops_cpu.cpp:8-13``): drops the root of the array heap in place."""
    _heap(keys, values)
    _lib.check(_lib.lib().pa_heapq_pop(_ptr(keys), _ptr(values), keys.numel()),
               'pa_heapq_pop')


def heapq_pushpop(keys: torch.Tensor, values: torch.Tensor, key: float, value: int):
    """``kernels.heapq_pushpop`` (``pilot_ann/kernels/__init__.py:10-15``,
    ``ops_cpu.cpp:15-24``), in place."""
    _heap(keys, values)
    _lib.check(_lib.lib().pa_heapq_pushpop(
        _ptr(keys), _ptr(values), keys.numel(), float(key), int(value)),
        'pa_heapq_pushpop')


def heapq_replace(keys: torch.Tensor, values: torch.Tensor, key: float, value: int):
    """``kernels.heapq_replace`` (``pilot_ann/kernels/__init__.py:18-23``,
    ``ops_cpu.cpp:26-35``), in place."""
    _heap(keys, values)
    _lib.check(_lib.lib().pa_heapq_replace(
        _ptr(keys), _ptr(values), keys.numel(), float(key), int(value)),
        'pa_heapq_replace')


def bitmask_put(keys: torch.Tensor, n: int):
    """``kernels.bitmask_put`` (``pilot_ann/kernels/__init__.py:26-27``,
    ``ops_cpu.cpp:37-51``): int32 marks of ``n`` nodes, non-zero at ``keys``."""
    _check(keys, 'keys', 1, torch.int64, False)
    marks = torch.empty(int(n), dtype=torch.int32)
    _lib.check(_lib.lib().pa_bitmask_put(_ptr(marks), int(n), _ptr(keys),
                                         keys.numel()), 'pa_bitmask_put')
    return marks


def square_dist(query: torch.Tensor, storage: torch.Tensor, nodelist: torch.Tensor):
    """``kernels.square_dist`` (``pilot_ann/kernels/__init__.py:30-35``,
    ``ops_cpu.cpp:53-85``): squared L2 distances between ``query`` and the
    rows ``nodelist`` of ``storage``, host tensors."""
    _check(query, 'query', 1, torch.float32, False)
    _check(storage, 'storage', 2, torch.float32, False)
    _check(nodelist, 'nodelist', 1, torch.int64, False)
    _require(storage.size(-1) == query.size(0), 'storage.size(-1) == d_model')
    output = torch.zeros(nodelist.size(0), dtype=torch.float32)
    _lib.check(_lib.lib().pa_square_dist(
        _ptr(output), _ptr(query), _ptr(storage), _ptr(nodelist),
        nodelist.size(0), storage.size(0), query.size(0)), 'pa_square_dist')
    return output


def graph_sampling(indptr: torch.Tensor, indices: torch.Tensor, n_samples: int,
                   n_hops: int, seed: int = None):
    """``kernels.graph_sampling`` (``pilot_ann/kernels/__init__.py:38-44``,
    ``extension/sampling_cpu.cpp:5-65``): seed nodes and everything within
    ``n_hops`` edges of them until ``n_samples`` nodes are in; returns
    ``[nodelist, mapping]`` as lists.  The reference seeds its draws with the
    time; ``seed=None`` does the same, a number makes the sample repeatable."""
    import time
    from ..utils.graphs import graph_sampling as sample
    nodelist, mapping = sample(indptr, indices, n_samples=n_samples, n_hops=n_hops,
                               seed=int(time.time()) if seed is None else seed)
    return [nodelist.tolist(), mapping.tolist()]


# ---- host stages ------------------------------------------------------------

def traverse_cpu(output_I: torch.Tensor,
                 output_D: torch.Tensor,
                 initial_I: torch.Tensor,
                 initial_D: torch.Tensor,
                 indptr: torch.Tensor,
                 indices: torch.Tensor,
                 storage: torch.Tensor,
                 query: torch.Tensor,
                 ef_search: int):
    """``kernels.traverse_cpu`` (``pilot_ann/kernels/__init__.py:47-59``,
    checks of ``traverse_cpu.cpp:174-193``)."""
    _check(query, 'query', 2, torch.float32, False)
    _check(indptr, 'indptr', 1, torch.int64, False)
    _check(indices, 'indices', 1, torch.int64, False)
    _check(storage, 'storage', 2, torch.float32, False)
    _check(initial_I, 'initial_I', 2, torch.int64, False)
    _check(initial_D, 'initial_D', 2, torch.float32, False)
    _check(output_I, 'output_I', 2, torch.int64, False)
    _check(output_D, 'output_D', 2, torch.float32, False)
    batch_size, d_model = query.shape
    _require(storage.size(-1) == d_model, 'storage.size(-1) == d_model')
    _require(output_I.size(0) == batch_size, 'output_I.size(0) == batch_size')
    _require(initial_I.size(0) == batch_size,
             'initial_I.size(0) == batch_size')
    _require(output_I.size() == output_D.size(),
             'output_I.sizes() == output_D.sizes()')
    _require(initial_I.size() == initial_D.size(),
             'initial_I.sizes() == initial_D.sizes()')
    _require(ef_search <= 2048, 'ef_search supported')
    _lib.check(_lib.lib().pa_traverse_cpu(
        _ptr(output_I), _ptr(output_D), _ptr(initial_I), _ptr(initial_D),
        _ptr(indptr), _ptr(indices), _ptr(storage), _ptr(query), batch_size,
        storage.size(0), d_model, initial_I.size(-1), output_I.size(-1),
        int(ef_search)), 'pa_traverse_cpu')


def traverse_refine(output_I: torch.Tensor,
                    output_D: torch.Tensor,
                    buffer_I: torch.Tensor,
                    buffer_D: torch.Tensor,
                    initial_I: torch.Tensor,
                    initial_D: torch.Tensor,
                    subgraph: list,
                    fullgraph: list,
                    storage: torch.Tensor,
                    query: torch.Tensor,
                    ef_search: int,
                    d_principle: int):
    """``kernels.traverse_refine`` (``pilot_ann/kernels/__init__.py:78-94``,
    checks of ``traverse_cpu.cpp:270-294``).  ``initial_D`` is updated in
    place with the residual distance."""
    _require(len(subgraph) == 2, 'subgraph.size() == 2')
    _require(len(fullgraph) == 2, 'fullgraph.size() == 2')
    _check(query, 'query', 2, torch.float32, False)
    _check(storage, 'storage', 2, torch.float32, False)
    _check(initial_I, 'initial_I', 2, torch.int64, False)
    _check(initial_D, 'initial_D', 2, torch.float32, False)
    _check(buffer_I, 'buffer_I', 2, torch.int64, False)
    _check(buffer_D, 'buffer_D', 2, torch.float32, False)
    _check(output_I, 'output_I', 2, torch.int64, False)
    _check(output_D, 'output_D', 2, torch.float32, False)
    for g in (*subgraph, *fullgraph):
        _check(g, 'graph', 1, torch.int64, False)
    batch_size, d_model = query.shape
    _require(storage.size(-1) == d_model, 'storage.size(-1) == d_model')
    _require(output_I.size(0) == batch_size, 'output_I.size(0) == batch_size')
    _require(buffer_I.size(0) == batch_size, 'buffer_I.size(0) == batch_size')
    _require(initial_I.size(0) == batch_size,
             'initial_I.size(0) == batch_size')
    _require(output_I.size() == output_D.size(),
             'output_I.sizes() == output_D.sizes()')
    _require(buffer_I.size() == buffer_D.size(),
             'buffer_I.sizes() == buffer_D.sizes()')
    _require(initial_I.size() == initial_D.size(),
             'initial_I.sizes() == initial_D.sizes()')
    _require(ef_search <= 2048, 'ef_search supported')
    _lib.check(_lib.lib().pa_traverse_refine(
        _ptr(output_I), _ptr(output_D), _ptr(buffer_I), _ptr(buffer_D),
        _ptr(initial_I), _ptr(initial_D), _ptr(subgraph[0]),
        _ptr(subgraph[1]), _ptr(fullgraph[0]), _ptr(fullgraph[1]),
        _ptr(storage), _ptr(query), batch_size, storage.size(0), d_model,
        int(d_principle), initial_I.size(-1), buffer_I.size(-1),
        output_I.size(-1), int(ef_search)), 'pa_traverse_refine')


def prepare_full_graph(indptr, indices, n_neighbors=None):
    """:class:`PreparedGraph` of a graph in which every node has a row (the
    full graph of the refine): identity mapping.  ``n_neighbors`` defaults to
    the longest row."""
    _check(indptr, 'indptr', 1, torch.int64, True)
    n_nodes = indptr.size(0) - 1
    if n_neighbors is None:
        n_neighbors = int((indptr[1:] - indptr[:-1]).max().item())
    key = ('identity', str(indptr.device), n_nodes)
    mapping = _identity_maps.get(key)
    if mapping is None:
        mapping = torch.arange(n_nodes, dtype=torch.int64,
                               device=indptr.device)
        _identity_maps[key] = mapping
    return prepare_graph(indptr, indices, mapping, n_nodes, n_neighbors)


_identity_maps = {}


class PreparedRows:
    """Full-dimension rows in the layout the device refine streams (see
    ``pa_rows_prepare``): ``rows[n, d]`` float32 on the device, the pairs of
    every two groups of eight interleaved by lane."""

    def __init__(self, storage: torch.Tensor):
        _check(storage, 'storage', 2, torch.float32, True)
        _require(storage.size(-1) % 8 == 0, 'd_model % 8 == 0')
        self.n_rows, self.d_model = storage.shape
        self.rows = torch.empty_like(storage)
        with torch.cuda.device(storage.device):
            _lib.check(_lib.lib().pa_rows_prepare(
                _ptr(self.rows), _ptr(storage), self.n_rows, self.d_model,
                _stream()), 'pa_rows_prepare')


def prepare_rows(storage) -> PreparedRows:
    """Cached :class:`PreparedRows` of a plain ``[n, d]`` device tensor (the
    cache holds the tensor, an in-place change of it misses); a
    :class:`PreparedRows` is returned as it is."""
    if isinstance(storage, PreparedRows):
        return storage
    _check(storage, 'storage', 2, torch.float32, True)
    key = (storage.data_ptr(), storage._version, tuple(storage.shape),
           str(storage.device))
    hit = _rows_cache.get(key)
    if hit is not None:
        _rows_cache.move_to_end(key)
        return hit[0]
    rows = PreparedRows(storage)
    _rows_cache[key] = (rows, storage)
    while len(_rows_cache) > _ROWS_CACHE_SIZE:
        _rows_cache.popitem(last=False)
    return rows


_rows_cache = OrderedDict()
_ROWS_CACHE_SIZE = 4


def traverse_refine_cuda(output_I: torch.Tensor,
                         output_D: torch.Tensor,
                         buffer_I: torch.Tensor,
                         buffer_D: torch.Tensor,
                         initial_I: torch.Tensor,
                         initial_D: torch.Tensor,
                         subgraph: PreparedGraph,
                         fullgraph: PreparedGraph,
                         storage: PreparedRows,
                         query: torch.Tensor,
                         ef_search: int,
                         d_principle: int,
                         counters: torch.Tensor = None):
    """:func:`traverse_refine` on the device: the arguments of
    ``kernels.traverse_refine`` (``pilot_ann/kernels/__init__.py:78-94``) as
    device tensors, the two graphs in their prepared form (``subgraph`` from
    :func:`prepare_graph` as the traversal uses it, ``fullgraph`` from
    :func:`prepare_full_graph`), the rows from :func:`prepare_rows`.  Same
    results as the host function;
    ``initial_D`` is completed in place, ``buffer_*`` may be ``initial_*``.
    Enqueued on the current stream.  ``counters``: optional 6 int64."""
    _check(query, 'query', 2, torch.float32, True)
    if not isinstance(storage, PreparedRows):
        raise RuntimeError('storage must come from prepare_rows')
    _check(initial_I, 'initial_I', 2, torch.int64, True)
    _check(initial_D, 'initial_D', 2, torch.float32, True)
    _check(buffer_I, 'buffer_I', 2, torch.int64, True)
    _check(buffer_D, 'buffer_D', 2, torch.float32, True)
    _check(output_I, 'output_I', 2, torch.int64, True)
    _check(output_D, 'output_D', 2, torch.float32, True)
    batch_size, d_model = query.shape
    n_nodes = storage.n_rows
    _require(storage.d_model == d_model, 'storage.size(-1) == d_model')
    _require(output_I.size(0) == batch_size, 'output_I.size(0) == batch_size')
    _require(buffer_I.size(0) == batch_size, 'buffer_I.size(0) == batch_size')
    _require(initial_I.size(0) == batch_size,
             'initial_I.size(0) == batch_size')
    _require(output_I.size() == output_D.size(),
             'output_I.sizes() == output_D.sizes()')
    _require(buffer_I.size() == buffer_D.size(),
             'buffer_I.sizes() == buffer_D.sizes()')
    _require(initial_I.size() == initial_D.size(),
             'initial_I.sizes() == initial_D.sizes()')
    _require(ef_search <= 2048, 'ef_search supported')
    _require(d_model % 8 == 0 and d_principle % 8 == 0,
             'd_model % 8 == 0 and d_principle % 8 == 0')
    _require(subgraph.n_nodes == n_nodes, 'subgraph.n_nodes == n_storage')
    _require(fullgraph.n_nodes == n_nodes == fullgraph.n_storage,
             'fullgraph.n_nodes == n_storage')
    if counters is not None:
        _check(counters, 'counters', 1, torch.int64, True)
        _require(counters.numel() >= 6, 'counters.numel() >= 6')
    lib = _lib.lib()
    with torch.cuda.device(query.device):
        nbytes = ctypes.c_size_t()
        _lib.check(lib.pa_refine_plan(
            n_nodes, batch_size, d_model, int(ef_search), None,
            ctypes.byref(nbytes)), 'pa_refine_plan')
        ws = _workspace(query.device, nbytes.value)
        _lib.check(lib.pa_refine(
            _ptr(output_I), _ptr(output_D), _ptr(buffer_I), _ptr(buffer_D),
            _ptr(initial_I), _ptr(initial_D), _ptr(subgraph.adj),
            _ptr(subgraph.gid), _ptr(subgraph.mapping), _ptr(fullgraph.adj),
            _ptr(storage.rows), _ptr(query), batch_size, n_nodes, d_model,
            int(d_principle), initial_I.size(-1), buffer_I.size(-1),
            output_I.size(-1), int(ef_search), subgraph.n_neighbors,
            fullgraph.n_neighbors, _ptr(ws), ws.numel(), _ptr(counters),
            _stream()), 'pa_refine')


def pipeline(graph: list,
             subgraph: list,
             subgraph_cuda: list,
             storage: torch.Tensor,
             storage_cuda: torch.Tensor,
             query: torch.Tensor,
             query_cuda: torch.Tensor,
             initial_I: torch.Tensor,
             initial_D: torch.Tensor,
             n_neighbors: int,
             k: int,
             ef_search: int,
             d_principle: int,
             chunk_size: int):
    """``kernels.pipeline`` (``pilot_ann/kernels/__init__.py:106-124``, checks
    of ``pipeline_cpu.cpp:41-58``): device traversal in chunks overlapped
    with the host refine; returns ``(topk_I[B, k] int64, topk_D[B, k]
    float32)`` on the CPU."""
    _require(len(graph) == 2, 'graph.size() == 2')
    _require(len(subgraph) == 2, 'subgraph.size() == 2')
    _require(len(subgraph_cuda) == 3, 'subgraph_cuda.size() == 3')
    _check(query, 'query', 2, torch.float32, False)
    _check(storage, 'storage', 2, torch.float32, False)
    _check(graph[0], 'graph[0]', 1, torch.int64, False)
    _check(graph[1], 'graph[1]', 1, torch.int64, False)
    _check(subgraph[0], 'subgraph[0]', 1, torch.int64, False)
    _check(subgraph[1], 'subgraph[1]', 1, torch.int64, False)
    _check(query_cuda, 'query_cuda', 2, torch.float32, True)
    _check(storage_cuda, 'storage_cuda', 2, torch.float32, True)
    _check(subgraph_cuda[0], 'subgraph_cuda[0]', 1, torch.int64, True)
    _check(subgraph_cuda[1], 'subgraph_cuda[1]', 1, torch.int64, True)
    _check(subgraph_cuda[2], 'subgraph_cuda[2]', 1, torch.int64, True)
    _check(initial_I, 'initial_I', 2, torch.int64, True)
    _check(initial_D, 'initial_D', 2, torch.float32, True)
    batch_size, d_model = query.shape
    _require(batch_size % chunk_size == 0, 'batch_size % chunk_size == 0')
    _require(storage.size(-1) == d_model, 'storage.size(-1) == d_model')
    _require(query_cuda.size(0) == batch_size,
             'query_cuda.size(0) == batch_size')
    _require(query_cuda.size(-1) == d_principle == storage_cuda.size(-1),
             'query_cuda.size(-1) == d_principle')
    _require(initial_I.size(0) == batch_size,
             'initial_I.size(0) == batch_size')
    _require(initial_I.size() == initial_D.size(),
             'initial_I.sizes() == initial_D.sizes()')
    _require(1 <= n_neighbors <= 64, '1 <= n_neighbors <= 64')
    _require(BEAM_WIDTH * ef_search <= 2048, 'heapq_size supported')
    prepared = prepare_graph(subgraph_cuda[0], subgraph_cuda[1],
                             subgraph_cuda[2], storage_cuda.size(0),
                             n_neighbors)
    storage_cuda = prepare_rows(storage_cuda).rows
    topk_I = torch.empty(batch_size, k, dtype=torch.int64)
    topk_D = torch.empty(batch_size, k, dtype=torch.float32)
    with torch.cuda.device(query_cuda.device):
        _lib.check(_lib.lib().pa_pipeline(
            _ptr(topk_I), _ptr(topk_D), _ptr(graph[0]), _ptr(graph[1]),
            _ptr(subgraph[0]), _ptr(subgraph[1]), _ptr(storage), _ptr(query),
            _ptr(prepared.adj), _ptr(prepared.gid), _ptr(prepared.mapping),
            _ptr(storage_cuda), _ptr(query_cuda), _ptr(initial_I),
            _ptr(initial_D), batch_size, prepared.n_nodes,
            prepared.n_storage, d_model, int(d_principle),
            initial_I.size(-1), int(n_neighbors), int(ef_search), int(k),
            int(chunk_size), _stream()), 'pa_pipeline')
    return topk_I, topk_D
