"""Proximity graphs in the reference's layout.

Layout (``pilot_ann/utils/graphs.py:22-40``): ``indptr[i] = i * n_neighbors``,
``indices`` padded with ``-1`` after a row's last neighbour.  A subgraph keeps
global ids and one (possibly empty) row per global node
(``graphs.py:118-129``).  Construction differs from the reference, which
delegates to faiss: here an exact k-nearest-neighbour table (on a GPU: the
fused half-precision kernel ``pa_knn`` plus an exact float32 ranking of its
candidates) is pruned with the usual occlusion rule and completed with
reverse edges; the candidates of a node are its nearest among the nodes that
come before it in a seeded random order (:func:`insertion_order_candidates`),
which is what gives an incrementally built graph its long edges.  Everything runs on the device ``x`` lives on: a million
768-dimensional nodes take ten seconds on an MI355X, ten million five and a
half minutes.
"""
import torch


# Called with a short text when a long step of a build has finished a part
# (a pass of the neighbour kernel over two million rows, say): a caller that
# must show signs of life sets it (``graphs.progress = print``).
progress = None
# the pruning of the builder in one kernel (``kernels.graph_prune_rows``); off:
# gathered rows, a batched product of torch and ``kernels.graph_prune``
fused_prune = True


def knn_graph(x: torch.Tensor, k: int, chunk: int = None,
              compute_dtype: torch.dtype = None):
    """Exact ``k`` nearest other rows of every row: ``(ids[N, k], d2[N, k])``
    sorted by squared L2, self excluded.  ``compute_dtype`` (e.g. float16 on
    a GPU) is used for the N×N products only."""
    n = x.size(0)
    k = min(k, n - 1)
    # the kernel's candidates are ranked in half precision: 16 more than
    # asked for are taken, so that float32 can settle the last places
    if x.is_cuda and x.dtype == torch.float32 and 1 <= k <= 496 and n > 128:
        return _knn_graph_device(x, k)
    if chunk is None:
        chunk = max(64, min(4096, (1 << 29) // max(n, 1)))
    norms = x.float().square().sum(-1)
    xt = x.T.contiguous()
    if compute_dtype is not None:
        xt = xt.to(compute_dtype)
    ids, dists = [], []
    for lo in range(0, n, chunk):
        rows = x[lo:lo + chunk]
        if compute_dtype is not None:
            dots = (rows.to(compute_dtype) @ xt).float()
        else:
            dots = rows @ xt
        d = norms.unsqueeze(0) - 2.0 * dots
        ar = torch.arange(rows.size(0), device=x.device)
        d[ar, ar + lo] = float('inf')
        top = torch.topk(d, k=k, dim=-1, largest=False)
        ids.append(top.indices)
        dists.append(top.values + norms[lo:lo + chunk].unsqueeze(-1))
        del d, dots
    return torch.cat(ids), torch.cat(dists).clamp_(min=0.0)


def _knn_graph_device(x: torch.Tensor, k: int, rows_per_pass: int = None):
    """:func:`knn_graph` on the device: candidates from the fused
    half-precision kernel (``kernels.knn_candidates``, more of them than
    asked for), then exact float32 distances to those candidates decide."""
    from .. import kernels
    n, d = x.shape
    keep = next(size for size in (64, 128, 256, 512) if k + 16 <= size)
    rows = kernels.HalfRows(x)
    out_i = torch.empty(n, k, dtype=torch.long, device=x.device)
    out_d = torch.empty(n, k, dtype=torch.float32, device=x.device)
    # candidate lists of a pass: 2 * (keep + 384) * 4 bytes a row
    pass_rows = 1 << 21
    fused = d % 4 == 0 and d <= 4096 and rows_per_pass is None
    if rows_per_pass is None:
        rows_per_pass = max(256, min(8192, (1 << 29) // (keep * d)))
    for lo in range(0, n, pass_rows):
        hi = min(n, lo + pass_rows)
        cand = kernels.knn_candidates(rows.rows(lo, hi), rows, keep)
        if fused:
            # exact distances to the candidates by one kernel
            d2 = kernels.knn_rerank(x, cand, lo)
            top = torch.topk(d2, k, dim=-1, largest=False)
            out_i[lo:hi] = torch.gather(cand, 1, top.indices)
            out_d[lo:hi] = top.values
            if __debug__:
                # a kernel that left a place unwritten must raise here, not
                # fault in a later gather
                assert int(out_i[lo:hi].max()) < n and int(out_i[lo:hi].min()) >= -1
            del d2
            if progress is not None:
                torch.cuda.synchronize(x.device)   # report what is done, not what is queued
                progress(f'neighbour table: {hi} of {n} rows')
            continue
        own = torch.arange(lo, hi, device=x.device).unsqueeze(-1)
        for a in range(0, hi - lo, rows_per_pass):
            b = min(hi - lo, a + rows_per_pass)
            c = cand[a:b]
            diff = x[c.clamp(min=0)] - x[lo + a:lo + b].unsqueeze(1)
            d2 = diff.square_().sum(-1)
            d2[(c < 0) | (c == own[a:b])] = float('inf')
            top = torch.topk(d2, k, dim=-1, largest=False)
            out_i[lo + a:lo + b] = torch.gather(c, 1, top.indices)
            out_d[lo + a:lo + b] = top.values
            del diff, d2
        if progress is not None:
            progress(f'neighbour table: {hi} of {n} rows')
    return out_i, out_d


def _knn_rows_device(x, rows, lo: int, hi: int, n_base: int, k: int):
    """The ``k`` nearest of rows ``0 .. n_base`` of ``x`` for rows ``lo .. hi``
    (the row itself excluded), as :func:`_knn_graph_device` ranks them:
    candidates from ``pa_knn`` on the half-precision copy ``rows``
    (``kernels.HalfRows(x)``), exact float32 distances decide.  ``lo`` and
    ``n_base`` are multiples of the kernel's tile (or ``n_base`` is all of
    ``x``).  Places without a candidate hold ``-1`` / infinity."""
    from .. import kernels
    keep = next(size for size in (64, 128, 256, 512) if k + 16 <= size)
    base = rows if n_base == rows.n else rows.rows(0, n_base)
    cand = kernels.knn_candidates(rows.rows(lo, hi), base, keep)
    d2 = kernels.knn_rerank(x, cand, lo)
    top = torch.topk(d2, min(k, d2.size(1)), dim=-1, largest=False)
    ids = torch.gather(cand, 1, top.indices)
    if __debug__:
        # a kernel that left a place unwritten must raise here, not fault in
        # a later gather
        assert int(ids.max()) < n_base and int(ids.min()) >= -1
    ids = torch.where(torch.isinf(top.values), torch.full_like(ids, -1), ids)
    if ids.size(1) < k:
        pad = k - ids.size(1)
        ids = torch.cat([ids, ids.new_full((hi - lo, pad), -1)], 1)
        dist = torch.cat([top.values, top.values.new_full((hi - lo, pad), float('inf'))], 1)
        return ids, dist
    return ids, top.values


def _knn_rows_host(x, lo: int, hi: int, n_base: int, k: int, chunk: int = 2048):
    """:func:`_knn_rows_device` with torch alone (any device)."""
    base = x[:n_base].float()
    norms = base.square().sum(-1)
    kk = min(k, n_base - 1)
    ids, dist = [], []
    for a in range(lo, hi, chunk):
        b = min(hi, a + chunk)
        q = x[a:b].float()
        d = norms.unsqueeze(0) - 2.0 * (q @ base.T) + q.square().sum(-1, keepdim=True)
        own = torch.arange(a, b, device=x.device)
        inside = own < n_base
        d[torch.nonzero(inside).flatten(), own[inside]] = float('inf')
        top = torch.topk(d, kk, dim=-1, largest=False)
        i, v = top.indices, top.values.clamp_(min=0.0)
        if kk < k:
            i = torch.cat([i, i.new_full((b - a, k - kk), -1)], 1)
            v = torch.cat([v, v.new_full((b - a, k - kk), float('inf'))], 1)
        ids.append(i)
        dist.append(v)
    return torch.cat(ids), torch.cat(dist)


def insertion_order_candidates(x: torch.Tensor, pool: int, first: int = 1024):
    """Candidate lists in the way an incrementally built graph finds them
    (faiss' HNSW, which the reference takes its base layer from,
    ``pilot_ann/utils/graphs.py:43-77``, inserts the nodes one after the
    other, and a node's candidates are its nearest among those inserted
    before it): with the rows of ``x`` taken as already in insertion order,
    the first ``first`` rows rank each other, and each following batch — rows
    ``b .. 2b`` — ranks rows ``0 .. 2b``.  Half of the nodes so see the whole
    set; an early node sees a thin sample of it, so its candidates lie far
    apart, across clusters, and those long edges are what lets a search that
    starts anywhere get everywhere.  The later, nearer nodes reach an early
    node through their own lists (reverse edges).  Returns ``(ids, d2)``
    ``[N, pool]``, closest first, ``-1`` / infinity where a batch had fewer
    rows than ``pool``.  Exact nearest neighbours throughout (two thirds of
    the products of one table over all rows)."""
    n = x.size(0)
    device_path = x.is_cuda and x.dtype == torch.float32 and pool <= 496
    rows = None
    if device_path:
        from .. import kernels
        rows = kernels.HalfRows(x)
        first = max(first, rows.tile) // rows.tile * rows.tile
    ids = torch.empty(n, pool, dtype=torch.long, device=x.device)
    dist = torch.empty(n, pool, dtype=torch.float32, device=x.device)
    lo, hi = 0, min(n, first)
    while lo < n:
        # at most 2^21 rows a pass: the candidate lists of a pass are
        # 2 * (keep + 384) * 4 bytes a row
        for a in range(lo, hi, 1 << 21):
            b = min(hi, a + (1 << 21))
            if device_path and hi > 128:
                ids[a:b], dist[a:b] = _knn_rows_device(x, rows, a, b, hi, pool)
            else:
                ids[a:b], dist[a:b] = _knn_rows_host(x, a, b, hi, pool)
            if progress is not None:
                if x.is_cuda:
                    torch.cuda.synchronize(x.device)
                progress(f'neighbour table: {b} of {n} rows')
        lo, hi = hi, min(n, 2 * hi)
    return ids, dist


def _occlusion_prune(x, cand, cand_d, m_keep: int, fill: bool, chunk: int):
    """Keep candidate e (closest first) unless an already kept r is closer to
    e than the node itself is; with ``fill`` the nearest rejected candidates
    top the row up to ``m_keep``.  Returns ids[N, m_keep], ``-1`` padded."""
    n, K = cand.shape
    out = torch.full((n, m_keep), -1, dtype=torch.long, device=x.device)
    col = torch.arange(K, device=x.device)
    on_device = x.is_cuda and K <= 512
    if on_device:
        from .. import kernels
    if on_device and K <= 256 and x.dtype == torch.float32 and fused_prune:
        # gather, pairwise distances and the greedy pass in one kernel
        sel = kernels.graph_prune_rows(x.contiguous(), cand.contiguous(),
                                       cand_d.float().contiguous(), min(m_keep, K), fill)
        if __debug__:
            # selections a kernel left unwritten must raise, not fault the gather
            assert int(sel.max()) < K and int(sel.min()) >= -1
        ids = torch.gather(cand, 1, sel.clamp(min=0))
        out[:, :ids.size(1)] = torch.where(sel >= 0, ids, torch.full_like(ids, -1))
        return out
    norms = x.float().square().sum(-1)
    for lo in range(0, n, chunk):
        if progress is not None and (lo // chunk) % 512 == 511:
            progress(f'pruning: {lo} of {n} rows')
        c = cand[lo:lo + chunk]
        cd = cand_d[lo:lo + chunk]
        present = c >= 0               # lists end in -1 where a set was small
        v = x[c.clamp(min=0)].float()
        sq = norms[c.clamp(min=0)]
        # |a|^2 + |b|^2 - 2 a.b in one pass over the products
        pair = torch.baddbmm(sq.unsqueeze(-1) + sq.unsqueeze(-2), v, v.mT, alpha=-2.0)
        del v
        if on_device:
            # the greedy pass over the candidates, one wavefront per node
            sel = kernels.graph_prune(pair.contiguous(), cd.float().contiguous(),
                                      min(m_keep, K), fill)
            if __debug__:
                assert int(sel.max()) < K and int(sel.min()) >= -1
            ids = torch.gather(c, 1, sel.clamp(min=0))
            out[lo:lo + chunk, :ids.size(1)] = torch.where(
                sel >= 0, ids, torch.full_like(ids, -1))
            continue
        keep = torch.zeros_like(c, dtype=torch.bool)
        count = torch.zeros(c.size(0), dtype=torch.long, device=x.device)
        for j in range(K):
            blocked = ((pair[:, j, :] < cd[:, j:j + 1]) & keep).any(-1)
            take = (~blocked) & (count < m_keep) & present[:, j]
            keep[:, j] = take
            count += take
        # kept ones first (by distance rank), then the nearest rejected
        rank = col.unsqueeze(0) + (~keep) * K + (~present) * 2 * K
        order = torch.argsort(rank, dim=-1)[:, :m_keep]
        ids = torch.gather(c, 1, order)
        if not fill:
            kept = torch.gather(keep, 1, order)
            ids = torch.where(kept, ids, torch.full_like(ids, -1))
        out[lo:lo + chunk, :ids.size(1)] = ids
    return out


def _add_reverse(forward: torch.Tensor, degree: int):
    """Rows of ``degree`` slots: the forward edges, then nodes that point at
    the row's node and are not in it yet, strongest (lowest forward rank)
    first, until the row is full.  ``-1`` pads."""
    n, m = forward.shape
    dev = forward.device
    adj = torch.full((n, degree), -1, dtype=torch.long, device=dev)
    # compact forward edges to the left of each row
    valid = forward >= 0
    order = torch.argsort((~valid).to(torch.int8), dim=-1, stable=True)
    fwd = torch.gather(forward, 1, order)[:, :degree]
    adj[:, :fwd.size(1)] = fwd
    used = (fwd >= 0).sum(-1)

    src = torch.arange(n, device=dev).unsqueeze(-1).expand(n, m)
    rank = torch.arange(m, device=dev).unsqueeze(0).expand(n, m)
    mask = valid
    dst, src, rank = forward[mask], src[mask], rank[mask]
    # drop reverse edges whose target already lists the source
    fkey = (src * n + dst)
    rkey = (dst * n + src)
    new = ~torch.isin(rkey, fkey)
    dst, src, rank = dst[new], src[new], rank[new]
    # group by target, closest-ranked first
    key = dst * m + rank
    order = torch.argsort(key, stable=True)
    dst, src = dst[order], src[order]
    start = torch.searchsorted(dst, torch.arange(n, device=dev))
    pos = torch.arange(dst.numel(), device=dev) - start[dst]
    slot = used[dst] + pos
    ok = slot < degree
    adj[dst[ok], slot[ok]] = src[ok]
    return adj


def reachable(adj: torch.Tensor, sources: torch.Tensor, reverse: bool = False):
    """Boolean mask of the nodes a walk along the edges of ``adj[N, deg]``
    (``-1`` padded) reaches from ``sources``; with ``reverse`` the nodes from
    which a walk reaches one of ``sources``."""
    n = adj.size(0)
    mark = torch.zeros(n, dtype=torch.bool, device=adj.device)
    mark[sources] = True
    if reverse:
        valid = adj >= 0
        safe = adj.clamp(min=0)
        while True:
            grown = mark | (mark[safe] & valid).any(-1)
            if bool((grown == mark).all()):
                return mark
            mark = grown
    frontier = sources.flatten()
    while frontier.numel():
        nb = adj[frontier].flatten()
        nb = nb[nb >= 0]
        frontier = torch.unique(nb[~mark[nb]])
        mark[frontier] = True
    return mark


def _add_edge(row, protected, u: int, v: int):
    """Edge u -> v into ``row``, the row of u (a view, changed in place): into
    its first free slot, else over its farthest neighbour that is not itself
    an edge added here."""
    if u == v or bool((row == v).any()):
        return
    free = torch.nonzero(row < 0).flatten()
    if free.numel():
        row[int(free[0])] = v
        return
    deg = row.numel()
    if int(protected[u]) >= max(1, deg // 4):
        return
    row[deg - 1 - int(protected[u])] = v
    protected[u] += 1


def connect_graph(x: torch.Tensor, adj: torch.Tensor, hub: int = None,
                  max_rounds: int = 32, per_round: int = 1024, seed: int = 0):
    """Makes every node of ``adj[N, deg]`` reachable from the hub (the node
    nearest to the mean of ``x``) and the hub reachable from every node, so
    that a search started anywhere can get everywhere: what faiss' NSG build
    ensures with its spanning tree from the navigating node and an HNSW base
    layer gets from incremental insertion, and a pruned k-nearest-neighbour
    table alone does not (separated clusters stay separate).  Per round, up to
    ``per_round`` nodes that are cut off are each linked, both ways, with the
    nearest node that is not; the rest of their cluster follows through its
    own edges.  Edges go to free slots first, else over the row's farthest
    neighbours (at most a quarter of a row).  In place; returns the number of
    rounds used, or -1 if ``max_rounds`` did not suffice."""
    n, deg = adj.shape
    dev = adj.device
    if hub is None:
        hub = int(torch.argmin((x.float() - x.float().mean(0)).square().sum(-1)))
    hub_t = torch.tensor([hub], device=dev)
    protected = torch.zeros(n, dtype=torch.long)
    g = torch.Generator().manual_seed(seed)
    xf = x.float()
    for round_ in range(max_rounds):
        fwd = reachable(adj, hub_t)
        bwd = reachable(adj, hub_t, reverse=True)
        ok = fwd & bwd
        if bool(ok.all()):
            return round_
        cut = torch.nonzero(~ok).flatten()
        if progress is not None:
            progress(f'connectivity: round {round_}, {cut.numel()} of {n} nodes cut off')
        if cut.numel() > per_round:
            pick = torch.randperm(cut.numel(), generator=g)[:per_round]
            cut = cut[pick.to(dev)]
        inside = torch.nonzero(ok).flatten()
        # connected nodes whose row can still take an edge
        room = (adj[inside] < 0).any(-1) | \
            (protected.to(dev)[inside] < max(1, deg // 4))
        if bool(room.any()):
            inside = inside[room]
        # nearest such node of every picked node, in chunks
        norms = xf[inside].square().sum(-1)
        nearest = []
        step = max(1, (1 << 28) // max(1, inside.numel()))
        for lo in range(0, cut.numel(), step):
            q = xf[cut[lo:lo + step]]
            d = norms.unsqueeze(0) - 2.0 * (q @ xf[inside].T)
            nearest.append(inside[torch.argmin(d, -1)])
        nearest = torch.cat(nearest)
        # the rows that get edges, edited on the host and written back
        touched = torch.unique(torch.cat([cut, nearest]))
        rows = adj[touched].cpu()
        place = {node: i for i, node in enumerate(touched.tolist())}
        for u, t in zip(cut.tolist(), nearest.tolist()):
            _add_edge(rows[place[t]], protected, t, u)
            _add_edge(rows[place[u]], protected, u, t)
        adj[touched] = rows.to(dev)
    fwd = reachable(adj, hub_t)
    bwd = reachable(adj, hub_t, reverse=True)
    return max_rounds if bool((fwd & bwd).all()) else -1


def graph_init(x: torch.Tensor, graph_type: str, n_neighbors: int,
               ef_construct: int = 240, compute_dtype: torch.dtype = None,
               connect: bool = True, seed: int = 0,
               insertion_order: bool = True):
    """``(indptr, indices)`` int64 tensors on the CPU
    (``pilot_ann/utils/graphs.py:80-93``).

    ``nsw``: ``n_neighbors/2`` pruned-and-filled forward edges per node plus
    reverse edges up to ``n_neighbors`` — the shape of an HNSW base layer with
    M = n_neighbors/2 (``graphs.py:52-54``).  ``nsg``: up to ``n_neighbors``
    pruned forward edges without filling, then reverse edges where room is
    left, so rows can end in ``-1`` padding as faiss' NSG rows do.
    ``ef_construct`` is the candidate pool per node.  With ``insertion_order``
    (default; sets of more than 2048 nodes) the nodes are taken in a seeded
    random order and a node's pool is its exact nearest among those before it
    (:func:`insertion_order_candidates`), as in an incrementally built graph:
    the early nodes carry the long edges that make the graph navigable from
    any entry, across clusters (measured on 60 000 unit vectors in 64
    well-separated clusters, 32 random entries, full dimension: recall@10
    0.90 / 0.998 at ef 32 / 128, against 0.39 / 0.48 with every pool taken
    from the whole set, whose edges all stay inside a cluster).  Without it
    the pool is the node's exact nearest neighbours in the whole set.  A large
    pool is what makes the graphs accurate with little effort, and the device
    builds the larger table in nearly the same time.  With ``connect``
    (default) :func:`connect_graph` then links what is still cut off and a
    warning tells if it could not."""
    if x.dim() != 2:
        raise RuntimeError
    n = x.size(0)
    pool = min(max(n_neighbors, ef_construct), n - 1)
    perm = None
    m_fwd = n_neighbors // 2 if graph_type == 'nsw' else n_neighbors
    fill = graph_type == 'nsw'
    if graph_type not in ('nsw', 'nsg'):
        raise RuntimeError
    budget = 1 << (29 if x.is_cuda else 27)      # elements of a chunk's largest tensor
    chunk = max(16, min(2048, budget // (pool * max(x.size(1), pool))))
    if insertion_order and n > 2048:
        g = torch.Generator().manual_seed(seed)
        perm = torch.randperm(n, generator=g).to(x.device)
        x = x[perm].contiguous()
    if perm is not None:
        cand, cand_d = insertion_order_candidates(x, pool)
    else:
        cand, cand_d = knn_graph(x, pool, compute_dtype=compute_dtype)
    fwd = _occlusion_prune(x, cand, cand_d, m_fwd, fill, chunk)
    del cand, cand_d
    adj = _add_reverse(fwd, n_neighbors)
    if connect and n > 1:
        rounds = connect_graph(x, adj)
        if rounds < 0:
            import warnings
            warnings.warn('graph_init: the connectivity pass left nodes cut '
                          'off from the rest of the graph')
            if progress is not None:
                progress('connectivity: nodes left cut off')
    if perm is not None:
        # rows and ids back from insertion order to the caller's numbering
        named = torch.where(adj >= 0, perm[adj.clamp(min=0)], adj)
        adj = torch.empty_like(named)
        adj[perm] = named
    indptr = torch.arange(n + 1, dtype=torch.long) * n_neighbors
    return indptr, adj.flatten().cpu()


def graph_sampling(indptr: torch.Tensor, indices: torch.Tensor,
                   n_samples: int, n_hops: int, seed: int = 0,
                   device: str = 'cpu', return_seeds: bool = False):
    """Seeded version of ``extension/sampling_cpu.cpp:5-65``.  The reference
    draws seed nodes one after the other and adds each with everything within
    ``n_hops`` edges of it, until at least ``n_samples`` nodes are in; the
    same here, with the seeds taken from a seeded random order of the nodes
    (the reference seeds ``rand()`` with the time).  As the sample only grows
    with every seed, the stopping point is found by bisection over the number
    of seeds instead of one seed at a time.  Returns the sorted ``nodelist``
    and ``mapping`` (global id → position in nodelist, else -1), and the
    seeds used with ``return_seeds``."""
    indptr = torch.as_tensor(indptr, dtype=torch.long).to(device)
    indices = torch.as_tensor(indices, dtype=torch.long).to(device)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(seed)
    order = torch.randperm(n, generator=g).to(device)
    row_of_edge = torch.repeat_interleave(
        torch.arange(n, device=device), indptr[1:] - indptr[:-1])

    def closure(m: int):
        mark = torch.zeros(n, dtype=torch.bool, device=device)
        mark[order[:m]] = True
        for _ in range(n_hops):
            hit = indices[mark[row_of_edge]]
            mark[hit[hit >= 0]] = True
        return mark

    lo, hi = 1, n
    while lo < hi:
        mid = (lo + hi) // 2
        if int(closure(mid).sum()) >= n_samples:
            hi = mid
        else:
            lo = mid + 1
    nodelist = torch.nonzero(closure(lo)).flatten().cpu()
    mapping = torch.full((n,), -1, dtype=torch.long)
    mapping[nodelist] = torch.arange(nodelist.numel())
    if return_seeds:
        return nodelist, mapping, order[:lo].cpu()
    return nodelist, mapping


def subgraph_init(indptr: torch.Tensor, indices: torch.Tensor,
                  storage: torch.Tensor, graph_type: str, n_samples: int,
                  n_neighbors: int, n_hops: int = 1, seed: int = 0,
                  compute_dtype: torch.dtype = None):
    """Sample nodes, build a graph on them alone, express it in global ids
    with one row per global node (``pilot_ann/utils/graphs.py:96-132``).
    Returns ``(indptr, indices, nodelist, mapping)``.  Padding stays ``-1``
    (the reference turns it into the last sampled node, ``graphs.py:123-126``;
    both end a row's useful part the same way for the search)."""
    nodelist, mapping = graph_sampling(indptr, indices, n_samples, n_hops,
                                       seed=seed, device=storage.device)
    sub = storage[nodelist.to(storage.device)]
    sg_indptr, sg_indices = graph_init(sub, graph_type, n_neighbors,
                                       compute_dtype=compute_dtype, seed=seed)
    glob = torch.where(sg_indices >= 0,
                       nodelist[sg_indices.clamp(min=0)],
                       torch.full_like(sg_indices, -1))
    n = mapping.numel()
    rowlen = torch.zeros(n, dtype=torch.long)
    rowlen[nodelist] = sg_indptr[1:] - sg_indptr[:-1]
    new_indptr = torch.zeros(n + 1, dtype=torch.long)
    new_indptr[1:] = torch.cumsum(rowlen, 0)
    return new_indptr, glob, nodelist, mapping
