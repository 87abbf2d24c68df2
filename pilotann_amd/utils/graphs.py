"""Proximity graphs in the reference's layout, built with torch only.

Layout (``pilot_ann/utils/graphs.py:22-40``): ``indptr[i] = i * n_neighbors``,
``indices`` padded with ``-1`` after a row's last neighbour.  A subgraph keeps
global ids and one (possibly empty) row per global node
(``graphs.py:118-129``).  Construction differs from the reference, which
delegates to faiss: here an exact k-nearest-neighbour table is pruned with the
usual occlusion rule and completed with reverse edges.  Everything runs on the
device ``x`` lives on, so a million-node build is a matter of a GPU minute.
"""
import torch


def knn_graph(x: torch.Tensor, k: int, chunk: int = None,
              compute_dtype: torch.dtype = None):
    """Exact ``k`` nearest other rows of every row: ``(ids[N, k], d2[N, k])``
    sorted by squared L2, self excluded.  ``compute_dtype`` (e.g. float16 on
    a GPU) is used for the N×N products only."""
    n = x.size(0)
    k = min(k, n - 1)
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


def _occlusion_prune(x, cand, cand_d, m_keep: int, fill: bool, chunk: int):
    """Keep candidate e (closest first) unless an already kept r is closer to
    e than the node itself is; with ``fill`` the nearest rejected candidates
    top the row up to ``m_keep``.  Returns ids[N, m_keep], ``-1`` padded."""
    n, K = cand.shape
    out = torch.full((n, m_keep), -1, dtype=torch.long, device=x.device)
    col = torch.arange(K, device=x.device)
    for lo in range(0, n, chunk):
        c = cand[lo:lo + chunk]
        cd = cand_d[lo:lo + chunk]
        v = x[c].float()
        sq = v.square().sum(-1)
        pair = sq.unsqueeze(-1) + sq.unsqueeze(-2) - 2.0 * (v @ v.mT)
        keep = torch.zeros_like(c, dtype=torch.bool)
        count = torch.zeros(c.size(0), dtype=torch.long, device=x.device)
        for j in range(K):
            blocked = ((pair[:, j, :] < cd[:, j:j + 1]) & keep).any(-1)
            take = (~blocked) & (count < m_keep)
            keep[:, j] = take
            count += take
        # kept ones first (by distance rank), then the nearest rejected
        rank = col.unsqueeze(0) + (~keep) * K
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


def graph_init(x: torch.Tensor, graph_type: str, n_neighbors: int,
               ef_construct: int = 80, compute_dtype: torch.dtype = None):
    """``(indptr, indices)`` int64 tensors on the CPU
    (``pilot_ann/utils/graphs.py:80-93``).

    ``nsw``: ``n_neighbors/2`` pruned-and-filled forward edges per node plus
    reverse edges up to ``n_neighbors`` — the shape of an HNSW base layer with
    M = n_neighbors/2 (``graphs.py:52-54``).  ``nsg``: up to ``n_neighbors``
    pruned forward edges without filling, then reverse edges where room is
    left, so rows can end in ``-1`` padding as faiss' NSG rows do.
    ``ef_construct`` bounds the candidate pool per node."""
    if x.dim() != 2:
        raise RuntimeError
    n = x.size(0)
    pool = max(n_neighbors, min(ef_construct, 2 * n_neighbors))
    pool = min(pool, n - 1)
    cand, cand_d = knn_graph(x, pool, compute_dtype=compute_dtype)
    chunk = max(16, min(2048, (1 << 27) // (pool * max(x.size(1), pool))))
    if graph_type == 'nsw':
        fwd = _occlusion_prune(x, cand, cand_d, n_neighbors // 2, True, chunk)
    elif graph_type == 'nsg':
        fwd = _occlusion_prune(x, cand, cand_d, n_neighbors, False, chunk)
    else:
        raise RuntimeError
    adj = _add_reverse(fwd, n_neighbors)
    indptr = torch.arange(n + 1, dtype=torch.long) * n_neighbors
    return indptr, adj.flatten().cpu()


def graph_sampling(indptr: torch.Tensor, indices: torch.Tensor,
                   n_samples: int, n_hops: int, seed: int = 0,
                   device: str = 'cpu'):
    """Seeded version of ``extension/sampling_cpu.cpp:5-65``: random seed
    nodes, each with its ``n_hops`` neighbourhood, are added in a fixed random
    order until at least ``n_samples`` nodes are in.  Returns the sorted
    ``nodelist`` and ``mapping`` (global id → position in nodelist, else -1).
    """
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
                                       compute_dtype=compute_dtype)
    glob = torch.where(sg_indices >= 0,
                       nodelist[sg_indices.clamp(min=0)],
                       torch.full_like(sg_indices, -1))
    n = mapping.numel()
    rowlen = torch.zeros(n, dtype=torch.long)
    rowlen[nodelist] = sg_indptr[1:] - sg_indptr[:-1]
    new_indptr = torch.zeros(n + 1, dtype=torch.long)
    new_indptr[1:] = torch.cumsum(rowlen, 0)
    return new_indptr, glob, nodelist, mapping
