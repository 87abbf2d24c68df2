"""A best-first graph search in plain Python, the yardstick the reference's
graph tests measure a freshly built graph with
(``pilot_ann/utils/search.py:6-102``, used by ``test/kernel/test_graphs.py``).
It is not the search of the kernels: open list and result list are ordinary
binary heaps, and missing entries are drawn at random."""
import heapq
import random

import torch


def search_simple(indptr, indices, mapping, storage: torch.Tensor,
                  query: torch.Tensor, k: int, ef_search: int,
                  closedlist=None, max_iterations: int = 1024, ep=None,
                  rng: random.Random = None):
    """Searches one ``query``.  ``indptr`` / ``indices``: padded CSR in
    global ids (``-1`` pads), ``mapping``: global id -> row of ``storage``.
    ``ep``: entry ids, taken from the back; while the open list holds fewer
    than ``ef_search`` nodes further entries are drawn at random (``rng``,
    default the module ``random``) among the graph's edge targets.
    ``closedlist``: ids to treat as visited.  Returns the reference's
    dictionary: ``topk`` (ids, unordered), ``n_steps``, ``visited``,
    ``n_visited``, ``n_computed``."""
    assert query.dim() == 1 and storage.dim() == 2
    assert query.size(-1) == storage.size(-1)
    assert len(mapping) == len(indptr) - 1
    rng = rng or random
    ep = list(ep) if ep else []

    def dist(u):
        return torch.dist(query, storage[mapping[u]], p=2.0).item()

    visited, computed = set(), set()
    openlist, best = [], []          # best: max-heap through negated keys
    pool = None
    while True:
        if ep:
            u = ep.pop()
        elif len(openlist) >= ef_search:
            break
        else:
            if pool is None:
                pool = [v for v in indices if v >= 0]
            if len(visited) >= len(set(pool)):
                break                # fewer reachable nodes than ef_search
            u = rng.choice(pool)
        if u in visited:
            continue
        visited.add(u)
        d = dist(u)
        heapq.heappush(openlist, (d, u))
        heapq.heappush(best, (-d, u))
    for u in closedlist or ():
        visited.add(u)

    step = 0
    for step in range(min(max_iterations, 2 * ef_search)):
        if not openlist:
            break
        if len(openlist) > ef_search:
            openlist = [heapq.heappop(openlist) for _ in range(ef_search)]
        while len(best) > ef_search:
            heapq.heappop(best)
        d, u = heapq.heappop(openlist)
        if d >= -best[0][0]:
            break
        fresh = []
        for v in indices[indptr[u]:indptr[u + 1]]:
            if v < 0 or v in visited:
                continue
            fresh.append(v)
            computed.add(v)
            visited.add(v)
        for v in fresh:
            d = dist(v)
            heapq.heappush(openlist, (d, v))
            heapq.heappush(best, (-d, v))
    while len(best) > k:
        heapq.heappop(best)
    return {
        'topk': [u for _, u in best],
        'n_steps': step,
        'visited': visited,
        'n_visited': len(visited),
        'n_computed': len(computed),
    }
