import random

import torch


def router_init(storage: torch.Tensor, init_nodes: list, n_routers: int,
                n_leaves: int, seed: int = 0):
    """Two-level entry router, as ``pilot_ann/utils/router.py:5-58`` builds
    it, with a seeded generator instead of the process-global one.

    Level 0: grow a set of ``n_routers`` route nodes; each round draws
    ``n_routers`` random nodes and keeps the one whose summed distance to the
    routes chosen so far is largest.  Level 1: ``n_leaves`` rounds; each round
    draws min(1024, n_routers²) unseen nodes (taken from the end of
    ``init_nodes`` while it lasts) and gives every route its nearest of them
    as a leaf.  Returns ``(route_vectors[R, d], entry_nodes[R, L] int64)``.
    """
    assert storage.dim() == 2
    rng = random.Random(seed)
    n_storage = storage.size(0)
    init_nodes = list(init_nodes) if init_nodes else []

    if n_routers > n_storage:
        raise RuntimeError(f'{n_routers} routes from {n_storage} nodes')
    chosen = [rng.randrange(n_storage)]
    member = set(chosen)
    while len(chosen) < n_routers:
        nodes = [rng.randrange(n_storage) for _ in range(n_routers)]
        dists = torch.cdist(storage[nodes].float(), storage[chosen].float())
        pick = nodes[int(torch.argmax(dists.sum(-1)))]
        if pick not in member:
            member.add(pick)
            chosen.append(pick)
    route_vectors = storage[chosen]

    visited = set()
    entry_nodes = [[] for _ in range(n_routers)]
    per_round = min(1024, n_routers ** 2)
    if n_routers > n_storage or per_round * n_leaves > n_storage:
        # the rounds below draw unseen nodes until they have enough
        raise RuntimeError(
            f'router{n_routers}x{n_leaves} needs {per_round * n_leaves} '
            f'distinct nodes, the set has {n_storage}')
    for _ in range(n_leaves):
        nodes = []
        while len(nodes) < per_round:
            if init_nodes:
                new_node = init_nodes.pop(-1)
            else:
                new_node = rng.randrange(n_storage)
            if new_node in visited:
                continue
            visited.add(new_node)
            nodes.append(new_node)
        dists = torch.cdist(route_vectors.float(), storage[nodes].float())
        nearest = torch.argmin(dists, dim=-1).tolist()
        for r in range(n_routers):
            entry_nodes[r].append(nodes[nearest[r]])
    return route_vectors, torch.tensor(entry_nodes, dtype=torch.long)
