"""Order of the reduced rows in device memory.

The traversal marks visited rows in a bitmask with one bit per storage row.
A search touches a few thousand rows that are close to each other in space;
when rows that are close in space are also close in memory, those marks fall
into a fraction of the bitmask's cache lines and the atomic updates find them
in L2.  The reference keeps the sampled rows in the order of their global ids
(``pilot_ann/utils/graphs.py:118-129``), which carries no locality; the order
is free, since ``mapping`` is whatever assigns a row to a node.
"""
import torch


def locality_order(rows: torch.Tensor, n_cells: int = None, seed: int = 0,
                   chunk: int = 16384) -> torch.Tensor:
    """A permutation of ``range(len(rows))`` that puts rows of the same cell
    next to each other: ``n_cells`` rows drawn with ``seed`` are the cell
    centres, every row belongs to its nearest centre, cells follow each other
    in the order of their centres' first coordinate and rows keep their order
    inside a cell.  ``result[r]`` is the old position of the row that comes
    to position ``r``."""
    n = rows.size(0)
    if n_cells is None:
        n_cells = max(16, min(1024, n // 1024))
    n_cells = max(1, min(n_cells, n))
    g = torch.Generator().manual_seed(seed)
    pick = torch.randperm(n, generator=g)[:n_cells].to(rows.device)
    centres = rows[pick].float()
    cell = torch.cat([
        torch.cdist(rows[i:i + chunk].float(), centres).argmin(1)
        for i in range(0, n, chunk)])
    rank = torch.argsort(torch.argsort(centres[:, 0]))
    return torch.argsort(rank[cell], stable=True)
