"""Shared builders and comparisons for the tests."""
import numpy as np
import torch

from pilotann_amd import utils


class Problem:
    """A small index: rotated base set, full graph, sampled subgraph."""

    def __init__(self, n=4000, d=32, n_centers=16, sigma=0.6, deg=32,
                 graph_type='nsw', sample_ratio=0.25, seed=0, n_query=64,
                 pad_like_reference=False):
        self.n, self.d, self.deg = n, d, deg
        x = utils.gaussian_mixture(n, d, n_centers, sigma, seed=seed)
        self.x = x.contiguous()
        self.query = utils.gaussian_mixture(
            n_query, d, n_centers, sigma, seed=seed + 1, center_seed=seed)
        self.indptr, self.indices = utils.graph_init(x, graph_type, deg)
        if sample_ratio is None:
            self.sub_indptr, self.sub_indices = self.indptr, self.indices
            self.nodelist = torch.arange(n)
            self.mapping = torch.arange(n)
        else:
            sub = utils.subgraph_init(
                self.indptr, self.indices, x, graph_type,
                n_samples=round(sample_ratio * n), n_neighbors=deg,
                seed=seed + 2)
            self.sub_indptr, self.sub_indices, self.nodelist, self.mapping = sub
            if pad_like_reference:
                # pilot_ann/utils/graphs.py:123-126 turns -1 padding into the
                # last sampled node
                last = int(self.nodelist[-1])
                self.sub_indices = torch.where(
                    self.sub_indices < 0,
                    torch.full_like(self.sub_indices, last), self.sub_indices)

    def entries(self, n_init, seed, dp=None, sampled_only=False):
        """Random entry ids with their exact reduced-space distances."""
        g = torch.Generator().manual_seed(seed)
        B = self.query.size(0)
        if sampled_only:
            pick = torch.randint(high=self.nodelist.numel(),
                                 size=[B, n_init], generator=g)
            ids = self.nodelist[pick]
        else:
            ids = torch.randint(high=self.n, size=[B, n_init], generator=g)
        dp = dp or self.d
        import oracle
        dist = np.stack([
            oracle.square_dist(
                np.ascontiguousarray(self.query[b, :dp].numpy()),
                np.ascontiguousarray(self.x[:, :dp].numpy()),
                ids[b].numpy().copy())
            for b in range(B)])
        return ids.contiguous(), torch.from_numpy(dist)


def assert_same_search(I_a, D_a, I_b, D_b, worst_tie=None):
    """Distances identical bit for bit; ids identical except inside a run of
    equal distances of one row, where only the set has to agree.

    ``worst_tie(row, ids)`` (optional) is asked when the sets differ at the
    worst distance a row keeps: two candidates at exactly that distance
    competed for the last place, and which of them a list drops first is
    heap-structure detail with no effect on the search.  It gets the ids of
    the first list at that distance and must check that each is a candidate
    at exactly that distance."""
    D_a, D_b = np.asarray(D_a), np.asarray(D_b)
    I_a, I_b = np.asarray(I_a), np.asarray(I_b)
    assert D_a.shape == D_b.shape and I_a.shape == I_b.shape
    same_d = (D_a == D_b) | (np.isnan(D_a) & np.isnan(D_b))
    assert same_d.all(), (
        f'{(~same_d).sum()} distances differ; first row '
        f'{np.argwhere(~same_d)[0]}')
    bad = np.argwhere((I_a != I_b).any(-1)).flatten()
    for r in bad:
        real = I_a[r] >= 0
        worst = D_a[r][real].max() if real.any() else None
        for dist in np.unique(D_a[r][I_a[r] != I_b[r]]):
            sel = D_a[r] == dist
            if sorted(I_a[r][sel]) == sorted(I_b[r][sel]):
                continue
            assert worst_tie is not None and dist == worst, (
                f'row {r}: ids differ outside a tie at distance {dist}')
            assert (I_a[r][sel] >= 0).all() and (I_b[r][sel] >= 0).all()
            worst_tie(int(r), I_a[r][sel], dist)
