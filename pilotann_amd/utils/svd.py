import torch


def svd(x: torch.Tensor, max_size: int, seed: int = 0):
    """Rotate ``x`` onto its right singular vectors, strongest first.

    Returns ``(x @ V, V)`` like ``pilot_ann/utils/svd.py:4-21``.  The basis
    comes from the eigenvectors of the d×d Gram matrix of (a seeded sample of
    at most ``max_size`` rows of) ``x``, accumulated in float64: the same
    subspace as ``torch.svd`` gives, at O(n·d²) instead of a full SVD.
    """
    assert x.dim() == 2
    rows = x
    if x.size(0) > max_size:
        g = torch.Generator().manual_seed(seed)
        index = torch.randint(high=x.size(0), size=[max_size], generator=g)
        rows = torch.index_select(x, 0, index.to(x.device))
    gram = torch.zeros(x.size(1), x.size(1), dtype=torch.float64,
                       device=x.device)
    for part in torch.split(rows, 262144):
        part = part.double()
        gram += part.T @ part
    evals, evecs = torch.linalg.eigh(gram)
    order = torch.argsort(evals, descending=True)
    V = evecs[:, order].to(x.dtype).contiguous()
    out = torch.cat([part @ V for part in torch.split(x, 262144)])
    return out, V
