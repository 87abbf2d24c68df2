"""Seeded synthetic data in the shapes the benchmark configurations name."""
import torch


def gaussian_mixture(n: int, d: int, n_centers: int, sigma: float, seed: int,
                     normalize: bool = False, device: str = 'cpu',
                     center_seed: int = None, decay: float = 0.0,
                     device_rng: bool = False):
    """``n`` points of an isotropic Gaussian mixture: centres ~ N(0, I_d),
    a uniformly drawn centre plus ``sigma``·N(0, I_d) per point; optionally
    projected onto the unit sphere.  ``center_seed`` fixes the centres apart
    from the points, so that queries (another ``seed``) share the base set's
    mixture.  With ``decay`` > 0 coordinate j (of centres and noise alike)
    is scaled by (1 + j)^(-decay): a power-law spectrum like that of learned
    embeddings, where the leading SVD coordinates carry most of a distance;
    ``decay`` = 0 is the isotropic mixture.  ``device_rng`` draws the noise
    with ``device``'s own generator (another stream of numbers for the same
    seed; for sets too large to draw on the host in reasonable time)."""
    gc = torch.Generator(device='cpu').manual_seed(
        seed if center_seed is None else center_seed)
    centers = torch.randn(n_centers, d, generator=gc)
    g = torch.Generator(device='cpu').manual_seed(seed + 7919)
    which = torch.randint(high=n_centers, size=[n], generator=g)
    out = torch.empty(n, d, device=device)
    scale = torch.arange(1, d + 1, dtype=torch.float32).pow(-decay).to(device)
    centers = centers.to(device)
    gd = None
    if device_rng:
        gd = torch.Generator(device=device).manual_seed(seed + 7919)
    for lo in range(0, n, 131072):
        hi = min(n, lo + 131072)
        if device_rng:
            noise = torch.randn(hi - lo, d, generator=gd, device=device)
        else:
            noise = torch.randn(hi - lo, d, generator=g).to(device)
        out[lo:hi] = (centers[which[lo:hi].to(device)] + sigma * noise) * scale
    if normalize:
        out = torch.nn.functional.normalize(out, dim=-1)
    return out


def brute_force_topk(query: torch.Tensor, storage: torch.Tensor, k: int,
                     chunk: int = 1024):
    """Exact k nearest rows of ``storage`` (squared L2) for every query."""
    norms = storage.square().sum(-1)
    ids = []
    for q in torch.split(query, chunk):
        d = norms.unsqueeze(0) - 2.0 * (q @ storage.T)
        ids.append(torch.topk(d, k=k, dim=-1, largest=False).indices)
    return torch.cat(ids)
