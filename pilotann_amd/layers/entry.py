import torch
from torch import nn

from .. import kernels, utils


class IndexEntry(nn.Module):
    """Entry-point selection, interface of ``pilot_ann/layers/entry.py:6-89``.

    ``method`` is ``random<n>`` (a fixed random list of n entries shared by
    all queries) or ``router<R>x<L>`` (R route vectors with L leaf entries
    each; a query takes all leaves of its nearest route).  ``seed`` fixes the
    random choices the reference leaves to the global generators.
    """

    def __init__(self, d_model: int, method: str = 'random32', seed: int = 0):
        super().__init__()
        self.method = method
        self.d_model = d_model
        self.seed = seed
        self.register_buffer('entry_nodes', None)
        self.register_buffer('entry_vectors', None)
        self.register_buffer('route_vectors', None)

    def nodes(self):
        return self.entry_nodes.flatten().tolist()

    def train(self, storage: torch.Tensor, init_nodes: list = None):
        assert isinstance(storage, torch.Tensor)
        if storage.dim() != 2:
            raise RuntimeError
        if storage.size(-1) != self.d_model:
            raise RuntimeError
        if self.entry_nodes is not None:
            return
        print('[INFO] building entry')
        if self.method.startswith('random'):
            n_entries = int(self.method.removeprefix('random'))
            g = torch.Generator().manual_seed(self.seed)
            entry_nodes = torch.randint(high=storage.size(0), size=[n_entries],
                                        dtype=torch.long, generator=g)
            route_vectors = None
        elif self.method.startswith('router'):
            n_routers, n_leaves = [
                int(x) for x in self.method.removeprefix('router').split('x')]
            route_vectors, entry_nodes = utils.router_init(
                storage=storage, init_nodes=init_nodes, n_routers=n_routers,
                n_leaves=n_leaves, seed=self.seed)
            route_vectors = route_vectors.contiguous()
        else:
            raise NotImplementedError
        self.register_buffer('entry_nodes', entry_nodes)
        self.register_buffer(
            'entry_vectors',
            storage[entry_nodes.to(storage.device)].contiguous())
        self.register_buffer('route_vectors', route_vectors)
        return self

    @torch.no_grad()
    def search(self, query: torch.Tensor):
        """``(EP_I, EP_D)``: entry ids ``[B, n]`` and their squared distances
        (``entry.py:64-89``).  On a GPU both modes run the library's distance
        kernel; on the CPU the random mode falls back to torch, as in the
        reference, and the router mode is not available."""
        assert query.dim() == 2
        batch_size = query.size(0)
        if self.route_vectors is None:
            assert self.entry_vectors.dim() == 2
            if query.is_cuda:
                EP_D = kernels.entry_distances(query, self.entry_vectors)
            else:
                EP_D = torch.square(
                    torch.cdist(query, self.entry_vectors, p=2.0))
            EP_I = torch.tile(self.entry_nodes.unsqueeze(0),
                              dims=[batch_size, 1])
        else:
            assert query.is_cuda is True
            assert self.entry_vectors.dim() == 3
            _, EP_D, EP_I = kernels.routing_cuda(
                query, self.route_vectors, entry_nodes=self.entry_nodes,
                entry_vectors=self.entry_vectors, return_entries=True)
        return EP_I, EP_D
