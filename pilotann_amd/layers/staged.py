import torch
from torch import nn

from .. import kernels, utils
from .entry import IndexEntry


class GraphModule(nn.Module):
    """CSR graph as two int64 buffers (``layers/staged.py:6-17``)."""

    def __init__(self, indptr, indices):
        super().__init__()
        self.register_buffer(
            'indptr', torch.as_tensor(indptr, dtype=torch.long).contiguous())
        self.register_buffer(
            'indices', torch.as_tensor(indices, dtype=torch.long).contiguous())


class IndexStaged(nn.Module):
    """Three-stage index, interface of ``pilot_ann/layers/staged.py:20-228``:
    device traversal of the sampled subgraph on the first ``d_principle``
    rotated coordinates, then the host refine on the subgraph and on the full
    graph in full dimension.

    ``seed`` and ``build_device`` are additions: every random choice of the
    build is seeded, and the build-time matrix products run where
    ``build_device`` says (the search-time split is the reference's).
    So are :meth:`stage_refine` and ``search(..., refine='device')``: with the
    full-dimension rows and the full graph on the device as well, the refine
    runs there too and gives the host refine's results.
    """

    def __init__(self, d_model: int, d_principle: int, sample_ratio: float,
                 graph_method: str = 'nsw32', entry_method: str = 'random32',
                 seed: int = 0, build_device: str = 'cpu'):
        super().__init__()
        assert d_principle <= d_model
        self.d_model = d_model
        self.d_principle = d_principle
        self.sample_ratio = sample_ratio
        self.graph_method = graph_method
        self.entry_method = entry_method
        self.seed = seed
        self.build_device = build_device
        self.cuda_device = None
        for graph_type in ['nsw', 'nsg']:
            if graph_method.startswith(graph_type):
                self.graph_type = graph_type
                self.n_neighbors = int(graph_method.removeprefix(graph_type))
                break
        else:
            raise NotImplementedError
        self.entry = IndexEntry(d_model=d_principle, method=entry_method,
                                seed=seed + 3)
        self.storage_cuda = None
        self.subgraph_cuda = None
        self.mapping_cuda = None
        self.fullgraph_cuda = None
        self.storage_full_cuda = None
        self.VT_cuda = None
        self._full_prepared = None
        self._streams = None

    # -- checkpoint: layers/staged.py:59-122 ---------------------------------
    @classmethod
    def load(cls, ckpt_file):
        checkpoint = torch.load(ckpt_file, weights_only=True)
        state = checkpoint['state_dict']
        config = checkpoint['config']
        index = cls(d_model=config['d_model'],
                    d_principle=config['d_principle'],
                    graph_method=config['graph_method'],
                    entry_method=config['entry_method'], sample_ratio=-1.0)
        for name in ['VT', 'storage', 'mapping', 'nodelist']:
            index.register_buffer(name, state[name])
        index.register_module('subgraph', GraphModule(
            state['subgraph.indptr'], state['subgraph.indices']))
        index.register_module('fullgraph', GraphModule(
            state['fullgraph.indptr'], state['fullgraph.indices']))
        for name in ['entry_nodes', 'entry_vectors', 'route_vectors']:
            if 'entry.' + name in state:
                index.entry.register_buffer(name, state['entry.' + name])
        return index

    def dump(self):
        keep = ('VT', 'storage', 'mapping', 'nodelist', 'subgraph.',
                'fullgraph.', 'entry.')
        return {
            'config': {
                'd_model': self.d_model,
                'd_principle': self.d_principle,
                'graph_method': self.graph_method,
                'entry_method': self.entry_method,
            },
            'state_dict': {k: v for k, v in self.state_dict().items()
                           if k.startswith(keep)},
        }

    # -- device residency: layers/staged.py:124-139 ---------------------------
    def to(self, device):
        """Copies what the device stage needs: entries, mapping, the subgraph
        and the first ``d_principle`` coordinates of the sampled rows; the
        search form of the subgraph is prepared here, once."""
        self.cuda_device = device
        self.entry.to(device=device)
        self.subgraph_cuda = GraphModule(self.subgraph.indptr,
                                         self.subgraph.indices).to(device)
        rows = torch.index_select(self.storage, 0, self.nodelist)
        rows = rows[:, :self.d_principle].contiguous().to(device)
        # device rows in a locality-preserving order (utils/layout.py); the
        # host copies (checkpoint format) keep the order of the global ids
        order = utils.locality_order(rows, seed=self.seed)
        place = torch.empty_like(order)
        place[order] = torch.arange(order.numel(), device=order.device)
        self.storage_cuda = rows[order].contiguous()
        mapping = self.mapping.to(device=device).clone()
        sampled = mapping >= 0
        mapping[sampled] = place[mapping[sampled]]
        self.mapping_cuda = mapping
        if torch.device(device).type == 'cuda':
            self.VT_cuda = self.VT.to(device)
            kernels.prepare_graph(
                self.subgraph_cuda.indptr, self.subgraph_cuda.indices,
                self.mapping_cuda, self.storage_cuda.size(0), self.n_neighbors)
            # The two streams of the device search are made and used once
            # now, early: the runtime hands streams their hardware queue (of
            # a few) at first use, in turn, and a pair first used later may
            # end up sharing a queue with the stream the search is called on
            # (the two halves of a batch then run one after the other:
            # measured 10.9 instead of 8.8 ms per 10 000 queries).
            if self._streams is None:
                self._streams = [torch.cuda.Stream(device=device)
                                 for _ in range(2)]
                for stream in self._streams:
                    with torch.cuda.stream(stream):
                        torch.zeros(1, device=device)
                    stream.synchronize()
        return self

    def stage_refine(self):
        """Copies what the refine needs to the device chosen by :meth:`to`:
        all rows in full dimension, the full graph (prepared once) and the
        rotation."""
        device = self.cuda_device
        assert device is not None and self.storage_cuda is not None, \
            'call .to(device) first (again after a new build)'
        # not through the cache of prepare_rows: the plain device copy is
        # dropped once its device layout exists
        self.storage_full_cuda = kernels.PreparedRows(
            self.storage.to(device).contiguous())
        self.VT_cuda = self.VT.to(device)
        self.fullgraph_cuda = GraphModule(self.fullgraph.indptr,
                                          self.fullgraph.indices).to(device)
        # kept: a later search neither measures the longest row again (a
        # reduction and a device synchronisation) nor looks the graph up
        self._full_prepared = kernels.prepare_full_graph(
            self.fullgraph_cuda.indptr, self.fullgraph_cuda.indices)
        return self

    def _drop_device_copies(self):
        """What :meth:`to` and :meth:`stage_refine` put on the device belongs
        to the buffers they were made from: after the buffers change (a new
        build, buffers registered again) the copies are made anew."""
        self.storage_cuda = self.subgraph_cuda = self.mapping_cuda = None
        self.fullgraph_cuda = self.storage_full_cuda = self.VT_cuda = None
        self._full_prepared = None

    # -- build: layers/staged.py:141-189 --------------------------------------
    def train(self, x: torch.Tensor):
        assert x.dim() == 2
        assert x.size(-1) == self.d_model
        assert 0.0 < self.sample_ratio <= 1.0
        self._drop_device_copies()
        dev = self.build_device
        half = torch.float16 if torch.device(dev).type == 'cuda' else None

        print('svd', self.d_principle)
        xr, V = utils.svd(x.to(dev), max_size=10_000_000, seed=self.seed)
        self.register_buffer('storage', xr.cpu().contiguous())
        self.register_buffer('VT', V.T.contiguous().cpu())

        print('build', self.graph_type)
        graph = utils.graph_init(xr, graph_type=self.graph_type,
                                 n_neighbors=self.n_neighbors,
                                 compute_dtype=half, seed=self.seed)
        self.register_module('fullgraph', GraphModule(graph[0], graph[1]))

        print('sampling', self.sample_ratio)
        sub = utils.subgraph_init(
            indptr=graph[0], indices=graph[1], storage=xr,
            graph_type=self.graph_type,
            n_samples=round(self.sample_ratio * x.size(0)),
            n_neighbors=self.n_neighbors, seed=self.seed + 1,
            compute_dtype=half)
        self.register_module('subgraph', GraphModule(sub[0], sub[1]))
        self.register_buffer('nodelist', sub[2].contiguous())
        self.register_buffer('mapping', sub[3].contiguous())

        self.entry.train(self.storage[:, :self.d_principle])
        return self

    # -- search: layers/staged.py:191-228 -------------------------------------
    @torch.no_grad()
    def search(self, query: torch.Tensor, k: int, ef_search: int,
               chunk_size: int = 128, refine: str = 'host',
               rotate: str = 'device', traversal: str = 'exact'):
        """``rotate='device'`` (default on a GPU) uploads the query and
        rotates it there (``kernels.rotate``), then copies the rotated query
        back for the host refine; ``rotate='host'`` is the reference's host
        matmul (``layers/staged.py:198``).  The two agree to float rounding.
        ``traversal='wide'`` (with ``refine='device'``) takes the candidates
        from the labelled throughput mode of the traversal
        (``kernels.traverse_wide_prepared``) instead of the exact one."""
        assert query.dim() == 2
        assert traversal in ('exact', 'wide')
        if refine == 'device':
            return self._search_on_device(query, k, ef_search, traversal)
        assert refine == 'host' and traversal == 'exact'
        if rotate == 'device' and self.VT_cuda is not None:
            rotated = kernels.rotate(
                query.to(device=self.cuda_device).contiguous(), self.VT_cuda)
            query_cuda = rotated[:, :self.d_principle].contiguous()
            query = rotated.cpu()
        else:
            query = torch.matmul(query, self.VT.T).contiguous()
            query_cuda = query[:, :self.d_principle].contiguous().to(
                device=self.cuda_device)
        EP_I, EP_D = self.entry.search(query_cuda)
        return kernels.pipeline(
            graph=[self.fullgraph.indptr, self.fullgraph.indices],
            storage=self.storage,
            subgraph=[self.subgraph.indptr, self.subgraph.indices],
            subgraph_cuda=[self.subgraph_cuda.indptr,
                           self.subgraph_cuda.indices, self.mapping_cuda],
            storage_cuda=self.storage_cuda, query=query,
            query_cuda=query_cuda, initial_I=EP_I.contiguous(),
            initial_D=EP_D.contiguous(), k=k, n_neighbors=self.n_neighbors,
            ef_search=ef_search, d_principle=self.d_principle,
            chunk_size=chunk_size)

    @torch.no_grad()
    def search_cpu(self, query: torch.Tensor, k: int, ef_search: int):
        """The search without a device, as a baseline: rotation on the host,
        the entry ids the router would give (nearest route vector over the
        first ``d_principle`` coordinates) with their full-dimension
        distances, then ``traverse_cpu`` on the full graph in full dimension.
        Not part of the reference's index; it plays the role faiss' HNSW has
        in the reference's benchmark (``script/common.py:103-120``)."""
        query = torch.matmul(query.cpu(), self.VT.T).contiguous()
        entry = self.entry
        nodes = entry.entry_nodes.cpu()
        batch = query.size(0)
        if entry.route_vectors is not None:
            route = torch.cdist(query[:, :self.d_principle],
                                entry.route_vectors.cpu()).argmin(-1)
            ids = nodes[route].contiguous()
            dist = torch.empty(ids.shape, dtype=torch.float)
            for r in torch.unique(route).tolist():
                rows = torch.nonzero(route == r).flatten()
                leaves = self.storage[nodes[r]]
                dist[rows] = torch.cdist(query[rows], leaves).square()
        else:
            ids = nodes.unsqueeze(0).expand(batch, -1).contiguous()
            dist = torch.cdist(query, self.storage[nodes]).square().contiguous()
        topk_I = torch.empty(batch, k, dtype=torch.long)
        topk_D = torch.empty(batch, k, dtype=torch.float)
        kernels.traverse_cpu(topk_I, topk_D, ids, dist, self.fullgraph.indptr,
                             self.fullgraph.indices, self.storage, query,
                             max(ef_search, k))
        return topk_I, topk_D

    def _search_on_device(self, query, k, ef_search, traversal='exact'):
        """All three stages on the device: entries, subgraph traversal, refine,
        top-k copied back at the end.  A batch of 2048 queries or more is
        searched as two halves on two streams: while the last searches of one
        half's launch finish, the other half's launch fills the idle
        wavefront slots (6 % on the headline configuration; more chunks only
        add launches).  The query is rotated on the device
        (``kernels.rotate``); given the same rotated query the results are
        those of the host refine."""
        assert self.storage_cuda is not None, \
            'call .to(device) first (again after a new build)'
        if self.storage_full_cuda is None or self._full_prepared is None:
            self.stage_refine()
        device = self.cuda_device
        query = kernels.rotate(query.to(device).contiguous(), self.VT_cuda)
        query_cuda = query[:, :self.d_principle].contiguous()
        EP_I, EP_D = self.entry.search(query_cuda)
        EP_I, EP_D = EP_I.contiguous(), EP_D.contiguous()
        batch = query.size(0)
        cand_I = torch.empty(batch, kernels.BEAM_WIDTH, ef_search,
                             dtype=torch.long, device=device)
        cand_D = torch.empty(batch, kernels.BEAM_WIDTH, ef_search,
                             dtype=torch.float, device=device)
        topk_I = torch.empty(batch, k, dtype=torch.long, device=device)
        topk_D = torch.empty(batch, k, dtype=torch.float, device=device)
        sub = kernels.prepare_graph(
            self.subgraph_cuda.indptr, self.subgraph_cuda.indices,
            self.mapping_cuda, self.storage_cuda.size(0), self.n_neighbors)
        full = self._full_prepared

        traverse = (kernels.traverse_wide_prepared if traversal == 'wide'
                    else kernels.traverse_prepared)

        def run(lo, hi):
            traverse(cand_I[lo:hi], cand_D[lo:hi], sub, self.storage_cuda,
                     query_cuda[lo:hi], EP_I[lo:hi], EP_D[lo:hi])
            c_I, c_D = cand_I[lo:hi].flatten(1), cand_D[lo:hi].flatten(1)
            kernels.traverse_refine_cuda(
                topk_I[lo:hi], topk_D[lo:hi], c_I, c_D, c_I, c_D, sub, full,
                self.storage_full_cuda, query[lo:hi], ef_search,
                self.d_principle)

        if batch < 2048:
            run(0, batch)
        else:
            if self._streams is None:
                self._streams = [torch.cuda.Stream(device=device)
                                 for _ in range(2)]
            current = torch.cuda.current_stream(device)
            ready = torch.cuda.Event()
            ready.record(current)
            half = (batch + 1) // 2
            for stream, (lo, hi) in zip(self._streams,
                                        [(0, half), (half, batch)]):
                stream.wait_event(ready)
                with torch.cuda.stream(stream):
                    run(lo, hi)
            for stream in self._streams:
                current.wait_stream(stream)
        return topk_I.cpu(), topk_D.cpu()
