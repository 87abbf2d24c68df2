"""Command line benchmark in the shape of the reference's ``script/bench_1.py``
and ``script/common.py``: build an index, then for every ``ef_search`` run
warm-up + timed searches of ``n_queries`` queries and print

    search-pilot: recall=0.904, duration=15.630ms

(mean recall@k and mean wall-clock milliseconds per call, ``perf_counter``
around ``IndexStaged.search``; 2 warm-up and 20 timed repeats like
``script/common.py:151-197``, each on a fresh random draw of the query pool,
without the reference's two-second sleeps).  The reference's second method,
faiss on the CPU, is not available here; its role — the search without a GPU
— is played by the library's host search on the full graph
(``host-cpu: recall=…, duration=…ms``).

Datasets: the reference's names (``deep-1m``, ``text2img-10m``, ``wiki-1m``,
``laion-1m``, ``fuzz-64k`` …, read by ``utils.DataLoader`` from
``--data_root``, default ``.dataset`` as in the reference), or a synthetic
unit-norm Gaussian mixture, ``synth:<n>x<d>[:<centres>[:<spectrum
exponent>]]``; the default is the shape of the headline benchmark
(``synth:1000000x768:1024:0`` with ``--d_principle 128 --n_neighbors 64
--router router64x64``).

    python -m pilotann_amd.cli --dataset synth:200000x128:64:0.5 \\
        --d_principle 64 --n_neighbors 32 --router router32x32 --ef_search 16,32,64
"""
import argparse
import time

import torch

from . import layers, utils

N_WARMUP = 2
CHUNK_SIZE = 256          # script/common.py:23
QUERY_POOL = 4096         # utils/loader.py:10


def parse_dataset(name: str):
    """``synth:<n>x<d>[:<centres>[:<spectrum exponent>]]`` -> generator
    arguments (unit-norm mixture, sigma 1, seed 7)."""
    parts = name[len('synth:'):].split(':')
    n, d = (int(v) for v in parts[0].lower().split('x'))
    centres = int(parts[1]) if len(parts) > 1 else 64
    decay = float(parts[2]) if len(parts) > 2 else 0.0
    return dict(n=n, d=d, n_centers=centres, sigma=1.0, decay=decay,
                normalize=True, seed=7)


class Profiler:
    """``ANNProfiler`` of ``script/common.py:21-197`` for this library."""

    def __init__(self, dataset, algorithm, n_queries, d_principle,
                 entry_method, sample_ratio, device, refine='host',
                 data_root='.dataset', seed=7, traversal='exact'):
        self.algorithm = algorithm
        self.n_queries = n_queries
        self.d_principle = d_principle
        self.entry_method = entry_method
        self.sample_ratio = sample_ratio
        self.device = device
        self.refine = refine
        self.traversal = traversal
        self.seed = seed
        self.index = None
        self.method = None
        self.loader = None
        self.targets = {}
        self.draw = torch.Generator().manual_seed(seed + 2)
        if dataset.startswith('synth:'):
            s = parse_dataset(dataset)
            kw = dict(normalize=s['normalize'], device=device, decay=s['decay'])
            self.storage = utils.gaussian_mixture(
                s['n'], s['d'], s['n_centers'], s['sigma'], seed=s['seed'], **kw)
            self.queries = utils.gaussian_mixture(
                QUERY_POOL, s['d'], s['n_centers'], s['sigma'], seed=s['seed'] + 1,
                center_seed=s['seed'], **kw)
        else:
            try:
                self.loader = utils.DataLoader(dataset, root=data_root, seed=seed,
                                               device=device)
            except NotImplementedError:
                raise SystemExit(
                    f'unknown dataset {dataset!r}: a name of the reference '
                    '(deep-1m, text2img-1m, wiki-1m, laion-1m, fuzz-64k, ...) or '
                    'synth:<n>x<d>[:<centres>[:<spectrum exponent>]]')
            self.storage = self.loader.load_storage()
            if self.storage is None:
                raise SystemExit(f'{dataset}: no base vectors under {data_root}')
        print('[{}] dataset: {}, d_model: {}'.format(
            algorithm, dataset, self.storage.size(-1)))

    def target(self, k):
        if k not in self.targets:
            self.targets[k] = utils.brute_force_topk(
                self.queries, self.storage, k).cpu()
        return self.targets[k]

    def load_query(self, k):
        if self.loader is not None:
            return self.loader.load_query(self.n_queries, k=k)
        pick = torch.randperm(QUERY_POOL, generator=self.draw)[:self.n_queries]
        return self.queries[pick.to(self.queries.device)].cpu(), self.target(k)[pick]

    def build(self, method, n_neighbors):
        self.method = method
        if self.index is not None:
            return          # both methods search the same index
        prefix = {'hnsw': 'nsw', 'nsg': 'nsg'}[self.algorithm]
        index = layers.IndexStaged(
            d_model=self.storage.size(-1), d_principle=self.d_principle,
            sample_ratio=self.sample_ratio, entry_method=self.entry_method,
            graph_method=f'{prefix}{n_neighbors}', seed=self.seed,
            build_device=self.device)
        index.train(self.storage)
        index.to(self.device)
        self.index = index

    def load(self, checkpoint):
        self.index = layers.IndexStaged.load(checkpoint)
        self.index.to(self.device)

    def dump(self, checkpoint):
        torch.save(self.index.dump(), checkpoint)

    def search_pilot(self, query, k, ef_search):
        before = time.perf_counter()
        out = self.index.search(query, k=k, ef_search=ef_search,
                                chunk_size=CHUNK_SIZE, refine=self.refine,
                                traversal=self.traversal)[0].cpu()
        return out, time.perf_counter() - before

    def search_host(self, query, k, ef_search):
        before = time.perf_counter()
        out = self.index.search_cpu(query, k=k, ef_search=ef_search)[0]
        return out, time.perf_counter() - before

    def run(self, k, ef_search, n_repeats=20):
        timings, recalls = [], []
        for _ in range(n_repeats + N_WARMUP):
            query, target = self.load_query(k)
            if self.method == 'search-pilot':
                indices, duration = self.search_pilot(query, k, ef_search)
            else:
                indices, duration = self.search_host(query, k, ef_search)
            recalls.append(utils.recall(indices, target=target))
            timings.append(1000.0 * duration)
        recalls, timings = recalls[N_WARMUP:], timings[N_WARMUP:]
        return sum(recalls) / len(recalls), sum(timings) / len(timings)


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__.split('\n\n')[0])
    parser.add_argument('--top_k', type=int, default=10)
    parser.add_argument('--d_principle', type=int, default=128)
    parser.add_argument('--sample_ratio', type=float, default=0.25)
    parser.add_argument('--n_neighbors', type=int, default=64)
    parser.add_argument('--ef_search', type=lambda s: [int(v) for v in s.split(',')],
                        default=[16, 32, 48, 64, 96, 128, 192, 256])
    parser.add_argument('--n_queries', type=int, default=1024)
    parser.add_argument('--algorithm', type=str, default='hnsw',
                        choices=['hnsw', 'nsg'])
    parser.add_argument('--router', type=str, default='router64x64')
    parser.add_argument('--dataset', type=str,
                        default='synth:1000000x768:1024:0')
    parser.add_argument('--data_root', default='.dataset',
                        help="directory of the reference's dataset folders")
    parser.add_argument('--refine', choices=['host', 'device'], default='host',
                        help="where stages 2 and 3 run (the reference: host)")
    parser.add_argument('--traversal', choices=['exact', 'wide'], default='exact',
                        help="'wide': the labelled throughput mode of the "
                        "device stage (several nodes per step; other candidates "
                        "than the host kernel's, --refine device only)")
    parser.add_argument('--methods', type=lambda s: s.split(','),
                        default=['search-pilot', 'host-cpu'])
    parser.add_argument('--n_repeats', type=int, default=20)
    parser.add_argument('--device', default='cuda:0')
    parser.add_argument('--load', default=None, help='checkpoint to search '
                        '(IndexStaged.dump format) instead of building')
    parser.add_argument('--dump', default=None, help='write the built index')
    args = parser.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit('pilotann_amd.cli: no GPU')
    if args.traversal == 'wide' and args.refine != 'device':
        raise SystemExit('pilotann_amd.cli: --traversal wide needs --refine device')

    profiler = Profiler(dataset=args.dataset, algorithm=args.algorithm,
                        entry_method=args.router,
                        sample_ratio=args.sample_ratio,
                        d_principle=args.d_principle, n_queries=args.n_queries,
                        device=args.device, refine=args.refine,
                        data_root=args.data_root, traversal=args.traversal)
    if args.load:
        profiler.load(args.load)
    records = {method: [] for method in args.methods}
    for method in records:
        profiler.build(method=method, n_neighbors=args.n_neighbors)
        if args.dump:
            profiler.dump(args.dump)
        for ef_search in args.ef_search:
            recall, timing = profiler.run(k=args.top_k, ef_search=ef_search,
                                          n_repeats=args.n_repeats)
            print('{}: recall={:.3f}, duration={:.3f}ms'.format(
                method, recall, timing), flush=True)
            records[method].append({
                'recall': recall, 'timing': timing,
                'n_neighbors': args.n_neighbors, 'ef_search': ef_search})
    for method in records:
        for record in records[method]:
            print(method, record)
    return records


if __name__ == '__main__':
    main()
