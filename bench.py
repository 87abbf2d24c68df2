"""Benchmark of the GPU search stage (entry router + subgraph traversal) on
one MI355X, on seeded synthetic data in the shape of the headline
configuration: 1M x 768 fp32 unit-norm vectors from a 1024-component mixture,
SVD to d_principle = 128, sample_ratio 0.25, a 64-neighbour base-layer graph
(HNSW M = 32 shape), router64x64, 10k queries, top-10.

A step = one pass of the hot path over the 10k-query batch: `routing_cuda`
then `traverse_cuda`, inputs resident in HBM, at the smallest ef of the sweep
whose end-to-end recall@10 (after the host refine) reaches 0.90.  One JSON
line is printed; `value` is queries per second of that step.

`value` is the rate of the GPU search stage alone (what this build replaces);
the rates of the whole search at the same recall, with the refine on the host
and on the device, are the top-level fields `end_to_end_qps_host_refine` and
`end_to_end_qps_device_refine`.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1..c5]
                    [--n-base N] [--queries B] [--ef EF] [--decay X] [--curve]
                    [--no-cpu-baseline] [--no-context] [--power-law-twin]
                    [--copy-calibration]
"""
import argparse
import contextlib
import hashlib
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = 'QPS @ recall@10>=0.90 (1M x 768 fp32, 1 GPU); traversal HBM GB/s'
HBM_PEAK_GBS = 8000.0

CONFIGS = {
    # the plumbing case: isotropic mixture as written, NSG rows, fixed random
    # entries, 1024 queries at ef = 64
    'c1': dict(n=100_000, d=96, dp=32, n_centers=64, sigma=0.3, decay=0.0,
               normalize=False, ratio=0.25, graph='nsg32', entry='random32',
               queries=1024, k=10, ef_sweep=[64], seed=101),
    # the configuration the metric is quoted on: the mixture as it is worded
    # (every coordinate with the same variance, then normalised), the ef range
    # that is named for it
    'c3': dict(n=1_000_000, d=768, dp=128, n_centers=1024, sigma=1.0,
               decay=0.0, normalize=True, ratio=0.25, graph='nsw64',
               entry='router64x64', queries=10_000, k=10,
               ef_sweep=[32, 48, 64, 96, 128, 192, 256], seed=301,
               curve=[8, 16, 24, 32, 64, 128, 256]),
    # large result lists: top-100, ef 256 / 512 (heaps of 1024 / 2048 entries)
    'c4': dict(n=1_000_000, d=768, dp=128, n_centers=1024, sigma=1.0,
               decay=0.0, normalize=True, ratio=0.5, graph='nsw64',
               entry='router64x64', queries=10_000, k=100,
               ef_sweep=[256, 512], seed=301),
    # the smaller 96-dimensional configuration
    'c2': dict(n=1_000_000, d=96, dp=64, n_centers=256, sigma=1.0,
               decay=0.0, normalize=False, ratio=0.25, graph='nsw32',
               entry='router32x32', queries=10_000, k=10,
               ef_sweep=[32, 64, 128], seed=201),
    # the memory-bounded case: 10M x 768, 2.5M reduced rows and their graph
    # on the device.  By default only the device stage is built, in under a
    # minute: the subgraph on a seeded random quarter of the nodes and no
    # full graph, hence no refine and no end-to-end recall (the recall
    # reported is that of the candidate lists); --full-index builds the whole
    # index (four minutes) and measures the whole search.
    'c5': dict(n=10_000_000, d=768, dp=128, n_centers=4096, sigma=1.0,
               decay=0.0, normalize=True, ratio=0.25, graph='nsg48',
               entry='router64x64', queries=10_000, k=10, ef_sweep=[128],
               seed=501, stage_only=True, device_rng=True),
}
# every ef of a configuration that is timed besides the chosen one
ALSO_TIMED = {'c4': [256, 512], 'c3': [16, 24]}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


TRAVERSAL_SOURCES = ('traverse.hip', 'search_lists.h', 'device_common.h')
WIDE_SOURCES = ('traverse_wide.hip', 'search_lists.h', 'device_common.h')


def kernel_sources_sha16(names=TRAVERSAL_SOURCES):
    """Hash of the sources a kernel is compiled from (default: the traversal
    kernel's); the counter figures in profiles/traffic.json carry the hash
    they were measured with."""
    h = hashlib.sha256()
    for name in names:
        h.update(name.encode())
        with open(os.path.join(ROOT, 'pilotann_amd', 'csrc', name), 'rb') as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def make_data(cfg, device):
    from pilotann_amd import utils
    kw = dict(normalize=cfg['normalize'], device=device, decay=cfg['decay'],
              device_rng=cfg.get('device_rng', False))
    x = utils.gaussian_mixture(cfg['n'], cfg['d'], cfg['n_centers'],
                               cfg['sigma'], seed=cfg['seed'], **kw)
    q = utils.gaussian_mixture(cfg['queries'], cfg['d'], cfg['n_centers'],
                               cfg['sigma'], seed=cfg['seed'] + 1,
                               center_seed=cfg['seed'], **kw)
    chunk = max(64, min(1024, (1 << 31) // cfg['n']))
    target = utils.brute_force_topk(q, x, cfg['k'], chunk=chunk).cpu()
    return x, q, target


def cache_key(cfg):
    """What of a configuration decides the content of a stage cache."""
    return {k: v for k, v in cfg.items() if k not in ('name', 'index_build_seconds')}


def save_stage_cache(path, cfg, index, q, target):
    """What the device stage of a `stage_only` configuration needs, so that a
    counter run does not pay for the index build again: rotation, sample,
    subgraph, router, queries, ground truth and the sampled rows' first
    d_principle coordinates."""
    torch.save({
        'config': cache_key(cfg),
        'VT': index.VT, 'nodelist': index.nodelist, 'mapping': index.mapping,
        'subgraph.indptr': index.subgraph.indptr,
        'subgraph.indices': index.subgraph.indices,
        'entry': index.entry.state_dict(),
        'rows': index.storage[index.nodelist][:, :cfg['dp']].contiguous(),
        'query': q, 'target': target,
    }, path)


def load_stage_cache(path, cfg, device):
    from pilotann_amd import IndexStaged
    from pilotann_amd.layers.staged import GraphModule
    saved = torch.load(path, weights_only=True)
    if saved['config'] != cache_key(cfg):
        raise SystemExit(f'{path} was written for another configuration')
    index = IndexStaged(d_model=cfg['d'], d_principle=cfg['dp'],
                        sample_ratio=cfg['ratio'], graph_method=cfg['graph'],
                        entry_method=cfg['entry'], seed=cfg['seed'],
                        build_device=device)
    for name in ['VT', 'nodelist', 'mapping']:
        index.register_buffer(name, saved[name])
    index.register_module('subgraph', GraphModule(
        saved['subgraph.indptr'], saved['subgraph.indices']))
    for name, value in saved['entry'].items():
        index.entry.register_buffer(name, value)
    # the rows the stage reads, at their global positions; the others (and the
    # coordinates past d_principle) are never looked at by the device stage
    storage = torch.zeros(cfg['n'], cfg['dp'])
    storage[saved['nodelist']] = saved['rows']
    index.register_buffer('storage', storage)
    index.fullgraph = None
    index.to(device)
    return index, saved['query'], saved['target']


def build_index(cfg, device, stage_cache=None):
    from pilotann_amd import IndexStaged
    if stage_cache and os.path.exists(stage_cache):
        t0 = time.time()
        out = load_stage_cache(stage_cache, cfg, device)
        log(f'[bench] index read from {stage_cache} {time.time() - t0:.1f}s')
        return out
    t0 = time.time()
    x, q, target = make_data(cfg, device)
    log(f'[bench] data + ground truth {time.time() - t0:.1f}s')
    index = IndexStaged(d_model=cfg['d'], d_principle=cfg['dp'],
                        sample_ratio=cfg['ratio'], graph_method=cfg['graph'],
                        entry_method=cfg['entry'], seed=cfg['seed'],
                        build_device=device)
    with contextlib.redirect_stdout(sys.stderr):  # keep stdout to the JSON line
        if cfg.get('stage_only'):
            train_stage_only(index, x, cfg)
        else:
            index.train(x)
    del x
    torch.cuda.empty_cache()
    index.to(device)
    cfg['index_build_seconds'] = round(time.time() - t0, 1)
    log(f'[bench] index built {time.time() - t0:.1f}s, '
        f'sampled {index.nodelist.numel()} of {cfg["n"]}')
    if stage_cache:
        save_stage_cache(stage_cache, cfg, index, q.cpu(), target)
        log(f'[bench] stage inputs written to {stage_cache}')
    return index, q.cpu(), target


def train_stage_only(index, x, cfg):
    """What the device stage needs of `IndexStaged.train`, for a base set whose
    full graph is out of reach of a benchmark run: rotation, a seeded random
    sample of the nodes, the subgraph on the sample, the entry router."""
    from pilotann_amd import utils
    from pilotann_amd.layers.staged import GraphModule
    n = x.size(0)
    print('svd', index.d_principle)
    xr, V = utils.svd(x, max_size=10_000_000, seed=index.seed)
    index.register_buffer('VT', V.T.contiguous().cpu())
    g = torch.Generator().manual_seed(index.seed + 1)
    nodelist = torch.randperm(n, generator=g)[:round(index.sample_ratio * n)]
    nodelist = nodelist.sort().values
    mapping = torch.full((n,), -1, dtype=torch.long)
    mapping[nodelist] = torch.arange(nodelist.numel())
    print('build', index.graph_type, 'on', nodelist.numel(), 'sampled nodes')
    sub = xr[nodelist.to(xr.device)]
    sg_indptr, sg_indices = utils.graph_init(
        sub, index.graph_type, index.n_neighbors, compute_dtype=torch.float16,
        seed=index.seed + 1)
    del sub
    glob_ids = torch.where(sg_indices >= 0, nodelist[sg_indices.clamp(min=0)],
                           torch.full_like(sg_indices, -1))
    rowlen = torch.zeros(n, dtype=torch.long)
    rowlen[nodelist] = sg_indptr[1:] - sg_indptr[:-1]
    indptr = torch.zeros(n + 1, dtype=torch.long)
    indptr[1:] = torch.cumsum(rowlen, 0)
    index.register_module('subgraph', GraphModule(indptr, glob_ids))
    index.register_buffer('nodelist', nodelist.contiguous())
    index.register_buffer('mapping', mapping.contiguous())
    index.register_buffer('storage', xr.cpu().contiguous())
    del xr
    index.fullgraph = None
    index.entry.train(index.storage[:, :index.d_principle])


class Stage:
    """The timed hot path: router then traversal, device resident."""

    def __init__(self, index, query, device):
        from pilotann_amd import kernels
        self.kernels = kernels
        self.index = index
        self.device = device
        # rotated on the device, as IndexStaged.search does (kernels.rotate)
        rotated = kernels.rotate(query.to(device).contiguous(), index.VT_cuda)
        self.query_rot = rotated.cpu()
        self.query_cuda = rotated[:, :index.d_principle].contiguous()
        self.graph = kernels.prepare_graph(
            index.subgraph_cuda.indptr, index.subgraph_cuda.indices,
            index.mapping_cuda, index.storage_cuda.size(0), index.n_neighbors)
        self.B = query.size(0)
        self.out = {}

    def buffers(self, ef):
        if ef not in self.out:
            self.out[ef] = (
                torch.empty(self.B, 4, ef, dtype=torch.long, device=self.device),
                torch.empty(self.B, 4, ef, dtype=torch.float, device=self.device))
        return self.out[ef]

    def entries(self):
        EP_I, EP_D = self.index.entry.search(self.query_cuda)
        return EP_I.contiguous(), EP_D.contiguous()

    def traverse(self, ef, EP_I, EP_D, counters=None, wide=0):
        """`wide` = 0: the exact mode; 1..4: the wide mode of that width."""
        out_I, out_D = self.buffers(ef)
        if wide:
            self.kernels.traverse_wide_prepared(
                out_I, out_D, self.graph, self.index.storage_cuda,
                self.query_cuda, EP_I, EP_D, counters, wide)
        else:
            self.kernels.traverse_prepared(
                out_I, out_D, self.graph, self.index.storage_cuda,
                self.query_cuda, EP_I, EP_D, counters)
        return out_I, out_D

    def step(self, ef, wide=0):
        EP_I, EP_D = self.entries()
        return self.traverse(ef, EP_I, EP_D, wide=wide)


def end_to_end_recall(index, stage, ef, target, k, wide=0):
    """Recall of the whole three-stage search at this ef: device candidates,
    then the host refine on the full-dimension vectors.  Without a full
    graph (stage-only index): the recall of the candidate lists themselves."""
    from pilotann_amd import kernels, utils
    out_I, out_D = stage.step(ef, wide)
    torch.cuda.synchronize()
    buf_I = out_I.flatten(1).cpu()
    buf_D = out_D.flatten(1).cpu()
    if index.fullgraph is None:
        # share of the true nearest neighbours found among the candidates
        hit = (buf_I.unsqueeze(-1) == target.unsqueeze(1)).any(1)
        return float(hit.float().mean()), float('nan')
    top_I = torch.empty(stage.B, k, dtype=torch.long)
    top_D = torch.empty(stage.B, k, dtype=torch.float)
    t0 = time.perf_counter()
    kernels.traverse_refine(
        top_I, top_D, buf_I, buf_D, buf_I, buf_D,
        [index.subgraph.indptr, index.subgraph.indices],
        [index.fullgraph.indptr, index.fullgraph.indices],
        index.storage, stage.query_rot, ef, index.d_principle)
    refine_s = time.perf_counter() - t0
    return utils.recall(top_I, target), refine_s


def algorithmic_bytes(counters, B, dp, n_init):
    """Bytes a search must move, per launch: 4-byte ids, 4-byte floats.
    query + entries + per expansion (pop id, row pointer) + adjacency entries
    + per evaluated neighbour (id + dp floats) + results written."""
    E, A, C, _, R = [int(c) for c in counters]
    w = 4
    return (B * (4 * dp + n_init * (w + 4)) + E * 2 * w + A * w
            + C * (w + 4 * dp) + R * (w + 4))


def traffic_key(cfg, B, ef):
    """Name of a measured workload in profiles/traffic.json."""
    return (f'{cfg["name"]}/n={cfg["n"]}/queries={B}/ef={ef}'
            f'/spectrum_exponent={cfg["decay"]}')


def measured_traffic(key, sources=TRAVERSAL_SOURCES):
    """Bytes per launch that left the L2 towards the fabric, from the
    rocprofv3 counter runs summarised under profiles/ (FETCH_SIZE and
    WRITE_SIZE, each scaled by what a plain copy of known size reads on the
    same counter), and whether the kernel sources are still the ones those
    runs were made with; (None, None) for a workload that has not been
    profiled."""
    path = os.path.join(ROOT, 'profiles', 'traffic.json')
    try:
        with open(path) as f:
            entry = json.load(f).get(key)
    except OSError:
        entry = None
    if not entry:
        return None, None
    return (entry.get('hbm_bytes_per_launch'),
            entry.get('kernel_sources_sha16') == kernel_sources_sha16(sources))


def time_stage(stage, ef, steps, warmup, wide=0):
    """Work counters of one launch (untimed), then `steps` timed passes of
    router + traversal; the traversal alone is bracketed by events on the
    launch stream."""
    device = stage.device
    EP_I, EP_D = stage.entries()
    counters = torch.zeros(5, dtype=torch.long, device=device)
    out_I, out_D = stage.traverse(ef, EP_I, EP_D, counters, wide)
    torch.cuda.synchronize()
    counts = counters.cpu().tolist()
    launch_bytes = algorithmic_bytes(counts, stage.B, stage.index.d_principle,
                                     EP_I.size(1))
    for _ in range(warmup):
        stage.step(ef, wide)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True),
           torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in ev:
        EP_I, EP_D = stage.entries()
        a.record()
        stage.traverse(ef, EP_I, EP_D, wide=wide)
        b.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / steps
    kernel_ms = float(np.mean([a.elapsed_time(b) for a, b in ev]))
    achieved = launch_bytes / (kernel_ms * 1e-3) / 1e9
    return dict(ef=ef, ms_per_step=ms_per_step, kernel_ms=kernel_ms,
                counts=counts, launch_bytes=launch_bytes, achieved=achieved,
                out_I=out_I, out_D=out_D)


def compare_search(I_a, D_a, I_b, D_b):
    """Two result sets of the same searches: are the distances identical bit
    for bit, and in how many rows do the ids differ anywhere but inside a run
    of equal distances (where only the set has to agree)?"""
    same_d = bool(np.array_equal(D_a, D_b))
    rows = np.flatnonzero((I_a != I_b).any(-1))
    outside_ties = 0
    for r in rows:
        if not np.array_equal(D_a[r], D_b[r]):
            outside_ties += 1
            continue
        for dist in np.unique(D_a[r][I_a[r] != I_b[r]]):
            sel = D_a[r] == dist
            if sorted(I_a[r][sel]) != sorted(I_b[r][sel]):
                outside_ties += 1
                break
    # ids that differ where the two distances differ as well: never allowed
    wrong = int(((I_a != I_b) & (D_a != D_b)).any(-1).sum()) if not same_d else 0
    out = dict(distances_identical=same_d,
               rows_with_other_order_inside_ties=int(len(rows) - outside_ties),
               rows_with_another_member_of_a_tie=int(outside_ties - wrong),
               rows_with_id_mismatch=wrong)
    if outside_ties and same_d:
        # a row in which one of several candidates at exactly the same
        # distance was kept by one search and another by the other
        for r in rows:
            pos = np.flatnonzero(I_a[r] != I_b[r])
            sel = np.isin(D_a[r], D_a[r][pos])
            if sorted(I_a[r][sel]) != sorted(I_b[r][sel]):
                out['example'] = dict(
                    row=int(r), positions=pos[:4].tolist(),
                    ids_a=I_a[r][pos[:4]].tolist(), ids_b=I_b[r][pos[:4]].tolist(),
                    distances=[float(x) for x in D_a[r][pos[:4]]])
                break
    return out


def cpu_baseline(index, stage, ef, EP_I, EP_D, budget_s=8.0):
    """The host search of the reference on the same subgraph, reduced rows and
    entries, timed on this box's cores on whole passes over the batch for
    about `budget_s` seconds each: the plain-C restatement in oracle/ and the
    library's own host search (`pa_traverse_cpu`: AVX2, four rows per
    distance call, prefetches, as traverse_cpu.cpp:92-135 has them).  The
    faster one is reported; both return the same results."""
    import oracle
    from pilotann_amd import kernels
    dp = index.d_principle
    reduced_t = index.storage[:, :dp].contiguous()
    reduced = reduced_t.numpy()
    q_t = stage.query_rot[:, :dp].contiguous()
    q = q_t.numpy()
    indptr_t, indices_t = index.subgraph.indptr, index.subgraph.indices
    indptr, indices = indptr_t.numpy(), indices_t.numpy()
    kk = 4 * ef
    I_t, D_t = EP_I.cpu(), EP_D.cpu()
    I, D = I_t.numpy(), D_t.numpy()
    B = stage.B

    def run_port(n):
        out_I = np.empty((n, kk), np.int64)
        out_D = np.empty((n, kk), np.float32)
        t0 = time.perf_counter()
        oracle.traverse_cpu(out_I, out_D, I[:n].copy(), D[:n].copy(), indptr,
                            indices, reduced, q[:n].copy(), kk)
        return time.perf_counter() - t0, out_I, out_D

    def run_avx2(n):
        out_I = torch.empty(n, kk, dtype=torch.long)
        out_D = torch.empty(n, kk, dtype=torch.float)
        i, d, qq = I_t[:n].clone(), D_t[:n].clone(), q_t[:n].clone()
        t0 = time.perf_counter()
        kernels.traverse_cpu(out_I, out_D, i, d, indptr_t, indices_t,
                             reduced_t, qq, kk)
        return time.perf_counter() - t0, out_I.numpy(), out_D.numpy()

    figures = {}
    results = {}
    for name, run in (('plain_c_port', run_port), ('avx2_host_search', run_avx2)):
        run(min(B, 512))  # warm-up: thread pool, page faults
        total_t, total_n, passes = 0.0, 0, 0
        while total_t < budget_s and passes < 1000:
            t, out_I, out_D = run(B)
            total_t += t
            total_n += B
            passes += 1
        figures[name] = dict(queries_per_s=round(total_n / total_t, 1),
                             passes=passes, seconds=round(total_t, 1))
        results[name] = (out_I, out_D)
    best = max(figures, key=lambda n: figures[n]['queries_per_s'])
    same = compare_search(*results['plain_c_port'], *results['avx2_host_search'])
    base = dict(value=figures[best]['queries_per_s'], unit='queries/s',
                cores=oracle.num_threads(), kind='port',
                implementation=best,
                sample=f'{figures[best]["passes"]} passes over the same {B}-query '
                       f'batch (same subgraph / reduced rows / entries, '
                       f'ef_search={kk}), {figures[best]["seconds"]}s of host search',
                both=figures, both_agree=same['distances_identical']
                and same['rows_with_id_mismatch'] == 0
                and same['rows_with_another_member_of_a_tie'] == 0)
    return base, results['plain_c_port']


def cpu_full_graph_baseline(index, query, stage, target, k, budget_s=6.0):
    """The search without a GPU (`IndexStaged.search_cpu`: rotation, the
    router's entries with full-dimension distances and the host search on the
    full graph in full dimension, all inside the timed region), at the
    smallest ef_search whose recall@k reaches 0.90 on a 2000-query sample —
    the role faiss' HNSW plays in the reference's own table
    (README.md:527-534)."""
    import oracle
    from pilotann_amd import utils
    if index.fullgraph is None:
        return None

    def run(n, ef_search):
        t0 = time.perf_counter()
        out_I, _ = index.search_cpu(query[:n], k=k, ef_search=ef_search)
        return time.perf_counter() - t0, out_I

    n_sample = min(2000, stage.B)
    sweep, chosen = [], None
    for ef_search in [e for e in (16, 24, 32, 48, 64, 96, 128, 192, 256, 384,
                                  512, 1024) if e >= k]:
        t, out_I = run(n_sample, ef_search)
        rec = utils.recall(out_I, target[:n_sample])
        sweep.append(dict(ef_search=ef_search, recall=round(rec, 4)))
        log(f'[bench] host search alone: ef_search={ef_search} recall@{k}={rec:.4f} '
            f'({n_sample} queries in {t:.2f}s)')
        if rec >= 0.90:
            chosen = ef_search
            break
    if chosen is None:
        chosen = sweep[-1]['ef_search']
    total_t, total_n, passes, rec = 0.0, 0, 0, None
    while total_t < budget_s and passes < 100:
        t, out_I = run(stage.B, chosen)
        rec = utils.recall(out_I, target)
        total_t += t
        total_n += stage.B
        passes += 1
    return dict(what='IndexStaged.search_cpu: rotation, router entries and '
                     'traverse_cpu (library host search, AVX2) on the full '
                     'graph in full dimension',
                ef_search=chosen, recall_at_k=round(rec, 4),
                queries_per_s=round(total_n / total_t, 1),
                cores=oracle.num_threads(), passes=passes, sweep=sweep)


def stage_record(t, B, key, kernel='traverse_kernel'):
    traffic, fresh = measured_traffic(key + ('/wide' if kernel == 'wide_kernel' else ''),
                                      WIDE_SOURCES if kernel == 'wide_kernel' else TRAVERSAL_SOURCES)
    rec = {
        'bound': 'hbm', 'achieved': round(t['achieved'], 1),
        'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
        'frac': round(t['achieved'] / HBM_PEAK_GBS, 4),
        'traffic': traffic,
        'kernel': kernel,
        'kernel_ms': round(t['kernel_ms'], 4),
        'algorithmic_bytes_per_launch': t['launch_bytes'],
        'counters': dict(zip(['expanded', 'adjacency_entries', 'distances',
                              'admitted', 'result_slots'], t['counts'])),
    }
    if traffic is not None:
        # the figure is a constant of a profiled run, not measured here
        rec['traffic_kernel_sources_unchanged'] = bool(fresh)
    return rec


PHASES = ['pop', 'adjacency_and_visited_marks_issued', 'visited_marks_waited_for',
          'rows_and_distances', 'inserts', 'per_query_set_up', 'per_query_results']


def phase_split(stage, ef):
    """Cycles per phase of the searches of one launch, from the tuning build
    whose kernel reads the cycle counter at every phase boundary after waiting
    for what the phase has outstanding: a phase's figure includes its memory
    waits, and that build overlaps less than the shipped one (its duration is
    reported beside the split, to compare)."""
    EP_I, EP_D = stage.entries()
    for _ in range(3):
        counters = torch.zeros(12, dtype=torch.long, device=stage.device)
        torch.cuda.synchronize()
        started = time.perf_counter()
        stage.traverse(ef, EP_I, EP_D, counters)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
    c = counters.cpu().tolist()
    cycles = c[5:12]
    total = max(sum(cycles), 1)
    return {
        'phase_split': 'traverse_kernel built with -DPA_PHASE_TIMERS',
        'ef': ef, 'queries': stage.B,
        'launch_ms_of_the_timed_build': round(elapsed * 1e3, 3),
        'expansions': c[0], 'distances': c[2], 'admitted': c[3],
        'share_of_wavefront_cycles': {n: round(v / total, 4)
                                      for n, v in zip(PHASES, cycles)},
        'cycles_per_expansion': {n: round(v / max(c[0], 1), 1)
                                 for n, v in zip(PHASES, cycles)},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--config', default='c3', choices=sorted(CONFIGS))
    ap.add_argument('--n-base', type=int, default=None)
    ap.add_argument('--queries', type=int, default=None)
    ap.add_argument('--ef', type=int, default=None)
    ap.add_argument('--decay', type=float, default=None,
                    help='exponent of the power-law spectrum of the synthetic '
                         'data (0, the default: the isotropic mixture the '
                         'configurations are worded with)')
    ap.add_argument('--curve', action='store_true',
                    help='time the stage at every ef of the sweep (no early '
                         'stop) and report recall and rate for each')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-context', action='store_true',
                    help='skip the context figures (PCIe-inclusive step, '
                         'fourfold batch, end-to-end search, isotropic data), '
                         'so that a kernel trace of the run holds the timed '
                         'launches only')
    ap.add_argument('--device-refine-only', action='store_true',
                    help='only measure the search with the refine on the '
                         'device and the refine kernel alone (needs --ef), '
                         'print those figures and exit; with --no-context '
                         'the refine kernel alone (4 launches)')
    ap.add_argument('--stage-cache', default=None, metavar='FILE',
                    help='configurations that build the device stage only '
                         '(c5): write the stage\'s inputs to FILE after the '
                         'build, or read them from FILE if it exists (for '
                         'counter runs, which slow the build down)')
    ap.add_argument('--full-index', action='store_true',
                    help='configurations that build the device stage only '
                         '(c5): build the whole index instead (full graph of '
                         'all nodes, the reference\'s sampler, host and device '
                         'refine), which takes minutes')
    ap.add_argument('--knn-only', action='store_true',
                    help="only time the graph builder's nearest-neighbour "
                         "kernel (pa_knn) on the configuration's base set "
                         "against itself, print its rate and exit")
    ap.add_argument('--traversal', default='exact', choices=['exact', 'wide'],
                    help="'wide': sweep and time the labelled throughput mode "
                         "(pa_traverse_wide) instead of the exact traversal; the "
                         "line says so in config.traversal (for profiles of that "
                         "kernel; the default run reports it as config.wide_mode)")
    ap.add_argument('--power-law-twin', action='store_true',
                    help='also build the configuration on data with a '
                         'power-law spectrum (exponent 0.5) and measure recall '
                         'and rate over a range of ef there (a second index '
                         'build; context, not part of `value`)')
    ap.add_argument('--phase-split', action='store_true',
                    help='only report where the searches of one launch spend '
                         'their cycles (pop, adjacency and visited marks, rows, '
                         'inserts, ...), measured with the tuning build of '
                         '`python -m pilotann_amd.build --phase-timers` (needs '
                         '--ef), and exit')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='only run a plain 1 GiB device copy five times (to '
                         'scale the FETCH_SIZE / WRITE_SIZE counters) and exit')
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this build measures one GPU; the search shards by '
              'query batch with no exchange, run it with --gpus 1',
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print('bench.py: no GPU', file=sys.stderr)
        sys.exit(1)

    if args.copy_calibration:
        torch.cuda.set_device(0)
        src = torch.empty(1 << 28, dtype=torch.float32, device='cuda:0').normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({'copy_calibration': '5 copies of 1 GiB (read 1 GiB, '
                                              'write 1 GiB each)'}))
        return

    if args.knn_only:
        print(json.dumps(knn_figures(dict(CONFIGS[args.config], name=args.config),
                                     args, 'cuda:0')), flush=True)
        return

    if args.phase_split:
        from pilotann_amd import _lib, build
        if not args.ef:
            ap.error('--phase-split needs --ef')
        if not os.path.exists(build.PHASE_LIB):
            ap.error(f'{build.PHASE_LIB} not found: '
                     'python -m pilotann_amd.build --phase-timers')
        _lib.LIB_PATH = build.PHASE_LIB      # before the first library call

    cfg = dict(CONFIGS[args.config], name=args.config)
    if args.n_base:
        cfg['n'] = args.n_base
    if args.queries:
        cfg['queries'] = args.queries
    if args.decay is not None:
        cfg['decay'] = args.decay
    device = 'cuda:0'
    torch.cuda.set_device(0)
    if args.full_index:
        cfg['stage_only'] = False
        from pilotann_amd.utils import graphs
        started = time.time()
        graphs.progress = lambda text: log(f'[bench] {time.time() - started:6.1f}s {text}')
    if args.stage_cache and not cfg.get('stage_only'):
        ap.error('--stage-cache is for configurations that build the device '
                 'stage only')
    index, query, target = build_index(cfg, device, args.stage_cache)
    stage = Stage(index, query, device)
    B, k, dp = stage.B, cfg['k'], cfg['dp']

    if args.phase_split:
        print(json.dumps(phase_split(stage, args.ef)), flush=True)
        return

    if args.device_refine_only:
        if not args.ef:
            ap.error('--device-refine-only needs --ef')
        print(json.dumps(device_refine_figures(
            cfg, index, stage, query, target, args.ef,
            whole_search=not args.no_context)), flush=True)
        return

    # pick ef: smallest of the sweep with end-to-end recall@k >= 0.90
    sweep = []
    chosen = None
    efs = [args.ef] if args.ef else cfg['ef_sweep']
    if args.curve and not args.ef:
        efs = cfg.get('curve', efs)
    wide = 4 if args.traversal == 'wide' else 0
    for ef in efs:
        rec, refine_s = end_to_end_recall(index, stage, ef, target, k, wide)
        sweep.append(dict(ef=ef, recall=round(rec, 4),
                          refine_qps=round(B / refine_s, 1)
                          if refine_s == refine_s else None))
        log(f'[bench] ef={ef} recall@{k}={rec:.4f} host refine {refine_s:.2f}s')
        if rec >= 0.90 and chosen is None:
            chosen = ef
            if not args.curve:
                break
    if chosen is None:
        chosen = sweep[-1]['ef']
    ef = chosen
    recall_at = [s for s in sweep if s['ef'] == ef][0]['recall']

    t = time_stage(stage, ef, args.steps, args.warmup, wide)
    # copies: later measurements (other ef, the wide mode) reuse the buffers
    out_I, out_D = t['out_I'].clone(), t['out_D'].clone()
    launch_bytes, ms_per_step = t['launch_bytes'], t['ms_per_step']
    key = traffic_key(cfg, B, ef)

    line = {
        'metric': METRIC,
        'value': round(B / (ms_per_step * 1e-3), 1),
        'unit': 'queries/s',
        'value_is': 'rate of the GPU search stage (routing_cuda + '
                    'traverse_cuda) at the ef whose end-to-end recall is '
                    'recall_at_k; whole-search rates: end_to_end_qps_*',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {
            'workload': f'{args.config}: {cfg["n"]} x {cfg["d"]} '
                        f'{"unit-norm " if cfg["normalize"] else ""}'
                        f'{cfg["n_centers"]}-component mixture '
                        f'(sigma {cfg["sigma"]}, spectrum exponent '
                        f'{cfg["decay"]}), dp={dp}, '
                        f'sample_ratio={cfg["ratio"]}, {cfg["graph"]}, '
                        f'{cfg["entry"]}, {B} queries, top-{k}',
            'ef': ef, 'k': k, 'recall_at_k': recall_at, 'sweep': sweep,
            'recall_is': ('candidate lists of the device stage (no full '
                          'graph, no refine)' if index.fullgraph is None else
                          'whole search: device candidates, then host refine'),
            'stage': 'routing_cuda + traverse_cuda (GPU search stage)',
            'traversal': ('exact: traverse_cpu step for step' if not wide else
                          'wide: the labelled throughput mode, not the host '
                          'search step for step (not the headline figure)'),
            # data, ground truth and the index on the device, when built here
            'index_build_seconds': cfg.get('index_build_seconds'),
        },
        'roofline': stage_record(t, B, key, 'wide_kernel' if wide else 'traverse_kernel'),
    }
    others = [e for e in (efs if args.curve else
                          ALSO_TIMED.get(args.config, []))
              if e != ef and not args.ef]
    if others:
        recalls = {s['ef']: s['recall'] for s in sweep}
        line['config']['other_ef'] = []
        for e in others:
            if e not in recalls:
                recalls[e] = round(end_to_end_recall(index, stage, e, target, k, wide)[0], 4)
            o = time_stage(stage, e, max(3, args.steps // 2), 1, wide)
            rec = stage_record(o, B, traffic_key(cfg, B, e),
                               'wide_kernel' if wide else 'traverse_kernel')
            line['config']['other_ef'].append(dict(
                ef=e, recall_at_k=recalls[e],
                queries_per_s=round(B / (o['ms_per_step'] * 1e-3), 1),
                ms_per_step=round(o['ms_per_step'], 4), roofline=rec))
            log(f'[bench] ef={e}: {o["kernel_ms"]:.3f} ms, frac {rec["frac"]}')
    if not args.no_context and not wide:
        context_figures(line, args, cfg, index, stage, query, target, ef,
                        launch_bytes, out_D)

    if not args.no_cpu_baseline and not wide:
        EP_I, EP_D = stage.entries()
        torch.cuda.synchronize()
        base, (ref_I, ref_D) = cpu_baseline(index, stage, ef, EP_I, EP_D)
        line['cpu_baseline'] = base
        # the whole batch against the oracle: distances bit for bit, ids
        # except inside runs of equal distances
        line['config']['matches_cpu_baseline'] = compare_search(
            out_I.flatten(1).cpu().numpy(), out_D.flatten(1).cpu().numpy(),
            ref_I, ref_D)
        full = cpu_full_graph_baseline(index, query, stage, target, k)
        if full:
            line['cpu_baseline']['without_gpu'] = full
    print(json.dumps(line), flush=True)


def context_figures(line, args, cfg, index, stage, query, target, ef,
                    launch_bytes, out_D):
    """Not part of `value`: the same step with its inputs and outputs
    crossing PCIe (pageable host memory), the launch over a fourfold batch,
    the whole three-stage search (`IndexStaged.search`: rotation, entries,
    pipeline), the same steps with two batches in flight and, on request, the
    workload's twin with a power-law spectrum."""
    B, k, dp, device = stage.B, cfg['k'], cfg['dp'], stage.device
    host_q = stage.query_rot[:, :dp].contiguous()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        stage.query_cuda.copy_(host_q)
        oI, oD = stage.step(ef)
        oI.cpu(), oD.cpu()
    line['config']['ms_per_step_with_pcie'] = round(
        1e3 * (time.perf_counter() - t0) / 3, 3)
    # context: the same launch over four copies of the batch.  One launch
    # keeps thousands of independent searches in flight; filling and draining
    # them weighs less on a longer batch, which shows the kernel's marginal rate.
    rep = 4
    big_q = stage.query_cuda.repeat(rep, 1).contiguous()
    big_EI, big_ED = [t.repeat(rep, 1).contiguous() for t in stage.entries()]
    big_I = torch.empty(rep * B, 4, ef, dtype=torch.long, device=device)
    big_D = torch.empty(rep * B, 4, ef, dtype=torch.float, device=device)
    big_ev = []
    for i in range(4):
        a, b = (torch.cuda.Event(enable_timing=True) for _ in range(2))
        a.record()
        stage.kernels.traverse_prepared(big_I, big_D, stage.graph,
                                        index.storage_cuda, big_q, big_EI,
                                        big_ED, None)
        b.record()
        big_ev.append((a, b))
    torch.cuda.synchronize()
    big_ms = float(np.mean([a.elapsed_time(b) for a, b in big_ev[1:]]))
    big_rate = rep * launch_bytes / (big_ms * 1e-3) / 1e9
    line['config']['batch_x4'] = {
        'queries': rep * B, 'kernel_ms': round(big_ms, 4),
        'queries_per_s': round(rep * B / (big_ms * 1e-3), 1),
        'achieved_GBps': round(big_rate, 1),
        'frac': round(big_rate / HBM_PEAK_GBS, 4),
        'same_results': bool(torch.equal(big_D[-B:], out_D))}
    del big_q, big_EI, big_ED, big_I, big_D


    if index.fullgraph is not None:
        chunk = 1000 if B % 1000 == 0 else B
        index.search(query, k=k, ef_search=ef, chunk_size=chunk)
        t0 = time.perf_counter()
        top_I, top_D = index.search(query, k=k, ef_search=ef, chunk_size=chunk)
        t_e2e = time.perf_counter() - t0
        from pilotann_amd import utils as _utils
        line['config']['end_to_end'] = {
            'api': 'IndexStaged.search', 'chunk_size': chunk,
            'queries_per_s': round(B / t_e2e, 1),
            'recall_at_k': round(_utils.recall(top_I, target), 4)}
        line['config']['end_to_end_device_refine'] = device_refine_figures(
            cfg, index, stage, query, target, ef, (top_I, top_D))
        line['end_to_end_qps_host_refine'] = \
            line['config']['end_to_end']['queries_per_s']
        line['end_to_end_qps_device_refine'] = \
            line['config']['end_to_end_device_refine']['queries_per_s']

    # context: the same steps with two batches in flight, as a serving loop
    # keeps them: steps alternate between two streams (each with its own
    # outputs; the library keeps scratch memory per stream), so the searches of
    # one step fill the wavefront slots that the last searches of the step
    # before leave empty
    # (the index's own pair of streams where it has one: streams made later
    # can share a hardware queue, and work on one queue does not overlap)
    streams = getattr(index, '_streams', None) or \
        [torch.cuda.Stream(device=device) for _ in range(2)]
    outs = [(torch.empty(B, 4, ef, dtype=torch.long, device=device),
             torch.empty(B, 4, ef, dtype=torch.float, device=device)) for _ in range(2)]

    def alternate(count):
        for i in range(count):
            with torch.cuda.stream(streams[i % 2]):
                EP_I, EP_D = stage.entries()
                stage.kernels.traverse_prepared(
                    outs[i % 2][0], outs[i % 2][1], stage.graph, index.storage_cuda,
                    stage.query_cuda, EP_I, EP_D, None)
    torch.cuda.synchronize()
    alternate(4)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    alternate(args.steps)
    torch.cuda.synchronize()
    t_two = time.perf_counter() - t0
    line['config']['two_batches_in_flight'] = {
        'what': 'the timed steps alternating between two streams',
        'steps': args.steps, 'ms_per_step': round(1e3 * t_two / args.steps, 4),
        'queries_per_s': round(args.steps * B / t_two, 1),
        # algorithmic bytes of all steps over the whole time (launches
        # overlap: not a per-launch figure like roofline.achieved)
        'aggregate_GBps': round(args.steps * launch_bytes / t_two / 1e9, 1),
        'aggregate_frac': round(args.steps * launch_bytes / t_two / 1e9 / HBM_PEAK_GBS, 4),
        'same_results': bool(torch.equal(outs[0][1], out_D) and
                             torch.equal(outs[1][1], out_D))}
    del outs

    line['config']['wide_mode'] = wide_mode_figures(
        cfg, index, stage, target, ef, args, line['config']['recall_at_k'])

    if args.power_law_twin:
        line['config']['power_law_spectrum'] = spectrum_twin(cfg, device, args)


def wide_mode_figures(cfg, index, stage, target, ef, args, exact_recall):
    """The labelled throughput mode (`pa_traverse_wide`: several nodes
    expanded per step, result and open list one sorted pool) on the same
    step: rate, algorithmic bytes of its own work over its kernel time, and
    the recall of the whole search with its candidates beside the exact
    mode's.  Context: never `value`."""
    out = {'what': 'pa_traverse_wide, width 4: not the host search step for '
                   'step; distances of returned ids exact',
           'ef': ef}
    rec, _ = end_to_end_recall(index, stage, ef, target, cfg['k'], wide=4)
    t = time_stage(stage, ef, max(3, args.steps // 2), 1, wide=4)
    out.update(
        recall_at_k=round(rec, 4), exact_mode_recall_at_k=exact_recall,
        recall_delta=round(rec - exact_recall, 4),
        queries_per_s=round(stage.B / (t['ms_per_step'] * 1e-3), 1),
        ms_per_step=round(t['ms_per_step'], 4),
        kernel_ms=round(t['kernel_ms'], 4),
        algorithmic_bytes_per_launch=t['launch_bytes'],
        achieved_GBps=round(t['achieved'], 1),
        frac=round(t['achieved'] / HBM_PEAK_GBS, 4),
        counters=dict(zip(['expanded', 'adjacency_entries', 'distances',
                           'admitted', 'result_slots'], t['counts'])))
    traffic, fresh = measured_traffic(traffic_key(cfg, stage.B, ef) + '/wide',
                                      WIDE_SOURCES)
    if traffic is not None:
        out.update(traffic=traffic, traffic_kernel_sources_unchanged=bool(fresh))
    log(f'[bench] wide mode ef={ef}: {t["kernel_ms"]:.3f} ms, recall {rec:.4f} '
        f'(exact {exact_recall:.4f}), frac {out["frac"]}')
    return out


def knn_figures(cfg, args, device):
    """The nearest-neighbour kernel of the graph builder on the rotated base
    set against itself (what `graph_init` runs first): seconds per pass and
    the rate of its half-precision products against the dense fp16 MFMA
    peak."""
    from pilotann_amd import kernels, utils
    torch.cuda.set_device(0)
    if args.n_base:
        cfg['n'] = args.n_base
    x, _, _ = make_data(dict(cfg, queries=8), device)
    x, _ = utils.svd(x, max_size=10_000_000, seed=cfg['seed'])
    rows = kernels.HalfRows(x)
    n, d = x.shape
    times = []
    for _ in range(max(2, args.warmup)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cand = kernels.knn_candidates(rows, rows, 256)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    t0 = time.perf_counter()
    ids, _ = utils.knn_graph(x, 240)
    torch.cuda.synchronize()
    whole = time.perf_counter() - t0
    flops = 2.0 * n * n * rows.half.size(1)
    return {
        'kernel': 'knn_kernel<256>', 'rows': n, 'd': d,
        'seconds_per_pass': round(min(times), 3),
        'roofline': {'bound': 'mfma', 'achieved': round(flops / min(times) / 1e12, 1),
                     'peak': 2500.0, 'unit': 'TFLOP/s',
                     'frac': round(flops / min(times) / 2.5e15, 4)},
        'knn_graph_seconds': round(whole, 2),
        'what': 'kernels.knn_candidates(x, x, 256): the 256 closest rows of every '
                'row by fp16 products, as the graph builder asks for them; '
                'knn_graph adds the exact float32 ranking of those candidates '
                '(240 kept)',
    }


def spectrum_twin(cfg, device, args):
    """The same configuration on data whose variance falls off along the
    coordinates like a power law (exponent 0.5, the way embedding sets
    concentrate their variance in few directions), so that the 128 kept
    coordinates carry most of a distance: recall of the whole search and rate
    of the GPU stage over a range of ef."""
    twin = dict(cfg, decay=0.5)
    index, query, target = build_index(twin, device)
    stage = Stage(index, query, device)
    rows = []
    for ef in (4, 6, 8, 16, 32, 64):
        rec, _ = end_to_end_recall(index, stage, ef, target, twin['k'])
        t = time_stage(stage, ef, 5, 1)
        rows.append(dict(ef=ef, recall_at_k=round(rec, 4),
                         queries_per_s=round(stage.B / (t['ms_per_step'] * 1e-3), 1),
                         kernel_ms=round(t['kernel_ms'], 4),
                         frac=round(t['achieved'] / HBM_PEAK_GBS, 4)))
        log(f'[bench] power-law spectrum ef={ef} recall {rec:.4f} '
            f'{t["kernel_ms"]:.3f} ms frac {rows[-1]["frac"]}')
    del index, stage
    torch.cuda.empty_cache()
    return dict(what='same sizes, seeds and pipeline, spectrum exponent 0.5',
                sweep=rows)


def device_refine_figures(cfg, index, stage, query, target, ef, host_top=None,
                          whole_search=True):
    """The whole search with the refine on the device as well
    (`IndexStaged.search(..., refine='device')`: the full-dimension rows and
    the full graph resident in HBM, one launch per stage, top-k copied back),
    and the refine kernel alone on the traversal's candidates."""
    from pilotann_amd import utils as _utils
    B, k, dp, d, device = stage.B, cfg['k'], cfg['dp'], cfg['d'], stage.device
    kernels = stage.kernels
    index.stage_refine()
    agree = top_I = t_all = None
    if whole_search:
        # same rotated query as the host path: results must agree
        same_I, same_D = index.search(query, k=k, ef_search=ef, refine='device')
        agree = None
        if host_top is not None:
            agree = {
                'distances_identical': bool(torch.equal(same_D, host_top[1])),
                'rows_with_identical_ids': round(float(
                    (same_I == host_top[0]).all(-1).float().mean()), 4)}
        query_dev = query.to(device)
        for _ in range(3):      # the device idles during the host stages
            index.search(query_dev, k=k, ef_search=ef, refine='device')
        torch.cuda.synchronize()
        reps = 10
        t0 = time.perf_counter()
        for _ in range(reps):
            top_I, _ = index.search(query_dev, k=k, ef_search=ef, refine='device')
        t_all = (time.perf_counter() - t0) / reps

    # the refine kernel alone
    EP_I, EP_D = stage.entries()
    cand_I, cand_D = stage.traverse(ef, EP_I, EP_D)
    cand_I, cand_D = cand_I.flatten(1).clone(), cand_D.flatten(1).clone()
    sub = stage.graph
    full = kernels.prepare_full_graph(index.fullgraph_cuda.indptr,
                                      index.fullgraph_cuda.indices)
    q_full = stage.query_rot.to(device).contiguous()
    init_I, init_D = cand_I.clone(), cand_D.clone()
    buf_I, buf_D = torch.empty_like(cand_I), torch.empty_like(cand_D)
    out_I = torch.empty(B, k, dtype=torch.long, device=device)
    out_D = torch.empty(B, k, dtype=torch.float, device=device)
    counters = torch.zeros(6, dtype=torch.long, device=device)
    times = []
    for i in range(4):
        init_D.copy_(cand_D)
        a, b = (torch.cuda.Event(enable_timing=True) for _ in range(2))
        a.record()
        kernels.traverse_refine_cuda(
            out_I, out_D, buf_I, buf_D, init_I, init_D, sub, full,
            index.storage_full_cuda, q_full, ef, dp,
            counters=counters if i == 0 else None)
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b))
    ms = float(np.mean(times[1:]))
    c = dict(zip(['expanded_subgraph', 'expanded_full', 'distances',
                  'admitted', 'completed', 'adjacency_entries'],
                 counters.cpu().tolist()))
    n_cand = cand_I.size(1)
    refine_traffic = measured_traffic(
        traffic_key(cfg, B, ef) + '/refine',
        ('refine.hip', 'search_lists.h', 'device_common.h'))
    # query + candidates read + completed tails + adjacency ids + full rows
    # (4-byte id each) + buffer and top-k written
    nbytes = (B * 4 * d + B * n_cand * 8 + c['completed'] * 4 * (d - dp)
              + c['adjacency_entries'] * 4 + c['distances'] * (4 + 4 * d)
              + B * (n_cand + k) * 8)
    return {
        'api': "IndexStaged.search(refine='device')",
        'queries_per_s': round(B / t_all, 1) if whole_search else None,
        'recall_at_k': (round(_utils.recall(top_I, target), 4)
                        if whole_search else None),
        'against_host_refine': agree,
        'refine_kernel_ms': round(ms, 3),
        'refine_counters': c,
        'refine_algorithmic_bytes': int(nbytes),
        'refine_hbm_traffic': refine_traffic[0],
        'refine_traffic_kernel_sources_unchanged': refine_traffic[1],
        'refine_achieved_GBps': round(nbytes / (ms * 1e-3) / 1e9, 1),
        'refine_frac_of_hbm_peak': round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}


if __name__ == '__main__':
    main()
