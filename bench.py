"""Benchmark of the GPU search stage (entry router + subgraph traversal) on
one MI355X, on seeded synthetic data in the shape of the headline
configuration: 1M x 768 fp32 unit-norm vectors from a 1024-component mixture,
SVD to d_principle = 128, sample_ratio 0.25, a 64-neighbour base-layer graph
(HNSW M = 32 shape), router64x64, 10k queries, top-10.

A step = one pass of the hot path over the 10k-query batch: `routing_cuda`
then `traverse_cuda`, inputs resident in HBM, at the smallest ef of the sweep
whose end-to-end recall@10 (after the host refine) reaches 0.90.  One JSON
line is printed; `value` is queries per second of that step.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--n-base N] [--queries B] [--ef EF] [--no-cpu-baseline]
                    [--no-context] [--copy-calibration]
"""
import argparse
import contextlib
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
    # the configuration the metric is quoted on
    'c3': dict(n=1_000_000, d=768, dp=128, n_centers=1024, sigma=1.0,
               decay=0.5, normalize=True, ratio=0.25, graph='nsw64',
               entry='router64x64', queries=10_000, k=10,
               ef_sweep=[4, 8, 16, 24, 32, 48, 64], seed=301),
    # large result lists: top-100, ef 256 / 512 (heaps of 1024 / 2048 entries)
    'c4': dict(n=1_000_000, d=768, dp=128, n_centers=1024, sigma=1.0,
               decay=0.5, normalize=True, ratio=0.5, graph='nsw64',
               entry='router64x64', queries=10_000, k=100,
               ef_sweep=[256, 512], seed=301),
    # the smaller 96-dimensional configuration
    'c2': dict(n=1_000_000, d=96, dp=64, n_centers=256, sigma=1.0,
               decay=0.5, normalize=False, ratio=0.25, graph='nsw32',
               entry='router32x32', queries=10_000, k=10,
               ef_sweep=[8, 16, 32, 64, 128], seed=201),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_index(cfg, device):
    from pilotann_amd import IndexStaged, utils
    t0 = time.time()
    x = utils.gaussian_mixture(
        cfg['n'], cfg['d'], cfg['n_centers'], cfg['sigma'], seed=cfg['seed'],
        normalize=cfg['normalize'], device=device, decay=cfg['decay'])
    q = utils.gaussian_mixture(
        cfg['queries'], cfg['d'], cfg['n_centers'], cfg['sigma'],
        seed=cfg['seed'] + 1, normalize=cfg['normalize'], device=device,
        decay=cfg['decay'], center_seed=cfg['seed'])
    target = utils.brute_force_topk(q, x, cfg['k']).cpu()
    log(f'[bench] data + ground truth {time.time() - t0:.1f}s')
    index = IndexStaged(d_model=cfg['d'], d_principle=cfg['dp'],
                        sample_ratio=cfg['ratio'], graph_method=cfg['graph'],
                        entry_method=cfg['entry'], seed=cfg['seed'],
                        build_device=device)
    with contextlib.redirect_stdout(sys.stderr):  # keep stdout to the JSON line
        index.train(x)
    del x
    torch.cuda.empty_cache()
    index.to(device)
    log(f'[bench] index built {time.time() - t0:.1f}s, '
        f'sampled {index.nodelist.numel()} of {cfg["n"]}')
    return index, q.cpu(), target


class Stage:
    """The timed hot path: router then traversal, device resident."""

    def __init__(self, index, query, device):
        from pilotann_amd import kernels
        self.kernels = kernels
        self.index = index
        self.device = device
        self.query_rot = torch.matmul(query, index.VT.T).contiguous()
        self.query_cuda = self.query_rot[:, :index.d_principle].contiguous().to(device)
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

    def traverse(self, ef, EP_I, EP_D, counters=None):
        out_I, out_D = self.buffers(ef)
        self.kernels.traverse_prepared(
            out_I, out_D, self.graph, self.index.storage_cuda,
            self.query_cuda, EP_I, EP_D, counters)
        return out_I, out_D

    def step(self, ef):
        EP_I, EP_D = self.entries()
        return self.traverse(ef, EP_I, EP_D)


def end_to_end_recall(index, stage, ef, target, k):
    """Recall of the whole three-stage search at this ef: device candidates,
    then the host refine on the full-dimension vectors."""
    from pilotann_amd import kernels, utils
    out_I, out_D = stage.step(ef)
    torch.cuda.synchronize()
    buf_I = out_I.flatten(1).cpu()
    buf_D = out_D.flatten(1).cpu()
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


def measured_traffic(key):
    """HBM bytes per launch from the rocprofv3 counter runs summarised under
    profiles/ (FETCH_SIZE and WRITE_SIZE, each scaled by what a plain copy of
    known size reads on the same counter), or None for a workload that has
    not been profiled."""
    path = os.path.join(ROOT, 'profiles', 'traffic.json')
    try:
        with open(path) as f:
            return json.load(f).get(key, {}).get('hbm_bytes_per_launch')
    except OSError:
        return None


def cpu_baseline(index, stage, ef, EP_I, EP_D, budget_s=12.0):
    """The host search of the reference (restated in oracle/) on the same
    subgraph, reduced rows and entries, timed on this box's cores on a sample
    of the batch sized for about `budget_s` seconds."""
    import oracle
    dp = index.d_principle
    reduced = np.ascontiguousarray(index.storage[:, :dp].numpy())
    q = np.ascontiguousarray(stage.query_rot[:, :dp].numpy())
    indptr = index.subgraph.indptr.numpy()
    indices = index.subgraph.indices.numpy()
    kk = 4 * ef
    I = EP_I.cpu().numpy()
    D = EP_D.cpu().numpy()

    def run(n):
        out_I = np.empty((n, kk), np.int64)
        out_D = np.empty((n, kk), np.float32)
        t0 = time.perf_counter()
        oracle.traverse_cpu(out_I, out_D, I[:n].copy(), D[:n].copy(), indptr,
                            indices, reduced, q[:n].copy(), kk)
        return time.perf_counter() - t0, out_I, out_D

    run(min(stage.B, 512))  # warm-up: thread pool, page faults
    # whole passes over the batch until the time budget is used
    total_t, total_n, passes = 0.0, 0, 0
    out_I = out_D = None
    while total_t < budget_s and passes < 1000:
        t, out_I, out_D = run(stage.B)
        total_t += t
        total_n += stage.B
        passes += 1
    return dict(value=total_n / total_t, unit='queries/s',
                cores=oracle.num_threads(), kind='port',
                sample=f'{passes} passes over the same {stage.B}-query batch '
                       f'(same subgraph / reduced rows / entries, '
                       f'ef_search={kk}), {total_t:.1f}s of host search'), \
        (out_I, out_D, stage.B)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--config', default='c3', choices=sorted(CONFIGS))
    ap.add_argument('--n-base', type=int, default=None)
    ap.add_argument('--queries', type=int, default=None)
    ap.add_argument('--ef', type=int, default=None)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-context', action='store_true',
                    help='skip the context figures (PCIe-inclusive step, '
                         'fourfold batch, end-to-end search), so that a '
                         'kernel trace of the run holds the timed launches '
                         'only')
    ap.add_argument('--device-refine-only', action='store_true',
                    help='only measure the search with the refine on the '
                         'device and the refine kernel alone (needs --ef), '
                         'print those figures and exit; with --no-context '
                         'the refine kernel alone (4 launches)')
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

    cfg = dict(CONFIGS[args.config], name=args.config)
    if args.n_base:
        cfg['n'] = args.n_base
    if args.queries:
        cfg['queries'] = args.queries
    device = 'cuda:0'
    torch.cuda.set_device(0)
    index, query, target = build_index(cfg, device)
    stage = Stage(index, query, device)
    B, k, dp = stage.B, cfg['k'], cfg['dp']

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
    for ef in ([args.ef] if args.ef else cfg['ef_sweep']):
        rec, refine_s = end_to_end_recall(index, stage, ef, target, k)
        sweep.append(dict(ef=ef, recall=round(rec, 4),
                          refine_qps=round(B / refine_s, 1)))
        log(f'[bench] ef={ef} recall@{k}={rec:.4f} host refine {refine_s:.2f}s')
        if rec >= 0.90:
            chosen = ef
            break
    if chosen is None:
        chosen = sweep[-1]['ef']
    ef = chosen
    recall_at = [s for s in sweep if s['ef'] == ef][0]['recall']

    # work counters of one launch (untimed), then the timed steps
    EP_I, EP_D = stage.entries()
    counters = torch.zeros(5, dtype=torch.long, device=device)
    out_I, out_D = stage.traverse(ef, EP_I, EP_D, counters)
    torch.cuda.synchronize()
    counts = counters.cpu().tolist()
    launch_bytes = algorithmic_bytes(counts, B, dp, EP_I.size(1))

    for _ in range(args.warmup):
        stage.step(ef)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True),
           torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for a, b in ev:
        EP_I, EP_D = stage.entries()
        a.record()
        stage.traverse(ef, EP_I, EP_D)
        b.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    kernel_ms = float(np.mean([a.elapsed_time(b) for a, b in ev]))
    achieved = launch_bytes / (kernel_ms * 1e-3) / 1e9

    line = {
        'metric': METRIC,
        'value': round(B / (ms_per_step * 1e-3), 1),
        'unit': 'queries/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {
            'workload': f'{args.config}: {cfg["n"]} x {cfg["d"]} '
                        f'{"unit-norm " if cfg["normalize"] else ""}'
                        f'{cfg["n_centers"]}-component mixture, dp={dp}, '
                        f'sample_ratio={cfg["ratio"]}, {cfg["graph"]}, '
                        f'{cfg["entry"]}, {B} queries, top-{k}',
            'ef': ef, 'k': k, 'recall_at_k': recall_at, 'sweep': sweep,
            'stage': 'routing_cuda + traverse_cuda (GPU search stage)',
        },
        'roofline': {
            'bound': 'hbm', 'achieved': round(achieved, 1),
            'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
            'frac': round(achieved / HBM_PEAK_GBS, 4),
            'traffic': measured_traffic(
                f'{args.config}/n={cfg["n"]}/queries={B}/ef={ef}'),
            'kernel': 'traverse_kernel',
            'kernel_ms': round(kernel_ms, 4),
            'algorithmic_bytes_per_launch': launch_bytes,
            'counters': dict(zip(['expanded', 'adjacency_entries',
                                  'distances', 'admitted', 'result_slots'],
                                 counts)),
        },
    }
    if not args.no_context:
        context_figures(line, args, cfg, index, stage, query, target, ef,
                        launch_bytes, out_D)

    if not args.no_cpu_baseline:
        EP_I, EP_D = stage.entries()
        torch.cuda.synchronize()
        base, (ref_I, ref_D, n) = cpu_baseline(index, stage, ef, EP_I, EP_D)
        line['cpu_baseline'] = base
        same = (np.array_equal(out_D.flatten(1)[:n].cpu().numpy(), ref_D))
        line['config']['matches_cpu_baseline'] = bool(same)
    print(json.dumps(line), flush=True)


def context_figures(line, args, cfg, index, stage, query, target, ef,
                    launch_bytes, out_D):
    """Not part of `value`: the same step with its inputs and outputs
    crossing PCIe (pageable host memory), the launch over a fourfold batch,
    and the whole three-stage search (`IndexStaged.search`: rotation on the
    host, entries, pipeline)."""
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
    # keeps 5120 independent searches in flight; filling and draining them
    # weighs less on a longer batch, which shows the kernel's marginal rate.
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
        'refine_hbm_traffic': measured_traffic(
            f'{cfg["name"]}/n={cfg["n"]}/queries={B}/ef={ef}/refine'),
        'refine_achieved_GBps': round(nbytes / (ms * 1e-3) / 1e9, 1),
        'refine_frac_of_hbm_peak': round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}


if __name__ == '__main__':
    main()
