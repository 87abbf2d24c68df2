"""Datasets by name, as ``pilot_ann/utils/loader.py`` hands them to the
reference's tests and benchmark scripts: ``DataLoader(name)`` with
``.load_storage()``, ``.load_query(n_queries, k)``, ``.d_model`` and
``.n_storage``.

Names and file layouts are the reference's (``loader.py:92-207``):

* ``fuzz-16k`` / ``fuzz-64k`` — uniform rows in [-1, 1), a random length
  around 16 384 / 65 536 and a random width out of {64, 96, 128, 200, 512,
  768}, 4096 queries, exact top-100 as ground truth (``loader.py:9-40``);
* ``deep-*`` / ``text2img-*`` (``64k``, ``1m``, ``10m``, ``100m``) — the
  big-ann-benchmarks binary layout under ``<root>/<family>-<1m|10m|100m>/``:
  ``base.fbin``, ``query.fbin`` (two int32 ``rows, columns`` then float32
  rows) and ``groundtruth.ibin`` (the same with int32 ids);
* ``wiki-*`` / ``laion-*`` — ``query.npy``, ``groundtruth.npy`` and the base
  vectors as every other ``*.npy`` of the directory, in sorted order.

A base file that holds more rows than the name asks for is cut down to a
random subset and the ground truth is recomputed by brute force
(``loader.py:78-89``).  What differs from the reference: files are memory
mapped, not read whole (only the rows that are used leave the disk); the
subset is drawn without repeats, so no row is in the index twice; every draw
takes a seed; the brute force runs on ``device`` when one is given.
"""
import math
import os

import numpy as np
import torch

N_QUERIES = 4096          # loader.py:10
TARGET_K = 100            # loader.py:37,56
FUZZ_WIDTHS = (64, 96, 128, 200, 512, 768)


def read_bins(filename: str, dtype) -> np.ndarray:
    """Memory map of a ``.fbin`` / ``.ibin`` file: int32 ``rows``, int32
    ``columns``, then ``rows x columns`` items of ``dtype`` (4 bytes each)."""
    dtype = np.dtype(dtype)
    if dtype.itemsize != 4:
        raise ValueError('fbin / ibin items are 4 bytes wide')
    head = np.fromfile(filename, dtype=np.int32, count=2)
    if head.size != 2 or head[0] < 0 or head[1] <= 0:
        raise ValueError(f'{filename}: no (rows, columns) header')
    rows, cols = int(head[0]), int(head[1])
    if os.path.getsize(filename) < 8 + 4 * rows * cols:
        raise ValueError(f'{filename}: shorter than its header says')
    return np.memmap(filename, dtype=dtype, mode='r', offset=8, shape=(rows, cols))


def write_bins(filename: str, array) -> None:
    """The inverse of :func:`read_bins` (float32 or int32 rows)."""
    array = np.ascontiguousarray(array)
    if array.ndim != 2 or array.dtype.itemsize != 4:
        raise ValueError('a 2-d array of 4-byte items is expected')
    with open(filename, 'wb') as f:
        np.asarray(array.shape, dtype=np.int32).tofile(f)
        array.tofile(f)


def search_target(query: torch.Tensor, storage: torch.Tensor,
                  top_k: int = TARGET_K, chunk_size: int = 1024,
                  device=None) -> torch.Tensor:
    """Exact ``top_k`` nearest rows (L2) of every query, ids ascending by
    distance (``loader.py:53-75``); ``storage`` is walked in pieces that fit
    the device."""
    device = torch.device(device) if device is not None else query.device
    top_k = min(top_k, storage.size(0))
    out = torch.empty(query.size(0), top_k, dtype=torch.long)
    piece = max(top_k, min(storage.size(0), (1 << 28) // max(chunk_size, 1)))
    for lo in range(0, query.size(0), chunk_size):
        q = query[lo:lo + chunk_size].to(device, torch.float32)
        qq = q.square().sum(-1, keepdim=True)
        best_d = torch.full((q.size(0), 0), 0.0, device=device)
        best_i = torch.zeros((q.size(0), 0), dtype=torch.long, device=device)
        for base in range(0, storage.size(0), piece):
            x = storage[base:base + piece].to(device, torch.float32)
            d = qq - 2.0 * (q @ x.T) + x.square().sum(-1).unsqueeze(0)
            ids = torch.arange(base, base + x.size(0), device=device)
            best_d = torch.cat([best_d, d], dim=1)
            best_i = torch.cat([best_i, ids.expand(q.size(0), -1)], dim=1)
            if best_d.size(1) > top_k:
                top = torch.topk(best_d, top_k, dim=-1, largest=False, sorted=True)
                best_d, best_i = top.values, torch.gather(best_i, 1, top.indices)
        order = torch.argsort(best_d, dim=-1, stable=True)
        out[lo:lo + chunk_size] = torch.gather(best_i, 1, order).cpu()
    return out


def _rows(array, index: torch.Tensor) -> torch.Tensor:
    """Rows ``index`` (ascending) of a memory map or tensor as a float32
    tensor in memory."""
    if isinstance(array, torch.Tensor):
        return array[index].float().contiguous()
    return torch.from_numpy(np.ascontiguousarray(array[index.numpy()], dtype=np.float32))


def shrink_dataset(query, storage, n_targets: int, generator=None, device=None):
    """``n_targets`` random rows of ``storage`` (ascending, no repeats) and
    the ground truth of ``query`` on them (``loader.py:78-89``)."""
    n = storage.shape[0]
    pick = torch.randperm(n, generator=generator)[:n_targets].sort().values
    kept = _rows(storage, pick)
    return kept, search_target(query, kept, device=device)


class _Concatenated:
    """Row-wise view of several memory maps of equal width."""

    def __init__(self, parts):
        self.parts = parts
        self.starts = np.cumsum([0] + [p.shape[0] for p in parts])
        self.shape = (int(self.starts[-1]), parts[0].shape[1])

    def __getitem__(self, index):
        index = np.asarray(index)
        out = np.empty((index.size, self.shape[1]), dtype=np.float32)
        which = np.searchsorted(self.starts, index, side='right') - 1
        for p, part in enumerate(self.parts):
            sel = np.nonzero(which == p)[0]
            if sel.size:
                out[sel] = part[index[sel] - self.starts[p]]
        return out


_SIZES = {'64k': 65536, '1m': 1_000_000, '10m': 10_000_000, '100m': 100_000_000}
# loader.py:151-167: the numpy families keep up to 999 rows more
_NUMPY_SIZES = {'64k': 65536, '1m': 1_000_999, '100m': 100_000_999}


def _split(name: str):
    family, _, size = name.partition('-')
    return family, size


def load_fuzz(name: str, generator=None, device=None):
    family, size = _split(name)
    if family != 'fuzz' or size not in ('16k', '64k'):
        raise NotImplementedError(name)
    around = 16384 if size == '16k' else 65536
    d_model = FUZZ_WIDTHS[int(torch.randint(len(FUZZ_WIDTHS), (1,), generator=generator))]
    n_storage = int(torch.randint(around // 2, 2 * around + 1, (1,), generator=generator))
    query = 2.0 * (torch.rand(N_QUERIES, d_model, generator=generator) - 0.5)
    storage = 2.0 * (torch.rand(n_storage, d_model, generator=generator) - 0.5)
    return query, storage, search_target(query, storage, device=device)


def load_bins(name: str, root: str, generator=None, device=None):
    family, size = _split(name)
    if family not in ('deep', 'text2img') or size not in _SIZES:
        raise NotImplementedError(name)
    folder = os.path.join(root, f'{family}-{"1m" if size == "64k" else size}')
    query = torch.from_numpy(np.array(read_bins(os.path.join(folder, 'query.fbin'), np.float32)))
    target = torch.from_numpy(
        np.array(read_bins(os.path.join(folder, 'groundtruth.ibin'), np.int32))).long()
    base = os.path.join(folder, 'base.fbin')
    if not os.path.exists(base):
        return query, None, target       # loader.py:137-138: queries only
    storage = read_bins(base, np.float32)
    if storage.shape[0] > _SIZES[size]:
        storage, target = shrink_dataset(query, storage, _SIZES[size], generator, device)
    else:
        storage = torch.from_numpy(np.array(storage))
    return query, storage, target


def load_numpy(name: str, root: str, generator=None, device=None):
    family, size = _split(name)
    if family not in ('wiki', 'laion') or size not in _NUMPY_SIZES:
        raise NotImplementedError(name)
    folder = os.path.join(root, f'{family}-{"1m" if size == "64k" else size}')
    query = torch.from_numpy(np.load(os.path.join(folder, 'query.npy'))).float()
    target = torch.from_numpy(np.load(os.path.join(folder, 'groundtruth.npy'))).long()
    shards = sorted(f for f in os.listdir(folder)
                    if f.endswith('.npy') and f not in ('query.npy', 'groundtruth.npy'))
    if not shards:
        return query, None, target
    parts = [np.load(os.path.join(folder, f), mmap_mode='r') for f in shards]
    storage = _Concatenated(parts)
    if storage.shape[0] > _NUMPY_SIZES[size]:
        storage, target = shrink_dataset(query, storage, _NUMPY_SIZES[size], generator, device)
    else:
        storage = torch.from_numpy(storage[np.arange(storage.shape[0])])
    return query, storage, target


class DataLoader:
    """``utils.DataLoader`` of the reference (``loader.py:210-249``).
    ``root`` is the directory of the datasets (the reference's ``.dataset``),
    ``seed`` fixes every random draw, ``device`` is where a ground truth is
    recomputed when a base file is cut down."""

    def __init__(self, name: str, root: str = '.dataset', seed: int = None,
                 device=None):
        self.generator = torch.Generator()
        if seed is None:
            self.generator.seed()
        else:
            self.generator.manual_seed(seed)
        family = _split(name)[0]
        if family == 'fuzz':
            output = load_fuzz(name, self.generator, device)
        elif family in ('deep', 'text2img'):
            output = load_bins(name, root, self.generator, device)
        elif family in ('wiki', 'laion'):
            output = load_numpy(name, root, self.generator, device)
        else:
            raise NotImplementedError(name)
        self.query, self.storage, self.target = output

    @property
    def d_model(self) -> int:
        return self.query.size(-1)

    @property
    def n_storage(self) -> int:
        return self.storage.size(0)

    def load_storage(self) -> torch.Tensor:
        return self.storage

    def load_query(self, n_queries: int, k: int):
        """``n_queries`` queries drawn with repeats, and the first ``k``
        columns of their ground truth (``loader.py:238-249``)."""
        if k > self.target.size(-1):
            raise RuntimeError(f'the ground truth holds {self.target.size(-1)} ids per query')
        pick = torch.randint(len(self.query), (n_queries,), generator=self.generator)
        return self.query[pick], self.target[pick][:, :k]
