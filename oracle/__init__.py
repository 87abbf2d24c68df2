"""ctypes front-end of the CPU oracle (``oracle.c``).

Test infrastructure only: imported by ``tests/``, by the smoke check and by
the benchmark's CPU-baseline leg, never by the package.  Arrays are numpy,
C-contiguous; ids int64, values float32, as in the reference's tensors
(``extension/inc/common.h:13-21``).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, 'liboracle.so')
N_COUNTERS = 5

_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)


def build(force: bool = False):
    """Compile ``liboracle.so`` next to this file (gcc, see Makefile)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(['make', '-s', '-C', _HERE, 'liboracle.so'], check=True)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.orc_square_dist.restype = ctypes.c_float
    return _lib


def _i64(a):
    assert a.dtype == np.int64 and a.flags['C_CONTIGUOUS']
    return a.ctypes.data_as(_i64p)


def _f32(a):
    assert a.dtype == np.float32 and a.flags['C_CONTIGUOUS']
    return a.ctypes.data_as(_f32p)


def heap_size(ef_search: int) -> int:
    return lib().orc_heap_size(int(ef_search))


def heap_pop(keys, values):
    k, v = ctypes.c_float(), ctypes.c_int64()
    lib().orc_heap_pop(_f32(keys), _i64(values), keys.size,
                       ctypes.byref(k), ctypes.byref(v))
    return k.value, v.value


def heap_pushpop(keys, values, key, value):
    lib().orc_heap_pushpop(_f32(keys), _i64(values), keys.size,
                           ctypes.c_float(key), ctypes.c_int64(value))


def heap_replace(keys, values, key, value):
    lib().orc_heap_replace(_f32(keys), _i64(values), keys.size,
                           ctypes.c_float(key), ctypes.c_int64(value))


def square_dist(query, storage, nodes):
    out = np.empty(nodes.size, np.float32)
    rc = lib().orc_square_dist_list(
        _f32(out), _f32(query), _f32(storage), _i64(nodes),
        ctypes.c_int64(nodes.size), storage.shape[1])
    if rc:
        raise RuntimeError('d_model must be a multiple of 8')
    return out


def traverse_cpu(output_I, output_D, initial_I, initial_D, indptr, indices,
                 storage, query, ef_search, counters=None):
    """Argument order of ``kernels.traverse_cpu``
    (pilot_ann/kernels/__init__.py:47-59); outputs written in place."""
    batch, d_model = query.shape
    assert storage.shape[1] == d_model
    assert output_I.shape == output_D.shape and output_I.shape[0] == batch
    assert initial_I.shape == initial_D.shape and initial_I.shape[0] == batch
    cptr = None
    if counters is not None:
        assert counters.size >= N_COUNTERS
        cptr = _i64(counters)
    rc = lib().orc_traverse_cpu(
        _i64(output_I), _f32(output_D), _i64(initial_I), _f32(initial_D),
        _i64(indptr), _i64(indices), _f32(storage), _f32(query),
        ctypes.c_int64(batch), ctypes.c_int64(storage.shape[0]),
        d_model, initial_I.shape[1], output_I.shape[1], int(ef_search), cptr)
    if rc:
        raise RuntimeError(f'oracle traverse_cpu: error {rc}')


def traverse_refine(output_I, output_D, buffer_I, buffer_D, initial_I,
                    initial_D, subgraph, fullgraph, storage, query,
                    ef_search, d_principle):
    """Argument order of ``kernels.traverse_refine``
    (pilot_ann/kernels/__init__.py:78-94)."""
    batch, d_model = query.shape
    rc = lib().orc_traverse_refine(
        _i64(output_I), _f32(output_D), _i64(buffer_I), _f32(buffer_D),
        _i64(initial_I), _f32(initial_D),
        _i64(subgraph[0]), _i64(subgraph[1]),
        _i64(fullgraph[0]), _i64(fullgraph[1]),
        _f32(storage), _f32(query), ctypes.c_int64(batch),
        ctypes.c_int64(storage.shape[0]), d_model, int(d_principle),
        initial_I.shape[1], buffer_I.shape[1], output_I.shape[1],
        int(ef_search))
    if rc:
        raise RuntimeError(f'oracle traverse_refine: error {rc}')


def route(query, route_vectors, entry_vectors):
    """``routing_cuda`` restated: (router[B] int64, distances[B, L] f32)."""
    batch, d = query.shape
    n_routers, n_leaves = entry_vectors.shape[:2]
    router = np.empty(batch, np.int64)
    dist = np.empty((batch, n_leaves), np.float32)
    rc = lib().orc_route(_i64(router), _f32(dist), _f32(query),
                         _f32(route_vectors), _f32(entry_vectors),
                         ctypes.c_int64(batch), n_routers, n_leaves, d)
    if rc:
        raise RuntimeError(f'oracle route: error {rc}')
    return router, dist


def traverse_wide(output_I, output_D, initial_I, initial_D, indptr, indices,
                  mapping, storage, query, width=4, counters=None):
    """The library's wide mode (``pa_traverse_wide``) restated: ``storage``
    rows by global id like :func:`traverse_cpu`, ``mapping`` global id →
    storage row (orders exact distance ties as the device does), outputs
    ``[B, k]`` written in place."""
    batch, d_model = query.shape
    assert storage.shape[1] == d_model and mapping.shape[0] == storage.shape[0]
    assert output_I.shape == output_D.shape and output_I.shape[0] == batch
    assert initial_I.shape == initial_D.shape and initial_I.shape[0] == batch
    cptr = None
    if counters is not None:
        assert counters.size >= N_COUNTERS
        cptr = _i64(counters)
    rc = lib().orc_traverse_wide(
        _i64(output_I), _f32(output_D), _i64(initial_I), _f32(initial_D),
        _i64(indptr), _i64(indices), _i64(mapping), _f32(storage), _f32(query),
        ctypes.c_int64(batch), ctypes.c_int64(storage.shape[0]), d_model,
        initial_I.shape[1], output_I.shape[1], int(width), cptr)
    if rc:
        raise RuntimeError(f'oracle traverse_wide: error {rc}')


def num_threads() -> int:
    return lib().orc_num_threads()
