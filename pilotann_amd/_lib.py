"""ctypes binding of ``csrc/libpilotann.so`` (declared in include/pilotann.h).

There is no fallback: if the library has not been built, or a call returns an
error, a ``RuntimeError`` is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'csrc', 'libpilotann.so')

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_sz = ctypes.c_size_t

_SIGNATURES = {
    'pa_error_string': (ctypes.c_char_p, [_int]),
    'pa_heap_size': (_int, [_int]),
    'pa_graph_prepare': (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp,
                                _vp, _vp, _vp]),
    'pa_traverse_plan': (_int, [_i64, _i64, _int, _int,
                                ctypes.POINTER(_int), ctypes.POINTER(_sz)]),
    'pa_traverse': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                           _i64, _i64, _i64, _int, _int, _int, _int, _int,
                           _vp, _sz, _vp, _vp]),
    'pa_traverse_static': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                  _i64, _i64, _i64, _int, _int, _int, _int,
                                  _int, _vp, _vp]),
    'pa_traverse_wide_plan': (_int, [_i64, _i64, _int, _int,
                                     ctypes.POINTER(_int), ctypes.POINTER(_sz)]),
    'pa_traverse_wide': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                _i64, _i64, _i64, _int, _int, _int, _int, _int,
                                _int, _vp, _sz, _vp, _vp]),
    'pa_route': (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _int,
                        _vp, _vp, _vp]),
    'pa_rotate': (_int, [_vp, _vp, _vp, _i64, _int, _int, _vp]),
    'pa_traverse_cpu': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                               _i64, _i64, _int, _int, _int, _int]),
    'pa_traverse_refine': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                  _vp, _vp, _vp, _vp, _i64, _i64, _int, _int,
                                  _int, _int, _int, _int]),
    'pa_knn_list_capacity': (_i64, [_int]),
    'pa_knn_tile_rows': (_int, []),
    'pa_knn_rerank': (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    'pa_knn': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _int, _vp]),
    'pa_graph_prune': (_int, [_vp, _vp, _vp, _i64, _int, _int, _int, _vp]),
    'pa_graph_prune_rows': (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int,
                            _int, _int, ctypes.c_float, _vp]),
    'pa_heapq_pop': (_int, [_vp, _vp, _i64]),
    'pa_heapq_pushpop': (_int, [_vp, _vp, _i64, ctypes.c_float, _i64]),
    'pa_heapq_replace': (_int, [_vp, _vp, _i64, ctypes.c_float, _i64]),
    'pa_bitmask_put': (_int, [_vp, _i64, _vp, _i64]),
    'pa_square_dist': (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int]),
    'pa_rows_prepare': (_int, [_vp, _vp, _i64, _int, _vp]),
    'pa_refine_plan': (_int, [_i64, _i64, _int, _int,
                              ctypes.POINTER(_int), ctypes.POINTER(_sz)]),
    'pa_refine': (_int, [_vp] * 12 + [_i64, _i64] + [_int] * 8 +
                  [_vp, _sz, _vp, _vp]),
    'pa_pipeline': (_int, [_vp] * 15 + [_i64, _i64, _i64] + [_int] * 7 + [_vp]),
}

_lib = None


def lib():
    """The loaded library; raises if it is not there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f'{LIB_PATH} not found: the HIP extension has not been '
                'built (python -m pilotann_amd.build); there is no fallback')
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            try:
                fn = getattr(handle, name)
            except AttributeError:
                continue
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(code: int, what: str):
    if code != 0:
        text = lib().pa_error_string(code).decode()
        raise RuntimeError(f'{what}: {text} ({code})')
