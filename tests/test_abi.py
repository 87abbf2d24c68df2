"""The C ABI: every function include/pilotann.h declares is exported by the
built library with C linkage, and the cheap host-only entry points answer.
No device work here."""
import ctypes
import os
import re

from pilotann_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, 'include', 'pilotann.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(pa_[a-z_]+)\s*\(', text)))


def test_header_symbols_are_exported():
    names = declared_functions()
    assert {'pa_traverse', 'pa_route', 'pa_pipeline', 'pa_graph_prepare',
            'pa_traverse_plan', 'pa_traverse_cpu', 'pa_traverse_refine',
            'pa_heap_size', 'pa_error_string'} <= set(names)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert getattr(lib, name) is not None, name


def test_bindings_cover_the_header():
    assert set(_lib._SIGNATURES) == set(declared_functions())


def test_host_only_entry_points():
    lib = _lib.lib()
    assert [lib.pa_heap_size(e) for e in (1, 16, 17, 256, 257, 2048, 2049)] == \
        [16, 16, 32, 256, 384, 2048, -1]
    assert lib.pa_error_string(0) == b'ok'
    assert b'multiple of 8' in lib.pa_error_string(-3)
    # argument errors are detected on the host, before any device call
    assert lib.pa_route(None, None, None, None, None, 4, 8, 24, 64, None, None, None) == -8
    assert lib.pa_route(None, None, None, None, None, 4, 8, 32, 60, None, None, None) == -3
    assert lib.pa_route(None, None, None, None, None, 4, 8, 32, 64, None, None, None) == -1
    assert lib.pa_traverse_cpu(None, None, None, None, None, None, None, None,
                               4, 100, 60, 8, 10, 16) == -3
    assert lib.pa_pipeline(*([None] * 15), 100, 1000, 250, 64, 32, 32, 32, 16,
                           10, 30, None) == -9
    # the wide mode: width 1..4, ids of 30 bits, then the pointers
    wide = [None] * 9
    assert lib.pa_traverse_wide(*wide, 4, 1000, 500, 64, 8, 4, 8, 16, 5, None, 0,
                                None, None) == -2
    assert lib.pa_traverse_wide(*wide, 4, (1 << 30) + 1, 500, 64, 8, 4, 8, 16, 4,
                                None, 0, None, None) == -10
    assert lib.pa_traverse_wide(*wide, 4, 1000, 500, 60, 8, 4, 8, 16, 4, None, 0,
                                None, None) == -3
    assert lib.pa_traverse_wide_plan(500, 4, 64, 4096, None, None) == -5
    assert lib.pa_rotate(None, None, None, 4, 60, 8, None) == -3
    assert lib.pa_rotate(None, None, None, 4, 64, 65, None) == -2
    assert lib.pa_rotate(None, None, None, 4, 64, 8, None) == -1
    assert lib.pa_rotate(None, None, None, 0, 64, 8, None) == 0
    # pa_graph_prepare: sizes first (indices of a negative length), then the
    # pointers; the content of indptr is checked on the device
    assert lib.pa_graph_prepare(None, None, None, 100, 50, -1, 32, None, None,
                                None, None) == -2
    assert lib.pa_graph_prepare(None, None, None, 100, 50, 1600, 32, None,
                                None, None, None) == -1


def test_device_refine_argument_errors_on_the_host():
    """pa_rows_prepare / pa_refine reject bad sizes before any device call;
    the Python wrappers refuse host tensors and plain rows."""
    import pytest
    import torch
    from pilotann_amd import kernels
    lib = _lib.lib()
    assert lib.pa_rows_prepare(None, None, 10, 60, None) == -3
    assert lib.pa_rows_prepare(None, None, -1, 64, None) == -2
    assert lib.pa_rows_prepare(None, None, 0, 64, None) == 0
    assert lib.pa_rows_prepare(None, None, 10, 64, None) == -1
    def refine(batch=4, n_nodes=100, d=64, dp=32, n_init=8, n_buf=8, k=5, ef=16,
               sub_deg=32, full_deg=32):
        return lib.pa_refine(*([None] * 12), batch, n_nodes, d, dp, n_init, n_buf,
                             k, ef, sub_deg, full_deg, None, 0, None, None)
    assert refine(batch=-1) == -2
    assert refine(n_nodes=1 << 31) == -10
    assert refine(sub_deg=0) == -4
    assert refine(full_deg=65) == -4
    assert refine(dp=12) == -3
    assert refine(dp=72) == -3
    x = torch.zeros(4, 64)
    with pytest.raises(RuntimeError):
        kernels.PreparedRows(x)
    ids, dist = torch.zeros(4, 8, dtype=torch.long), torch.zeros(4, 8)
    with pytest.raises(RuntimeError):
        kernels.traverse_refine_cuda(ids, dist, ids, dist, ids, dist, None, None,
                                     x, x, 16, 32)
