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
    assert lib.pa_route(None, None, None, None, None, 4, 8, 24, 64, None) == -8
    assert lib.pa_route(None, None, None, None, None, 4, 8, 32, 60, None) == -3
    assert lib.pa_route(None, None, None, None, None, 4, 8, 32, 64, None) == -1
    assert lib.pa_traverse_cpu(None, None, None, None, None, None, None, None,
                               4, 100, 60, 8, 10, 16) == -3
    assert lib.pa_pipeline(*([None] * 15), 100, 1000, 250, 64, 32, 32, 32, 16,
                           10, 30, None) == -9
