"""Compiles the HIP/C++ sources under ``csrc/`` into ``csrc/libpilotann.so``
for gfx950.  Run as ``python -m pilotann_amd.build``; the library stays in the
source tree, where the ctypes loader looks for it."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, 'csrc')
LIB = os.path.join(CSRC, 'libpilotann.so')
# tuning build whose traversal kernel tallies cycles per phase of a search
# (``python -m pilotann_amd.build --phase-timers``; ``bench.py --phase-split``
# loads it); not built by default and never the library the package loads
PHASE_LIB = os.path.join(CSRC, 'libpilotann_phase_timers.so')

HIP_SOURCES = ['traverse.hip', 'traverse_wide.hip', 'refine.hip', 'route.hip', 'rotate.hip',
               'knn.hip', 'pipeline.hip']
CXX_SOURCES = ['host_search.cpp']

HIP_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC',
    '-ffp-contract=off',
    # packed fp32 instructions off (device pass; the host pass warns that it
    # does not know the feature, which is harmless)
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wno-unused-command-line-argument', '-Wno-inline-asm',
]
# the reference's host flags (setup.py:39-44) minus -ffast-math: the host
# search must add in the order it is written
CXX_FLAGS = [
    '-O3', '-std=c++17', '-fPIC', '-mavx2', '-mfma', '-fopenmp',
    '-funroll-loops', '-ffp-contract=off', '-fno-fast-math',
]


def _run(cmd, verbose):
    if verbose:
        print(' '.join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build(verbose: bool = False, output: str = LIB,
          extra_hip_flags=()) -> str:
    """Compile everything and link ``output`` (default: the library the
    loader uses).  ``extra_hip_flags`` are added to the device compiles, e.g.
    ``-DPA_PHASE_TIMERS`` for the tuning build ``PHASE_LIB``."""
    include = os.path.join(ROOT, 'include')
    objects = []
    for name in HIP_SOURCES:
        src = os.path.join(CSRC, name)
        if not os.path.exists(src):
            continue
        obj = os.path.join(CSRC, name + '.o')
        _run(['hipcc', *HIP_FLAGS, *extra_hip_flags, '-I', include, '-c', src,
              '-o', obj], verbose)
        objects.append(obj)
    for name in CXX_SOURCES:
        src = os.path.join(CSRC, name)
        if not os.path.exists(src):
            continue
        obj = os.path.join(CSRC, name + '.o')
        _run(['g++', *CXX_FLAGS, '-I', include, '-c', src, '-o', obj], verbose)
        objects.append(obj)
    _run(['hipcc', '--offload-arch=gfx950', '-shared', '-fPIC', '-o', output,
          *objects, '-lgomp', '-lpthread'], verbose)
    for obj in objects:
        os.remove(obj)
    return output


if __name__ == '__main__':
    if '--phase-timers' in sys.argv:
        print(build(verbose='-q' not in sys.argv, output=PHASE_LIB,
                    extra_hip_flags=['-DPA_PHASE_TIMERS']))
    else:
        print(build(verbose='-q' not in sys.argv))
