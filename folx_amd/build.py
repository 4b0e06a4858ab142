"""Builds ``libfolx_hip.so`` (the C-ABI kernel library) for gfx950 with hipcc.

    python -m folx_amd.build

The library is written next to this package (``folx_amd/lib/``) so that it travels with
the source tree; nothing is installed outside of it.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIBDIR = os.path.join(HERE, 'lib')
LIBPATH = os.path.join(LIBDIR, 'libfolx_hip.so')

SOURCES = [
    'api.cpp',
    'elementwise.hip',
    'dense.hip',
    'dense_act.hip',
    'dense_act_wide.hip',
    'dot_two.hip',
    'pointwise.hip',
    'reduce.hip',
    'gather.hip',
    'slogdet.hip',
    'mhsa.hip',
    'mhsa_sparse.hip',
    'layernorm.hip',
    'linsolve.hip',
    'anysize.hip',
]

# Packed FP32 instructions are switched off for all device code (-packed-fp32-ops).
HIPCC_FLAGS = [
    '-O3',
    '--offload-arch=gfx950',
    '-fPIC',
    '-std=c++17',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wno-unused-command-line-argument',
]


def _hipcc() -> str:
    for cand in (os.environ.get('HIPCC'), '/opt/rocm/bin/hipcc', 'hipcc'):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return 'hipcc'


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError('command failed: ' + ' '.join(cmd))
    return res


def build(verbose: bool = True) -> str:
    """Compile every source and link the shared library.  Always recompiles."""
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, 'obj')
    os.makedirs(objdir, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(src):
        obj = os.path.join(objdir, os.path.splitext(src)[0] + '.o')
        cmd = [hipcc, *HIPCC_FLAGS, '-x', 'hip', '-c', os.path.join(CSRC, src), '-o', obj]
        _run(cmd)
        if verbose:
            print(f'[folx_amd.build] compiled {src}', flush=True)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    _run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIBPATH, *objs])
    if verbose:
        print(f'[folx_amd.build] linked {LIBPATH}', flush=True)
    return LIBPATH


if __name__ == '__main__':
    build()
