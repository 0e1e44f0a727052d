"""Builds quest_amd/libquest_hip.so for gfx950 with hipcc (no torch headers, no pybind).

    python -m quest_amd.build
"""
from __future__ import annotations

import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB_PATH = os.path.join(HERE, 'libquest_hip.so')
SOURCES = ['rowops.hip', 'hadamard_mfma.hip', 'gemm.hip', 'gemm_big.hip', 'gemm_small.hip', 'gemm_staged.hip',
           'gemm_decode.hip', 'gemm_e2m3.hip', 'capi.hip']

FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared',
    '-ffp-contract=off',                       # the quantiser's rounding steps must stay separate
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wall', '-Wno-unused-function',
]


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(' '.join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = '\n'.join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed ({res.returncode}):\n{err}')
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, extra_flags: list[str] | None = None, jobs: int = 4) -> str:
    """Compiles every source to an object (up to `jobs` at a time) and links the shared library."""
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    flags = [f for f in FLAGS if f != '-shared'] + list(extra_flags or [])
    with tempfile.TemporaryDirectory(prefix='quest_hip_build_') as tmp:
        objs = [os.path.join(tmp, os.path.splitext(s)[0] + '.o') for s in SOURCES]
        cmds = [[hipcc, *flags, '-c', os.path.join(CSRC, s), '-o', o] for s, o in zip(SOURCES, objs)]
        with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
            for fut in [pool.submit(_run, c, verbose) for c in cmds]:
                fut.result()
        _run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', *objs, '-o', LIB_PATH], verbose)
    return LIB_PATH


if __name__ == '__main__':
    print(build(verbose=True))
