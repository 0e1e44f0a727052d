"""Builds quest_amd/libquest_hip.so for gfx950 with hipcc (no torch headers, no pybind).

    python -m quest_amd.build
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB_PATH = os.path.join(HERE, 'libquest_hip.so')
SOURCES = ['rowops.hip', 'hadamard_mfma.hip', 'gemm.hip', 'gemm_decode.hip', 'capi.hip']

FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared',
    '-ffp-contract=off',                       # the quantiser's rounding steps must stay separate
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wall', '-Wno-unused-function',
]


def build(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    cmd = [hipcc, *FLAGS, *(extra_flags or []), *[os.path.join(CSRC, s) for s in SOURCES], '-o', LIB_PATH]
    if verbose:
        print(' '.join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = '\n'.join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed ({res.returncode}):\n{err}')
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == '__main__':
    print(build(verbose=True))
