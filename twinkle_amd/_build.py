"""Builds the gfx950 shared library in-tree with hipcc (no torch C++ ABI involved)."""
from __future__ import annotations

import os
import subprocess

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'csrc')
INCLUDE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'include')
LIB_PATH = os.path.join(CSRC, 'libtwinkle_amd.so')
SOURCES = ['api.hip', 'kernels_segments.hip', 'kernels_generic.hip', 'kernels_mfma.hip', 'kernels_shared.hip', 'kernels_optim.hip', 'kernels_grouped.hip', 'kernels_act.hip', 'kernels_yardstick.hip']

# -packed-fp32-ops is switched off on purpose: the compiler must not form packed fp32 VALU ops.
HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared', '-Xclang', '-target-feature', '-Xclang',
    '-packed-fp32-ops', '-Wno-unused-command-line-argument',
]


def build_library(verbose: bool = False) -> str:
    """Compile every HIP source into ``csrc/libtwinkle_amd.so`` and return its path."""
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    cmd = [hipcc, *HIPCC_FLAGS, '-I', INCLUDE, '-I', CSRC, *[os.path.join(CSRC, s) for s in SOURCES], '-o', LIB_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError('hipcc failed:\n' + ' '.join(cmd) + '\n' + proc.stdout + proc.stderr)
    if verbose:
        print(proc.stderr)
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(verbose=True))
