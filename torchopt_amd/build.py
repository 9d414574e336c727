"""Compile libtoa_adam.so (HIP, gfx950 only) in-tree with hipcc.

    python -m torchopt_amd.build

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, 'libtoa_adam.so')
SOURCES = [os.path.join(PKG_DIR, 'csrc', 'toa_adam.hip')]
HEADERS = [
    os.path.join(PKG_DIR, 'csrc', 'adam_kernels.hpp'),
    os.path.join(REPO_DIR, 'include', 'toa_adam.h'),
]

# -ffp-contract=off: results are pinned to a CPU build without FMA contraction;
#   every product and sum must round on its own.
# -packed-fp32-ops off: scalar fp32 VALU code only.
# No fast-math, no denormal flushing, correctly rounded divide/sqrt (defaults).
HIPCC_FLAGS = [
    '-O3',
    '-std=c++17',
    '--offload-arch=gfx950',
    '-fPIC',
    '-shared',
    '-ffp-contract=off',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-fvisibility=hidden',
    '-Wall',
]


def hipcc() -> str:
    exe = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
    if not os.path.exists(exe):
        raise RuntimeError('hipcc not found: ROCm is required to build libtoa_adam.so')
    return exe


def is_stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > built for p in SOURCES + HEADERS)


def build_library(force: bool = True, verbose: bool = False) -> str:
    """Run hipcc; returns the path of the built library."""
    if not force and not is_stale():
        return LIB_PATH
    cmd = [hipcc(), *HIPCC_FLAGS, '-I', os.path.join(REPO_DIR, 'include'),
           '-I', os.path.join(PKG_DIR, 'csrc'), *SOURCES, '-o', LIB_PATH + '.tmp']
    if verbose:
        print(' '.join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the device-only target feature; that warning is harmless
    noise = "is not a recognized feature for this target"
    err = '\n'.join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f'hipcc failed ({proc.returncode}):\n{err}')
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(LIB_PATH + '.tmp', LIB_PATH)
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(force=True, verbose=True))
