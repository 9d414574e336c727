"""Compile the two in-tree binaries:

  libtoa_adam.so              the HIP kernels behind the C ABI (hipcc, gfx950 only)
  _C.<python-abi>.so          the PyTorch extension module in front of it (g++, host only)

    python torchopt_amd/build.py

(run as a script, or load this file by path: importing the package itself needs the binaries
this file produces).  hipcc cross-compiles without a GPU, so this runs anywhere ROCm and PyTorch-ROCm are installed.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, 'libtoa_adam.so')
SOURCES = [os.path.join(PKG_DIR, 'csrc', 'toa_adam.hip')]
HEADERS = [
    os.path.join(PKG_DIR, 'csrc', 'adam_kernels.hpp'),
    os.path.join(PKG_DIR, 'csrc', 'plan_cache.hpp'),
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


BINDING_SRC = os.path.join(PKG_DIR, 'csrc', 'binding.cpp')
BINDING_PATH = os.path.join(PKG_DIR, '_C' + sysconfig.get_config_var('EXT_SUFFIX'))


def build_binding(verbose: bool = False) -> str:
    """Compile torchopt_amd/_C*.so: pybind11 + ATen on the host side, linked against
    libtoa_adam.so (found next to it at run time through an $ORIGIN rpath)."""
    import torch
    from torch.utils import cpp_extension

    if not os.path.exists(LIB_PATH):
        build_library()
    rocm = os.environ.get('ROCM_PATH', '/opt/rocm')
    torch_lib = cpp_extension.library_paths()[0]
    includes = [os.path.join(REPO_DIR, 'include'), *cpp_extension.include_paths(),
                sysconfig.get_paths()['include'], os.path.join(rocm, 'include')]
    cmd = [os.environ.get('CXX', 'g++'), '-O2', '-std=c++17', '-fPIC', '-shared',
           '-fvisibility=hidden', '-Wall', '-Wno-unused-function',
           '-D__HIP_PLATFORM_AMD__=1', '-DUSE_ROCM=1', '-DTORCH_EXTENSION_NAME=_C',
           f'-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}',
           *[f'-I{p}' for p in includes], BINDING_SRC, '-o', BINDING_PATH + '.tmp',
           f'-L{torch_lib}', f'-L{PKG_DIR}', f'-L{os.path.join(rocm, "lib")}',
           '-ltorch_python', '-ltorch', '-ltorch_cpu', '-lc10', '-lc10_hip', '-ltorch_hip',
           '-l:libtoa_adam.so', '-lamdhip64',
           '-Wl,-rpath,$ORIGIN', f'-Wl,-rpath,{torch_lib}', f'-Wl,-rpath,{os.path.join(rocm, "lib")}']
    if verbose:
        print(' '.join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f'{cmd[0]} failed ({proc.returncode}):\n{proc.stderr[-4000:]}')
    if verbose and proc.stderr.strip():
        print(proc.stderr, file=sys.stderr)
    os.replace(BINDING_PATH + '.tmp', BINDING_PATH)
    return BINDING_PATH


def build_all(verbose: bool = False) -> list[str]:
    return [build_library(force=True, verbose=verbose), build_binding(verbose=verbose)]


if __name__ == '__main__':
    for path in build_all(verbose=True):
        print(path)
