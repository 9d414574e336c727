"""ctypes front-end of the C oracle (liboracle_adam.so) on NumPy arrays.

TEST INFRASTRUCTURE, NOT PRODUCT: only tests, the smoke check and the
CPU-baseline leg of the benchmark may import this module.  The shipped operator
(torchopt_amd) never does.

`load_reference()` additionally loads, where it has been built, the reference's
own compiled CPU op (oracle/_ref/_C*.so, built by `make -C oracle ref` from the
sources under /root/reference) as a Python module exposing `adam_op.forward_`
and friends on CPU torch tensors.  `load_dropin()` loads the reference's extension
built with its device branch routed to libtoa_adam.so (oracle/_ref/dropin/).
"""

from __future__ import annotations

import ctypes
import glob
import importlib.util
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'liboracle_adam.so')

# float16 arrays are NumPy's own; bfloat16 has no NumPy dtype, so bfloat16 data travels as uint16
# bit patterns (a uint16 array always means bfloat16 here).
_SFX = {np.dtype(np.float32): 'f32', np.dtype(np.float64): 'f64', np.dtype(np.float16): 'f16',
        np.dtype(np.uint16): 'bf16'}

_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle (gcc, a second or two)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(['make', '-C', _HERE, '--no-print-directory'], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_adam_threads_for.restype = ctypes.c_int
        _lib.oracle_adam_threads_for.argtypes = [ctypes.c_size_t]
        for name in ('oracle_f16_from_f32', 'oracle_bf16_from_f32'):
            getattr(_lib, name).restype = ctypes.c_uint16
            getattr(_lib, name).argtypes = [ctypes.c_float]
        for name in ('oracle_f32_from_f16', 'oracle_f32_from_bf16'):
            getattr(_lib, name).restype = ctypes.c_float
            getattr(_lib, name).argtypes = [ctypes.c_uint16]
    return _lib


def _ptr(a: np.ndarray):
    assert a.flags['C_CONTIGUOUS'] and a.dtype in _SFX
    return a.ctypes.data_as(ctypes.c_void_p)


def _fn(name: str, dtype):
    return getattr(lib(), f'oracle_adam_{name}_{_SFX[np.dtype(dtype)]}')


_D = ctypes.c_double
_U64 = ctypes.c_uint64
_SZ = ctypes.c_size_t


def bf16_bits(a) -> np.ndarray:
    """float32 array -> bfloat16 bit patterns (uint16), round to nearest even, NaN -> 0x7fc0:
    the conversion c10::BFloat16 performs."""
    x = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    out = ((x + np.uint32(0x7fff) + ((x >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16))
    out = out.astype(np.uint16)
    out[np.isnan(np.asarray(a, dtype=np.float32))] = 0x7fc0
    return out


def bf16_to_f32(bits) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(
        np.float32)


def host_scalars(b1, b2, eps_root, count):
    out = (ctypes.c_double * 4)()
    lib().oracle_adam_host_scalars(_D(b1), _D(b2), _D(eps_root), _U64(count), out)
    return tuple(out)


def threads_for(n: int) -> int:
    return lib().oracle_adam_threads_for(n)


def forward_inplace(updates, mu, nu, b1, b2, eps, eps_root, count):
    """Mutates the three arrays, like `forward_`."""
    _fn('forward_inplace', updates.dtype)(_ptr(updates), _ptr(mu), _ptr(nu), _SZ(updates.size),
                                          _D(b1), _D(b2), _D(eps), _D(eps_root), _U64(count))
    return updates, mu, nu


def forward_mu(updates, mu, b1):
    out = np.empty_like(mu)
    _fn('forward_mu', updates.dtype)(_ptr(updates), _ptr(mu), _SZ(updates.size), _D(b1), _ptr(out))
    return out


def forward_nu(updates, nu, b2):
    out = np.empty_like(nu)
    _fn('forward_nu', updates.dtype)(_ptr(updates), _ptr(nu), _SZ(updates.size), _D(b2), _ptr(out))
    return out


def forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count):
    out = np.empty_like(new_mu)
    _fn('forward_updates', new_mu.dtype)(_ptr(new_mu), _ptr(new_nu), _SZ(new_mu.size), _D(b1),
                                         _D(b2), _D(eps), _D(eps_root), _U64(count), _ptr(out))
    return out


def backward_mu(dmu, b1):
    du, dm = np.empty_like(dmu), np.empty_like(dmu)
    _fn('backward_mu', dmu.dtype)(_ptr(dmu), _SZ(dmu.size), _D(b1), _ptr(du), _ptr(dm))
    return du, dm


def backward_nu(dnu, updates, b2):
    du, dn = np.empty_like(dnu), np.empty_like(dnu)
    _fn('backward_nu', dnu.dtype)(_ptr(dnu), _ptr(updates), _SZ(dnu.size), _D(b2), _ptr(du),
                                  _ptr(dn))
    return du, dn


def backward_updates(dupdates, updates, new_mu, b1, b2, eps_root, count):
    dm, dn = np.empty_like(dupdates), np.empty_like(dupdates)
    _fn('backward_updates', dupdates.dtype)(_ptr(dupdates), _ptr(updates), _ptr(new_mu),
                                            _SZ(dupdates.size), _D(b1), _D(b2), _D(eps_root),
                                            _U64(count), _ptr(dm), _ptr(dn))
    return dm, dn


def fused_step(params, updates, mu, nu, b1, b2, eps, eps_root, count, lr, maximize=False,
               write_updates=True, weight_decay=0.0, decoupled=False):
    """Mutates params, mu, nu (and updates when write_updates), like the reference's classic
    in-place chains: [negate], [L2 decay], forward_, [decoupled decay], scale by -lr, apply."""
    decay = 0 if weight_decay == 0.0 else (2 if decoupled else 1)
    if decay and params.dtype.itemsize == 2:
        raise ValueError('no weight decay on 16-bit tensors: torch.Tensor.add_(p, alpha=wd) is not '
                         'one arithmetic there (vectorized body and scalar tails round differently)')
    _fn('fused_step', params.dtype)(_ptr(params), _ptr(updates), _ptr(mu), _ptr(nu),
                                    _SZ(params.size), _D(b1), _D(b2), _D(eps), _D(eps_root),
                                    _U64(count), _D(lr), _D(weight_decay), ctypes.c_int(decay),
                                    ctypes.c_int(int(maximize)),
                                    ctypes.c_int(int(write_updates)))
    return params, updates, mu, nu


def reference_path():
    hits = sorted(glob.glob(os.path.join(_HERE, '_ref', '_C*.so')))
    return hits[0] if hits else None


def _load_extension(path):
    import torch  # noqa: F401  (libtorch must be loaded first)

    spec = importlib.util.spec_from_file_location('_C', path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load_reference():
    """Import the compiled reference CPU op, or return None if it was not built."""
    path = reference_path()
    return None if path is None else _load_extension(path)


def dropin_path():
    hits = sorted(glob.glob(os.path.join(_HERE, '_ref', 'dropin', '_C*.so')))
    return hits[0] if hits else None


def load_dropin():
    """Import the reference's own extension built with its device branch on libtoa_adam.so
    (`make -C oracle dropin`), or return None if it was not built.  This is the object under
    test of the drop-in boundary, not a checker."""
    path = dropin_path()
    return None if path is None else _load_extension(path)
