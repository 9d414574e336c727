"""ctypes binding of libtoa_adam.so (the C ABI in include/toa_adam.h).

The library is the only implementation behind this package: if it has not been
built, loading raises and every op fails loudly -- there is no CPU or eager
PyTorch fallback.
"""

from __future__ import annotations

import ctypes
import os
import threading

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, 'libtoa_adam.so')

TOA_F32 = 0
TOA_F64 = 1
TOA_F16 = 2
TOA_BF16 = 3
ABI_VERSION = 5

_vp = ctypes.c_void_p
_vpp = ctypes.POINTER(ctypes.c_void_p)
_sz = ctypes.c_size_t
_szp = ctypes.POINTER(ctypes.c_size_t)
_d = ctypes.c_double
_u64 = ctypes.c_uint64
_u64p = ctypes.POINTER(ctypes.c_uint64)
_i = ctypes.c_int

# name -> argtypes; every function returns int except the two noted below.
SIGNATURES = {
    'toa_adam_set_waves_per_cu': [_i],
    'toa_adam_set_max_grid': [ctypes.c_uint],
    'toa_adam_set_schedule': [_i],
    'toa_adam_set_load_order': [_i],
    'toa_adam_set_tuning': [_i],
    'toa_adam_tuned_load_order': [_i, _vp, _vp, _vp, _sz],
    'toa_adam_clock_probe': [_vp, ctypes.c_uint32, _vp],
    'toa_adam_set_plan_mode': [_i],
    'toa_adam_release_plans': [],
    'toa_adam_state_slack': [],
    'toa_adam_state_shift': [_vp, _i],
    'toa_adam_forward_inplace': [_i, _vp, _vp, _vp, _sz, _d, _d, _d, _d, _u64, _vp],
    'toa_adam_forward_mu': [_i, _vp, _vp, _sz, _d, _vp, _vp],
    'toa_adam_forward_nu': [_i, _vp, _vp, _sz, _d, _vp, _vp],
    'toa_adam_forward_updates': [_i, _vp, _vp, _sz, _d, _d, _d, _d, _u64, _vp, _vp],
    'toa_adam_backward_mu': [_i, _vp, _sz, _d, _vp, _vp, _vp],
    'toa_adam_backward_nu': [_i, _vp, _vp, _sz, _d, _vp, _vp, _vp],
    'toa_adam_backward_updates': [_i, _vp, _vp, _vp, _sz, _d, _d, _d, _u64, _vp, _vp, _vp],
    'toa_adam_forward_inplace_multi': [_i, _sz, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _d, _u64p,
                                       _u64, _vp],
    'toa_adam_forward_inplace_multi_noalloc': [_i, _sz, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _d,
                                               _u64p, _u64, _vp],
    'toa_adam_forward_mu_multi': [_i, _sz, _vpp, _vpp, _szp, _d, _vpp, _vp],
    'toa_adam_forward_nu_multi': [_i, _sz, _vpp, _vpp, _szp, _d, _vpp, _vp],
    'toa_adam_forward_updates_multi': [_i, _sz, _vpp, _vpp, _szp, _d, _d, _d, _d, _u64p, _u64,
                                       _vpp, _vp],
    'toa_adam_backward_mu_multi': [_i, _sz, _vpp, _szp, _d, _vpp, _vpp, _vp],
    'toa_adam_backward_nu_multi': [_i, _sz, _vpp, _vpp, _szp, _d, _vpp, _vpp, _vp],
    'toa_adam_backward_updates_multi': [_i, _sz, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _u64p, _u64,
                                        _vpp, _vpp, _vp],
    'toa_adam_forward_all': [_i, _vp, _vp, _vp, _sz, _d, _d, _d, _d, _u64, _vp, _vp, _vp, _vp],
    'toa_adam_forward_all_multi': [_i, _sz, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _d, _u64p, _u64,
                                   _vpp, _vpp, _vpp, _vp],
    'toa_adam_backward_all': [_i, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _d, _d, _d, _u64, _vp, _vp,
                              _vp, _vp],
    'toa_adam_backward_all_multi': [_i, _sz, _vpp, _vpp, _vpp, _vpp, _vpp, _vpp, _szp, _d, _d, _d,
                                    _u64p, _u64, _vpp, _vpp, _vpp, _vp],
    'toa_adam_fused_step': [_i, _vp, _vp, _vp, _vp, _sz, _d, _d, _d, _d, _u64, _d, _d, _i, _i, _i,
                            _vp],
    'toa_adam_fused_step_multi': [_i, _sz, _vpp, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _d, _u64p,
                                  _u64, _d, _d, _i, _i, _i, _vp],
    # step number on the device
    'toa_adam_bias_rows': [_i, _d, _d, _d, _u64, _sz, _vp],
    'toa_adam_bias_rows_needed': [_d, _d, _u64, _sz],
    'toa_adam_count_advance': [_vp, _vp],
    'toa_adam_forward_inplace_devcount': [_i, _vp, _vp, _vp, _sz, _d, _d, _d, _d, _vp, _u64, _sz,
                                          _vp, _vp],
    'toa_adam_forward_inplace_multi_devcount': [_i, _sz, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _d,
                                                _vp, _u64, _sz, _vp, _vp],
    'toa_adam_fused_step_devcount': [_i, _vp, _vp, _vp, _vp, _sz, _d, _d, _d, _d, _vp, _u64, _sz,
                                     _vp, _d, _d, _i, _i, _i, _vp],
    'toa_adam_fused_step_multi_devcount': [_i, _sz, _vpp, _vpp, _vpp, _vpp, _szp, _d, _d, _d, _d,
                                           _vp, _u64, _sz, _vp, _d, _d, _i, _i, _i, _vp],
}

_lib = None
_lock = threading.Lock()


class LibraryNotBuiltError(ImportError):
    """libtoa_adam.so is missing; run `python torchopt_amd/build.py`."""


def load() -> ctypes.CDLL:
    """Load the library once and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise LibraryNotBuiltError(
                f'{LIB_PATH} not found: the HIP library has not been built '
                '(run `python torchopt_amd/build.py`); there is no fallback path',
            )
        lib = ctypes.CDLL(LIB_PATH)
        lib.toa_adam_abi_version.restype = _i
        lib.toa_adam_abi_version.argtypes = []
        lib.toa_adam_error_string.restype = ctypes.c_char_p
        lib.toa_adam_error_string.argtypes = [_i]
        got = lib.toa_adam_abi_version()
        if got != ABI_VERSION:
            raise ImportError(f'{LIB_PATH}: ABI version {got}, expected {ABI_VERSION}; rebuild it')
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = {'toa_adam_set_max_grid': ctypes.c_uint,
                          'toa_adam_bias_rows_needed': ctypes.c_size_t,
                          'toa_adam_state_slack': ctypes.c_size_t,
                          'toa_adam_state_shift': ctypes.c_size_t}.get(name, _i)
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a non-zero return code into RuntimeError (the reference raises C++ exceptions)."""
    if rc != 0:
        msg = load().toa_adam_error_string(rc).decode()
        raise RuntimeError(f'{what}: {msg} (code {rc})')
