"""Drop-in for the reference's native module ``torchopt._C.adam_op`` on ROCm GPUs.

Same seven functions, keyword names, return conventions and error behaviour as
the pybind11 module registered in /root/reference/src/adam_op/adam_op.cpp:155-215
(type stub /root/reference/torchopt/_C/adam_op.pyi), with the device branch of
its dispatcher (adam_op.cpp:32-153) served by hand-written gfx950 kernels behind
the C ABI of libtoa_adam.so.  PyTorch is used only for what the reference uses
ATen for: `empty_like`, data pointers, and the current stream.

Differences from the reference, all deliberate:
  * only GPU tensors are served.  Any other device raises
    RuntimeError("Not implemented") -- the reference's own message for devices
    it has no kernel for (adam_op.cpp:47-49) -- instead of silently computing
    somewhere else;
  * kernels are enqueued on PyTorch's current stream of the tensors' device,
    not on the null stream (adam_op_impl_cuda.cu:83);
  * element counts, dtypes and devices are checked instead of assumed, and any
    length is handled (the reference's device kernels drop the last n % 4
    elements for n >= 1024, adam_op_impl_cuda.cu:95-96);
  * additive multi-tensor entry points (`forward_multi_`, ...) run a whole list
    of tensors in one launch;
  * additive `fused_step_` / `fused_step_multi_` run the classic in-place step
    (Adam, scale by -lr, add to the parameters) in one pass.
"""

from __future__ import annotations

import ctypes
import operator
from typing import Sequence

import torch

from torchopt_amd import _lib


__all__ = [
    'forward_',
    'forward_mu',
    'forward_nu',
    'forward_updates',
    'backward_mu',
    'backward_nu',
    'backward_updates',
    'forward_multi_',
    'forward_mu_multi',
    'forward_nu_multi',
    'forward_updates_multi',
    'backward_mu_multi',
    'backward_nu_multi',
    'backward_updates_multi',
    'fused_step_',
    'fused_step_multi_',
]

_DTYPES = {torch.float32: _lib.TOA_F32, torch.float64: _lib.TOA_F64,
           torch.float16: _lib.TOA_F16, torch.bfloat16: _lib.TOA_BF16}


# --------------------------------------------------------------------------- helpers


def _count(count) -> int:
    """`count` is a size_t in the reference (include/common.h:24): a Python int or anything
    with __index__, in practice a 0-dim int64 tensor (transform/scale_by_adam.py:323)."""
    c = operator.index(count)
    if c < 0:
        raise TypeError(f'count must be a non-negative integer, got {c}')
    return c


def _dtype_code(t: torch.Tensor, name: str) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        # wording of ATen's dispatch failure, which is what the reference raises
        raise RuntimeError(f'"{name}" not implemented for \'{t.dtype}\'') from None


def _dense(t: torch.Tensor) -> bool:
    """Non-overlapping and dense: the tensor's elements tile one span of memory."""
    if t.is_contiguous():
        return True
    expect = 1
    for size, stride in sorted(((s, st) for s, st in zip(t.shape, t.stride()) if s != 1),
                               key=lambda p: p[1]):
        if stride != expect:
            return False
        expect *= size
    return True


def _gate(name: str, lead: torch.Tensor, others: Sequence[torch.Tensor]) -> tuple[int, int]:
    """Device / dtype / size checks shared by all ops; returns (dtype code, n)."""
    if not lead.is_cuda:
        raise RuntimeError('Not implemented')
    code = _dtype_code(lead, name)
    n = lead.numel()
    for t in others:
        if t.device != lead.device:
            raise RuntimeError(
                f'{name}: expected all tensors on {lead.device}, got one on {t.device}')
        if t.dtype != lead.dtype:
            raise RuntimeError(f'{name}: expected scalar type {lead.dtype} but found {t.dtype}')
        if t.numel() != n:
            raise RuntimeError(f'{name}: size mismatch, {n} vs {t.numel()} elements')
    return code, n


def _as_layout_of(x: torch.Tensor, donor: torch.Tensor) -> torch.Tensor:
    """A read-only operand in the memory order of `donor`, copying only if it is not already."""
    if x.numel() <= 1 or (x.is_contiguous() and donor.is_contiguous()):
        return x
    if x.shape == donor.shape:
        return x if x.stride() == donor.stride() else torch.empty_like(donor).copy_(x)
    if donor.is_contiguous():
        return x.contiguous()
    raise RuntimeError('operands of different shapes must be contiguous')


def _require_dense(name: str, what: str, t: torch.Tensor) -> None:
    if not _dense(t):
        raise RuntimeError(f'{name}: `{what}` must be contiguous (non-overlapping and dense), '
                           f'got sizes {tuple(t.shape)} strides {t.stride()}')


class _on_device_of:  # noqa: N801
    """Make the tensor's device current for the launch (the C ABI uses the current device)."""

    __slots__ = ('idx', 'prev')

    def __init__(self, t: torch.Tensor) -> None:
        self.idx = t.device.index
        self.prev = -1

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)
        return torch.cuda.current_stream().cuda_stream

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


# --------------------------------------------------------------------------- single tensor


def forward_(updates, mu, nu, b1, b2, eps, eps_root, count):
    """Fused in-place Adam step; returns ``[updates, mu, nu]`` (the same tensors, mutated).

    Counterpart of adamForwardInplace (adam_op.cpp:32-50, adam_op_impl_cpu.cpp:64-91).
    """
    name = 'adamForwardInplace'
    code, n = _gate(name, updates, (mu, nu))
    c = _count(count)
    if n:
        for what, t in (('updates', updates), ('mu', mu), ('nu', nu)):
            _require_dense(name, what, t)
        if n > 1 and not (updates.stride() == mu.stride() == nu.stride()):
            raise RuntimeError(f'{name}: updates, mu and nu must share one memory layout')
        with _on_device_of(updates) as stream:
            rc = _lib.load().toa_adam_forward_inplace(
                code, updates.data_ptr(), mu.data_ptr(), nu.data_ptr(), n,
                b1, b2, eps, eps_root, c, stream)
        _lib.check(rc, name)
    return [updates, mu, nu]


def forward_mu(updates, mu, b1):
    """``b1*mu + (1-b1)*updates`` into a new tensor shaped like `mu` (adam_op.cpp:52-65)."""
    name = 'adamForwardMu'
    code, n = _gate(name, updates, (mu,))
    _require_dense(name, 'mu', mu)
    mu_out = torch.empty_like(mu)
    if n:
        updates = _as_layout_of(updates, mu)
        with _on_device_of(updates) as stream:
            rc = _lib.load().toa_adam_forward_mu(
                code, updates.data_ptr(), mu.data_ptr(), n, b1, mu_out.data_ptr(), stream)
        _lib.check(rc, name)
    return mu_out


def forward_nu(updates, nu, b2):
    """``b2*nu + (1-b2)*updates**2`` into a new tensor shaped like `nu` (adam_op.cpp:67-80)."""
    name = 'adamForwardNu'
    code, n = _gate(name, updates, (nu,))
    _require_dense(name, 'nu', nu)
    nu_out = torch.empty_like(nu)
    if n:
        updates = _as_layout_of(updates, nu)
        with _on_device_of(updates) as stream:
            rc = _lib.load().toa_adam_forward_nu(
                code, updates.data_ptr(), nu.data_ptr(), n, b2, nu_out.data_ptr(), stream)
        _lib.check(rc, name)
    return nu_out


def forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count):
    """Bias-corrected ``mu_hat / (sqrt(nu_hat + eps_root) + eps)`` (adam_op.cpp:82-99)."""
    name = 'adamForwardUpdates'
    code, n = _gate(name, new_mu, (new_nu,))
    c = _count(count)
    _require_dense(name, 'new_mu', new_mu)
    updates_out = torch.empty_like(new_mu)
    if n:
        new_nu = _as_layout_of(new_nu, new_mu)
        with _on_device_of(new_mu) as stream:
            rc = _lib.load().toa_adam_forward_updates(
                code, new_mu.data_ptr(), new_nu.data_ptr(), n, b1, b2, eps, eps_root, c,
                updates_out.data_ptr(), stream)
        _lib.check(rc, name)
    return updates_out


def backward_mu(dmu, updates, mu, b1):
    """VJP of `forward_mu`; returns ``[dupdates, dmu]``.  `updates` and `mu` only donate
    shape and layout (adam_op.cpp:101-115, adam_op_impl_cpu.cpp:228-245)."""
    name = 'adamBackwardMu'
    code, n = _gate(name, dmu, (updates, mu))
    _require_dense(name, 'updates', updates)
    _require_dense(name, 'mu', mu)
    dupdates_out = torch.empty_like(updates)
    dmu_out = torch.empty_like(mu)
    if n:
        if n > 1 and dupdates_out.stride() != dmu_out.stride():
            raise RuntimeError(f'{name}: updates and mu must share one memory layout')
        dmu = _as_layout_of(dmu, dmu_out)
        with _on_device_of(dmu) as stream:
            rc = _lib.load().toa_adam_backward_mu(
                code, dmu.data_ptr(), n, b1, dupdates_out.data_ptr(), dmu_out.data_ptr(), stream)
        _lib.check(rc, name)
    return [dupdates_out, dmu_out]


def backward_nu(dnu, updates, nu, b1):  # 4th name as registered (adam_op.cpp:203); it is b2
    """VJP of `forward_nu`; returns ``[dupdates, dnu]`` (adam_op.cpp:117-131,
    adam_op_impl_cpu.cpp:266-284).  The decay is `b2`; the keyword is spelled `b1` because the
    reference registers it so and callers pass it positionally."""
    name = 'adamBackwardNu'
    b2 = b1
    code, n = _gate(name, dnu, (updates, nu))
    _require_dense(name, 'updates', updates)
    _require_dense(name, 'nu', nu)
    dupdates_out = torch.empty_like(updates)
    dnu_out = torch.empty_like(nu)
    if n:
        if n > 1 and dupdates_out.stride() != dnu_out.stride():
            raise RuntimeError(f'{name}: updates and nu must share one memory layout')
        dnu = _as_layout_of(dnu, dnu_out)
        with _on_device_of(dnu) as stream:
            rc = _lib.load().toa_adam_backward_nu(
                code, dnu.data_ptr(), updates.data_ptr(), n, b2,
                dupdates_out.data_ptr(), dnu_out.data_ptr(), stream)
        _lib.check(rc, name)
    return [dupdates_out, dnu_out]


def backward_updates(dupdates, updates, new_mu, new_nu, b1, b2, eps_root, count):
    """The reference's VJP of `forward_updates`; `updates` is the forward output.  Returns
    ``[dnew_mu, dnew_nu]`` (adam_op.cpp:133-153, adam_op_impl_cpu.cpp:318-347)."""
    name = 'adamBackwardUpdates'
    code, n = _gate(name, dupdates, (updates, new_mu, new_nu))
    c = _count(count)
    _require_dense(name, 'new_mu', new_mu)
    _require_dense(name, 'new_nu', new_nu)
    dmu_out = torch.empty_like(new_mu)
    dnu_out = torch.empty_like(new_nu)
    if n:
        if n > 1 and dmu_out.stride() != dnu_out.stride():
            raise RuntimeError(f'{name}: new_mu and new_nu must share one memory layout')
        dupdates = _as_layout_of(dupdates, dmu_out)
        updates = _as_layout_of(updates, dmu_out)
        with _on_device_of(dupdates) as stream:
            rc = _lib.load().toa_adam_backward_updates(
                code, dupdates.data_ptr(), updates.data_ptr(), new_mu.data_ptr(), n,
                b1, b2, eps_root, c, dmu_out.data_ptr(), dnu_out.data_ptr(), stream)
        _lib.check(rc, name)
    return [dmu_out, dnu_out]


# --------------------------------------------------------------------------- multi tensor


def _ptr_array(tensors: Sequence[torch.Tensor]):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _size_array(tensors: Sequence[torch.Tensor]):
    return (ctypes.c_size_t * len(tensors))(*[t.numel() for t in tensors])


def _counts_array(counts, num: int):
    """Returns (uint64 array or None, count_all)."""
    if not isinstance(counts, (list, tuple)):
        return None, _count(counts)
    if len(counts) != num:
        raise RuntimeError(f'expected {num} counts, got {len(counts)}')
    if num and all(isinstance(c, torch.Tensor) for c in counts):
        # one device-to-host transfer for the whole list, not one per leaf
        values = torch.stack([c.reshape(()) for c in counts]).tolist()
    else:
        values = [_count(c) for c in counts]
    if any(v < 0 for v in values):
        raise TypeError('counts must be non-negative integers')
    if len(set(values)) <= 1:
        return None, (values[0] if values else 0)
    return (ctypes.c_uint64 * num)(*values), 0


def _gate_multi(name: str, lists: Sequence[Sequence[torch.Tensor]]) -> tuple[int, int]:
    """Checks for a multi-tensor call; returns (dtype code, number of tensors)."""
    num = len(lists[0])
    for lst in lists:
        if len(lst) != num:
            raise RuntimeError(f'{name}: tensor lists differ in length')
    if num == 0:
        return _lib.TOA_F32, 0
    lead = lists[0][0]
    if not lead.is_cuda:
        raise RuntimeError('Not implemented')
    code = _dtype_code(lead, name)
    for k in range(num):
        first = lists[0][k]
        n = first.numel()
        for lst in lists:
            t = lst[k]
            if t.device != lead.device:
                raise RuntimeError(f'{name}: all tensors of one call must be on {lead.device}')
            if t.dtype != lead.dtype:
                raise RuntimeError(
                    f'{name}: expected scalar type {lead.dtype} but found {t.dtype}')
            if t.numel() != n:
                raise RuntimeError(f'{name}: size mismatch in tensor {k}')
            if n > 1 and (t.stride() != first.stride() or not _dense(t)):
                raise RuntimeError(f'{name}: tensor {k} operands must share one dense layout')
    return code, num


def forward_multi_(updates, mu, nu, b1, b2, eps, eps_root, counts):
    """`forward_` over lists of tensors in one launch per 100-odd tensors; mutates all of them
    and returns ``(updates, mu, nu)`` (the lists it was given).  `counts` is one step number
    for all tensors or one per tensor (ints or 0-dim integer tensors)."""
    name = 'adamForwardInplaceMulti'
    code, num = _gate_multi(name, (updates, mu, nu))
    if num:
        carr, call = _counts_array(counts, num)
        with _on_device_of(updates[0]) as stream:
            rc = _lib.load().toa_adam_forward_inplace_multi(
                code, num, _ptr_array(updates), _ptr_array(mu), _ptr_array(nu),
                _size_array(updates), b1, b2, eps, eps_root, carr, call, stream)
        _lib.check(rc, name)
    return updates, mu, nu


def forward_mu_multi(updates, mu, b1):
    """`forward_mu` over lists; returns the list of new tensors."""
    name = 'adamForwardMuMulti'
    out = [torch.empty_like(t) for t in mu]
    code, num = _gate_multi(name, (updates, mu, out))
    if num:
        with _on_device_of(mu[0]) as stream:
            rc = _lib.load().toa_adam_forward_mu_multi(
                code, num, _ptr_array(updates), _ptr_array(mu), _size_array(mu), b1,
                _ptr_array(out), stream)
        _lib.check(rc, name)
    return out


def forward_nu_multi(updates, nu, b2):
    """`forward_nu` over lists; returns the list of new tensors."""
    name = 'adamForwardNuMulti'
    out = [torch.empty_like(t) for t in nu]
    code, num = _gate_multi(name, (updates, nu, out))
    if num:
        with _on_device_of(nu[0]) as stream:
            rc = _lib.load().toa_adam_forward_nu_multi(
                code, num, _ptr_array(updates), _ptr_array(nu), _size_array(nu), b2,
                _ptr_array(out), stream)
        _lib.check(rc, name)
    return out


def forward_updates_multi(new_mu, new_nu, b1, b2, eps, eps_root, counts):
    """`forward_updates` over lists; returns the list of new tensors."""
    name = 'adamForwardUpdatesMulti'
    out = [torch.empty_like(t) for t in new_mu]
    code, num = _gate_multi(name, (new_mu, new_nu, out))
    if num:
        carr, call = _counts_array(counts, num)
        with _on_device_of(new_mu[0]) as stream:
            rc = _lib.load().toa_adam_forward_updates_multi(
                code, num, _ptr_array(new_mu), _ptr_array(new_nu), _size_array(new_mu),
                b1, b2, eps, eps_root, carr, call, _ptr_array(out), stream)
        _lib.check(rc, name)
    return out


def backward_mu_multi(dmu, updates, mu, b1):
    """`backward_mu` over lists; returns ``(dupdates list, dmu list)``."""
    name = 'adamBackwardMuMulti'
    dupdates_out = [torch.empty_like(t) for t in updates]
    dmu_out = [torch.empty_like(t) for t in mu]
    dmu = [_as_layout_of(d, o) for d, o in zip(dmu, dmu_out)]
    code, num = _gate_multi(name, (dmu, dupdates_out, dmu_out))
    if num:
        with _on_device_of(dmu[0]) as stream:
            rc = _lib.load().toa_adam_backward_mu_multi(
                code, num, _ptr_array(dmu), _size_array(dmu), b1,
                _ptr_array(dupdates_out), _ptr_array(dmu_out), stream)
        _lib.check(rc, name)
    return dupdates_out, dmu_out


def backward_nu_multi(dnu, updates, nu, b2):
    """`backward_nu` over lists; returns ``(dupdates list, dnu list)``."""
    name = 'adamBackwardNuMulti'
    dupdates_out = [torch.empty_like(t) for t in updates]
    dnu_out = [torch.empty_like(t) for t in nu]
    dnu = [_as_layout_of(d, o) for d, o in zip(dnu, dnu_out)]
    code, num = _gate_multi(name, (dnu, updates, dupdates_out, dnu_out))
    if num:
        with _on_device_of(dnu[0]) as stream:
            rc = _lib.load().toa_adam_backward_nu_multi(
                code, num, _ptr_array(dnu), _ptr_array(updates), _size_array(dnu), b2,
                _ptr_array(dupdates_out), _ptr_array(dnu_out), stream)
        _lib.check(rc, name)
    return dupdates_out, dnu_out


def backward_updates_multi(dupdates, updates, new_mu, new_nu, b1, b2, eps_root, counts):
    """`backward_updates` over lists; returns ``(dnew_mu list, dnew_nu list)``."""
    name = 'adamBackwardUpdatesMulti'
    dmu_out = [torch.empty_like(t) for t in new_mu]
    dnu_out = [torch.empty_like(t) for t in new_nu]
    dupdates = [_as_layout_of(d, o) for d, o in zip(dupdates, dmu_out)]
    code, num = _gate_multi(name, (dupdates, updates, new_mu, dmu_out, dnu_out))
    if num:
        carr, call = _counts_array(counts, num)
        with _on_device_of(dupdates[0]) as stream:
            rc = _lib.load().toa_adam_backward_updates_multi(
                code, num, _ptr_array(dupdates), _ptr_array(updates), _ptr_array(new_mu),
                _size_array(dupdates), b1, b2, eps_root, carr, call,
                _ptr_array(dmu_out), _ptr_array(dnu_out), stream)
        _lib.check(rc, name)
    return dmu_out, dnu_out


# --------------------------------------------------------------------------- fused optimizer step


def fused_step_(params, updates, mu, nu, b1, b2, eps, eps_root, count, lr, *, maximize=False,
                write_updates=False):
    """The classic in-place step in one pass: `forward_`, then ``updates *= -lr``
    (/root/reference/torchopt/transform/scale.py:93-98) and ``params += updates``
    (/root/reference/torchopt/update.py:71-74), bit-identical to the three passes.

    Overwrites `params`, `mu`, `nu`; `updates` receives the scaled update only if
    `write_updates` (the reference chain leaves it there), otherwise it is only read.
    `maximize` negates the gradient first (/root/reference/torchopt/alias/utils.py:148).
    Returns ``[params, updates, mu, nu]``.
    """
    name = 'adamFusedStep'
    code, n = _gate(name, updates, (mu, nu, params))
    c = _count(count)
    if n:
        for what, t in (('params', params), ('updates', updates), ('mu', mu), ('nu', nu)):
            _require_dense(name, what, t)
        if n > 1 and not (params.stride() == updates.stride() == mu.stride() == nu.stride()):
            raise RuntimeError(f'{name}: params, updates, mu and nu must share one memory layout')
        with _on_device_of(updates) as stream:
            rc = _lib.load().toa_adam_fused_step(
                code, params.data_ptr(), updates.data_ptr(), mu.data_ptr(), nu.data_ptr(), n,
                b1, b2, eps, eps_root, c, lr, int(bool(maximize)), int(bool(write_updates)),
                stream)
        _lib.check(rc, name)
    return [params, updates, mu, nu]


def fused_step_multi_(params, updates, mu, nu, b1, b2, eps, eps_root, counts, lr, *,
                      maximize=False, write_updates=False):
    """`fused_step_` over lists of tensors; returns ``(params, updates, mu, nu)``."""
    name = 'adamFusedStepMulti'
    code, num = _gate_multi(name, (updates, mu, nu, params))
    if num:
        carr, call = _counts_array(counts, num)
        with _on_device_of(updates[0]) as stream:
            rc = _lib.load().toa_adam_fused_step_multi(
                code, num, _ptr_array(params), _ptr_array(updates), _ptr_array(mu),
                _ptr_array(nu), _size_array(updates), b1, b2, eps, eps_root, carr, call, lr,
                int(bool(maximize)), int(bool(write_updates)), stream)
        _lib.check(rc, name)
    return params, updates, mu, nu
