"""The fused Adam operator as `torch.library` operators, so that `torch.compile` can trace code
that calls it.

`torchopt_amd._C.adam_op` is a pybind11 module, as the reference's `torchopt._C.adam_op` is
(/root/reference/src/adam_op/adam_op.cpp:155-215): opaque to Dynamo, which would break the graph
at every call.  Each function is therefore also registered under the namespace `torchopt_amd`
with its schema (which arguments it overwrites) and a shape-only "fake" implementation; the real
implementation is the pybind11 function itself, so eager results, compiled results and the C ABI
underneath are one code path.

    torch.ops.torchopt_amd.forward_(updates, mu, nu, b1, b2, eps, eps_root, count)   -> None
    torch.ops.torchopt_amd.forward_mu / forward_nu / forward_updates(...)            -> Tensor
    torch.ops.torchopt_amd.backward_mu / backward_nu / backward_updates(...)         -> (Tensor, Tensor)
    torch.ops.torchopt_amd.forward_multi_ / fused_step_multi_(lists..., count, ...)  -> None
    torch.ops.torchopt_amd.count_advance_ / forward_multi_devcount_ /
        fused_step_multi_devcount_(..., bias_rows, first_count, count_tensor, ...)   -> None

In-place operators return nothing (an operator's outputs may not alias its inputs); `dispatch`
below gives every function the calling convention of its pybind11 twin and picks the registered
operator while a compiler is tracing, the direct call otherwise (the registered route costs a few
microseconds of dispatcher time per call, which an eager per-leaf loop would feel).
"""

from __future__ import annotations

from typing import List, Tuple

import torch
from torch import Tensor

from torchopt_amd._C import adam_op

_NS = 'torchopt_amd'


def _define(name: str, mutates: Tuple[str, ...] = ()):
    return torch.library.custom_op(f'{_NS}::{name}', mutates_args=mutates, device_types='cuda')


# ---- the reference's seven ------------------------------------------------------------------


@_define('forward_', ('updates', 'mu', 'nu'))
def _forward_(updates: Tensor, mu: Tensor, nu: Tensor, b1: float, b2: float, eps: float,
              eps_root: float, count: int) -> None:
    adam_op.forward_(updates, mu, nu, b1, b2, eps, eps_root, count)


@_define('forward_mu')
def _forward_mu(updates: Tensor, mu: Tensor, b1: float) -> Tensor:
    return adam_op.forward_mu(updates, mu, b1)


@_define('forward_nu')
def _forward_nu(updates: Tensor, nu: Tensor, b2: float) -> Tensor:
    return adam_op.forward_nu(updates, nu, b2)


@_define('forward_updates')
def _forward_updates(new_mu: Tensor, new_nu: Tensor, b1: float, b2: float, eps: float,
                     eps_root: float, count: int) -> Tensor:
    return adam_op.forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count)


@_define('backward_mu')
def _backward_mu(dmu: Tensor, updates: Tensor, mu: Tensor, b1: float) -> Tuple[Tensor, Tensor]:
    a, b = adam_op.backward_mu(dmu, updates, mu, b1)
    return a, b


@_define('backward_nu')
def _backward_nu(dnu: Tensor, updates: Tensor, nu: Tensor, b2: float) -> Tuple[Tensor, Tensor]:
    a, b = adam_op.backward_nu(dnu, updates, nu, b2)
    return a, b


@_define('backward_updates')
def _backward_updates(dupdates: Tensor, updates: Tensor, new_mu: Tensor, new_nu: Tensor,
                      b1: float, b2: float, eps_root: float, count: int) -> Tuple[Tensor, Tensor]:
    a, b = adam_op.backward_updates(dupdates, updates, new_mu, new_nu, b1, b2, eps_root, count)
    return a, b


# outputs take dtype, device and strides from the state tensor, as the native side allocates them
_forward_mu.register_fake(lambda updates, mu, b1: torch.empty_like(mu))
_forward_nu.register_fake(lambda updates, nu, b2: torch.empty_like(nu))
_forward_updates.register_fake(
    lambda new_mu, new_nu, b1, b2, eps, eps_root, count: torch.empty_like(new_mu))
_backward_mu.register_fake(
    lambda dmu, updates, mu, b1: (torch.empty_like(mu), torch.empty_like(mu)))
_backward_nu.register_fake(
    lambda dnu, updates, nu, b2: (torch.empty_like(nu), torch.empty_like(nu)))
_backward_updates.register_fake(
    lambda dupdates, updates, new_mu, new_nu, b1, b2, eps_root, count:
    (torch.empty_like(new_mu), torch.empty_like(new_mu)))


# ---- lists ----------------------------------------------------------------------------------


@_define('forward_multi_', ('updates', 'mu', 'nu'))
def _forward_multi_(updates: List[Tensor], mu: List[Tensor], nu: List[Tensor], b1: float,
                    b2: float, eps: float, eps_root: float, count: int) -> None:
    adam_op.forward_multi_(updates, mu, nu, b1, b2, eps, eps_root, count)


@_define('fused_step_multi_', ('params', 'updates', 'mu', 'nu'))
def _fused_step_multi_(params: List[Tensor], updates: List[Tensor], mu: List[Tensor],
                       nu: List[Tensor], b1: float, b2: float, eps: float, eps_root: float,
                       count: int, lr: float, maximize: bool, write_updates: bool,
                       weight_decay: float, decoupled: bool) -> None:
    adam_op.fused_step_multi_(params, updates, mu, nu, b1, b2, eps, eps_root, count, lr,
                              maximize=maximize, write_updates=write_updates,
                              weight_decay=weight_decay, decoupled=decoupled)


# ---- the step number on the device ----------------------------------------------------------


@_define('count_advance_', ('count',))
def _count_advance_(count: Tensor) -> None:
    adam_op.count_advance_(count)


@_define('forward_multi_devcount_', ('updates', 'mu', 'nu'))
def _forward_multi_devcount_(updates: List[Tensor], mu: List[Tensor], nu: List[Tensor], b1: float,
                             b2: float, eps: float, eps_root: float, bias_rows: Tensor,
                             first_count: int, count: Tensor) -> None:
    adam_op.forward_multi_devcount_(updates, mu, nu, b1, b2, eps, eps_root, bias_rows,
                                    first_count, count)


@_define('fused_step_multi_devcount_', ('params', 'updates', 'mu', 'nu'))
def _fused_step_multi_devcount_(params: List[Tensor], updates: List[Tensor], mu: List[Tensor],
                                nu: List[Tensor], b1: float, b2: float, eps: float,
                                eps_root: float, bias_rows: Tensor, first_count: int,
                                count: Tensor, lr: float, maximize: bool, write_updates: bool,
                                weight_decay: float, decoupled: bool) -> None:
    adam_op.fused_step_multi_devcount_(params, updates, mu, nu, b1, b2, eps, eps_root, bias_rows,
                                       first_count, count, lr, maximize=maximize,
                                       write_updates=write_updates, weight_decay=weight_decay,
                                       decoupled=decoupled)


# ---- one calling convention for both routes -------------------------------------------------


class dispatch:  # noqa: N801 - used as a namespace
    """The functions of `torchopt_amd._C.adam_op`, routed through the registered operators while
    `torch.compile` is tracing and called directly otherwise."""

    @staticmethod
    def forward_(updates, mu, nu, b1, b2, eps, eps_root, count):
        if torch.compiler.is_compiling():
            torch.ops.torchopt_amd.forward_(updates, mu, nu, b1, b2, eps, eps_root, count)
            return [updates, mu, nu]
        return adam_op.forward_(updates, mu, nu, b1, b2, eps, eps_root, count)

    @staticmethod
    def forward_mu(updates, mu, b1):
        if torch.compiler.is_compiling():
            return torch.ops.torchopt_amd.forward_mu(updates, mu, b1)
        return adam_op.forward_mu(updates, mu, b1)

    @staticmethod
    def forward_nu(updates, nu, b2):
        if torch.compiler.is_compiling():
            return torch.ops.torchopt_amd.forward_nu(updates, nu, b2)
        return adam_op.forward_nu(updates, nu, b2)

    @staticmethod
    def forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count):
        if torch.compiler.is_compiling():
            return torch.ops.torchopt_amd.forward_updates(new_mu, new_nu, b1, b2, eps, eps_root,
                                                          count)
        return adam_op.forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count)

    @staticmethod
    def backward_mu(dmu, updates, mu, b1):
        if torch.compiler.is_compiling():
            return torch.ops.torchopt_amd.backward_mu(dmu, updates, mu, b1)
        return adam_op.backward_mu(dmu, updates, mu, b1)

    @staticmethod
    def backward_nu(dnu, updates, nu, b2):
        if torch.compiler.is_compiling():
            return torch.ops.torchopt_amd.backward_nu(dnu, updates, nu, b2)
        return adam_op.backward_nu(dnu, updates, nu, b2)

    @staticmethod
    def backward_updates(dupdates, updates, new_mu, new_nu, b1, b2, eps_root, count):
        if torch.compiler.is_compiling():
            return torch.ops.torchopt_amd.backward_updates(dupdates, updates, new_mu, new_nu, b1,
                                                           b2, eps_root, count)
        return adam_op.backward_updates(dupdates, updates, new_mu, new_nu, b1, b2, eps_root, count)
