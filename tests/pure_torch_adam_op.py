"""The seven functions of `torchopt_amd._C.adam_op` written as ordinary tensor expressions.

The reference keeps such a module as the import fallback for a build without its C++ extension
(/root/reference/torchopt/accelerated_op/_src/adam_op.py:28-130, picked at
/root/reference/torchopt/accelerated_op/adam_op.py:27-30).  Here it is a test aid, kept with the
tests and outside the package: `torchopt_amd` refuses to import without its HIP library and has
nothing to fall back on.  It exists for what the reference's fallback is also good for -- a
statement of the mathematics that runs on any device PyTorch serves, to read and to check the
native op against (tests/test_src_statement.py).

Same names, argument order and return shapes as the native functions.  Results agree with the
native op closely, not bit for bit: PyTorch divides by the bias correction where the native op
multiplies by its reciprocal, fuses products into sums, and takes (1 - b) from Python's double
where the native op forms it in the element type (float32: 1.0f - 0.999f is 4.7e-5 above 0.001).
"""

from __future__ import annotations

from typing import Tuple

import torch
from torch import Tensor


def _first_moment(g: Tensor, mu: Tensor, b1: float) -> Tensor:
    return torch.lerp(g, mu, b1)  # g + b1 (mu - g) = b1 mu + (1 - b1) g


def _second_moment(g: Tensor, nu: Tensor, b2: float) -> Tensor:
    return torch.lerp(g * g, nu, b2)


def _bias(b: float, count: int) -> float:
    return 1.0 - b ** count


def _direction(new_mu: Tensor, new_nu: Tensor, b1: float, b2: float, eps: float, eps_root: float,
               count: int) -> Tensor:
    root = torch.sqrt(new_nu / _bias(b2, count) + eps_root)
    return (new_mu / _bias(b1, count)) / (root + eps)


def forward_(updates: Tensor, mu: Tensor, nu: Tensor, b1: float, b2: float, eps: float,
             eps_root: float, count: int) -> Tuple[Tensor, Tensor, Tensor]:
    """One Adam step in place: `mu`, `nu` become the new moments, `updates` the step direction."""
    mu.copy_(_first_moment(updates, mu, b1))
    nu.copy_(_second_moment(updates, nu, b2))
    updates.copy_(_direction(mu, nu, b1, b2, eps, eps_root, count))
    return updates, mu, nu


def forward_mu(updates: Tensor, mu: Tensor, b1: float) -> Tensor:
    return _first_moment(updates, mu, b1)


def forward_nu(updates: Tensor, nu: Tensor, b2: float) -> Tensor:
    return _second_moment(updates, nu, b2)


def forward_updates(new_mu: Tensor, new_nu: Tensor, b1: float, b2: float, eps: float,
                    eps_root: float, count: int) -> Tensor:
    return _direction(new_mu, new_nu, b1, b2, eps, eps_root, count)


def backward_mu(dmu: Tensor, updates: Tensor, mu: Tensor, b1: float) -> Tuple[Tensor, Tensor]:
    """Gradients of `forward_mu` with respect to (updates, mu)."""
    return dmu * (1.0 - b1), dmu * b1


def backward_nu(dnu: Tensor, updates: Tensor, nu: Tensor, b2: float) -> Tuple[Tensor, Tensor]:
    """Gradients of `forward_nu` with respect to (updates, nu)."""
    return dnu * updates * (2.0 * (1.0 - b2)), dnu * b2


def backward_updates(dupdates: Tensor, updates: Tensor, new_mu: Tensor, new_nu: Tensor, b1: float,
                     b2: float, eps_root: float, count: int) -> Tuple[Tensor, Tensor]:
    """Gradients of `forward_updates` with respect to (new_mu, new_nu), from its OUTPUT: with
    r = updates / new_mu = 1 / ((1 - b1^t) (sqrt(nu_hat + eps_root) + eps)),
        d/d new_mu = dupdates r,
        d/d new_nu = -dupdates updates ((1 - b1^t) r)^2 / (2 (1 - b2^t + eps_root)),
    and both zero where new_mu is zero (the native op skips those elements)."""
    ratio = updates / new_mu
    scaled = ratio * _bias(b1, count)
    d_mu = dupdates * ratio
    d_nu = dupdates * updates * scaled * scaled * (-0.5 / (_bias(b2, count) + eps_root))
    dead = new_mu == 0
    zero = torch.zeros((), dtype=d_mu.dtype, device=d_mu.device)
    return torch.where(dead, zero, d_mu), torch.where(dead, zero, d_nu)
