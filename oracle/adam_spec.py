"""NumPy one-rounding-per-operation specification of the fused Adam operator.

TEST INFRASTRUCTURE, NOT PRODUCT: only tests may import this module.

It is an independent second statement of the arithmetic in
/root/reference/src/adam_op/adam_op_impl_cpu.cpp, written so that every NumPy
array operation is exactly one IEEE-754 rounding in the element type (NumPy's
float32/float64 add, multiply, divide and sqrt are correctly rounded and never
fused).  The C oracle (adam_oracle.c) must agree with it bit for bit; a
disagreement means one of the two mis-states an evaluation order, a promotion
or a rounding point.

All functions are out-of-place and return new arrays.

float16 arrays are covered too: NumPy's float16 arithmetic converts to float32, operates and
rounds back, which is what c10::Half does for an operation between two halves.  Where the
reference's expression mixes a half with a float (the square root is the float overload, so
"sqrt(.) + eps" and the division stay in float) or a double (the tail of backward_updates),
the spec widens explicitly, and every scalar goes double -> float -> half as `Half(float(x))`
does.  bfloat16 has no NumPy type and is pinned by the compiled reference and the golden
vectors only.
"""

from __future__ import annotations

import math

import numpy as np


def host_scalars(b1: float, b2: float, eps_root: float, count: int):
    """Bias-correction scalars in double (adam_op_impl_cpu.cpp:73-74, 191-192, 328-329)."""
    pb1 = math.pow(b1, float(count))
    pb2 = math.pow(b2, float(count))
    return 1.0 / (1.0 - pb1), 1.0 / (1.0 - pb2), 1.0 - pb1, 1.0 / (1.0 - pb2 + eps_root)


def _t(dtype, x):
    """Python scalar -> element type; a half is reached through float, as c10::Half(float)."""
    if np.dtype(dtype) == np.float16:
        return np.float16(np.float32(x))
    return np.dtype(dtype).type(x)


def _wide(dtype):
    """The type in which an expression mixing the element type with a float runs."""
    return np.float32 if np.dtype(dtype) == np.float16 else np.dtype(dtype).type


def forward_mu(updates: np.ndarray, mu: np.ndarray, b1: float) -> np.ndarray:
    """adam_op_impl_cpu.cpp:93-125."""
    T = updates.dtype
    beta = _t(T, b1)
    one_minus = _t(T, 1) - beta  # formed in T
    left = beta * mu
    right = one_minus * updates
    return left + right


def forward_nu(updates: np.ndarray, nu: np.ndarray, b2: float) -> np.ndarray:
    """adam_op_impl_cpu.cpp:127-160."""
    T = updates.dtype
    beta = _t(T, b2)
    one_minus = _t(T, 1) - beta
    left = beta * nu
    right = (one_minus * updates) * updates  # left-to-right
    return left + right


def forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count) -> np.ndarray:
    """adam_op_impl_cpu.cpp:162-209."""
    T = new_mu.dtype
    c1d, c2d, _, _ = host_scalars(b1, b2, eps_root, count)
    c1, c2 = _t(T, c1d), _t(T, c2d)
    W = _wide(T)
    mu_hat = new_mu * c1
    nu_hat = new_nu * c2
    with np.errstate(all='ignore'):
        root = np.sqrt((nu_hat + _t(T, eps_root)).astype(W))  # the sum is rounded to T first
        return (mu_hat.astype(W) / (root + W(_t(T, eps)))).astype(T)


def forward_inplace(updates, mu, nu, b1, b2, eps, eps_root, count):
    """adam_op_impl_cpu.cpp:32-91; returns (new_updates, new_mu, new_nu)."""
    new_mu = forward_mu(updates, mu, b1)
    new_nu = forward_nu(updates, nu, b2)
    new_updates = forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count)
    return new_updates, new_mu, new_nu


def backward_mu(dmu: np.ndarray, b1: float):
    """adam_op_impl_cpu.cpp:211-245; returns (dupdates, dmu_out)."""
    T = dmu.dtype
    beta = _t(T, b1)
    return (_t(T, 1) - beta) * dmu, beta * dmu


def backward_nu(dnu: np.ndarray, updates: np.ndarray, b2: float):
    """adam_op_impl_cpu.cpp:247-284; returns (dupdates, dnu_out)."""
    T = dnu.dtype
    beta = _t(T, b2)
    two_one_minus = _t(T, 2) * (_t(T, 1) - beta)
    return (two_one_minus * updates) * dnu, beta * dnu


def backward_updates(dupdates, updates, new_mu, b1, b2, eps_root, count):
    """adam_op_impl_cpu.cpp:286-347; returns (dnew_mu, dnew_nu)."""
    T = dupdates.dtype
    _, _, p1d, q2d = host_scalars(b1, b2, eps_root, count)
    p1, q2 = _t(T, p1d), _t(T, q2d)
    with np.errstate(all='ignore'):
        ratio = updates / new_mu
        den = ratio * p1
        dnew_mu = dupdates * ratio
        head = ((-dupdates) * updates) * den  # two roundings in T
        # the literal 0.5 is a double: the remaining products run in float64
        tail = ((head.astype(np.float64) * 0.5) * np.float64(q2)) * den.astype(np.float64)
        dnew_nu = tail.astype(_wide(T)).astype(T)  # a half is reached through float
    zero = new_mu == 0  # true for +0 and -0, false for NaN
    dnew_mu = np.where(zero, _t(T, 0), dnew_mu)
    dnew_nu = np.where(zero, _t(T, 0), dnew_nu)
    return dnew_mu, dnew_nu
