"""The plain-PyTorch statement of the operator (`tests/pure_torch_adam_op.py`)
against the CPU oracle on CPU tensors, and -- on a GPU -- against the native op.  Agreement is to
a tolerance, not bit for bit: PyTorch divides by the bias correction where the native op
multiplies by its reciprocal, and forms (1 - b) in double where the native op forms it in the
element type (tolerances: 1e-4 for float32, 1e-13 for float64, relative to the element or, where
terms cancel, to the array's largest element)."""

from __future__ import annotations

import importlib.util
import os

import numpy as np
import pytest
import torch

from oracle import adam_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, 'pure_torch_adam_op.py')


def load_statement():
    # by path: it is a test aid beside this file, not a module of the package
    spec = importlib.util.spec_from_file_location('toa_src_adam_op', SRC)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


S = load_statement()
B1, B2, EPS, EPS_ROOT = 0.9, 0.999, 1e-8, 1e-8
# float32: the native op forms (1 - b2) in float, 1.0f - 0.999f = 0.00100004673, the statement
# in Python's double, 0.001: 4.7e-5 apart, and every term that carries the factor inherits it
TOL = {np.float32: 1e-4, np.float64: 1e-13}


def draw(dtype, n, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(n).astype(dtype), (0.1 * rng.standard_normal(n)).astype(dtype),
            np.abs(0.01 * rng.standard_normal(n)).astype(dtype))


def close(got, want, dtype, what):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else got
    # sums of terms that nearly cancel carry the rounding of the terms: absolute slack at the
    # scale of the array's largest element
    finite = np.abs(want[np.isfinite(want)])
    np.testing.assert_allclose(got, want, rtol=TOL[dtype],
                               atol=TOL[dtype] * float(finite.max(initial=0.0)), err_msg=what)


@pytest.mark.parametrize('dtype', [np.float32, np.float64])
@pytest.mark.parametrize('count', [1, 3, 1000])
def test_statement_matches_the_oracle_on_cpu(dtype, count):
    g, m, v = draw(dtype, 4099, 3)
    T = torch.from_numpy
    e_m, e_v = O.forward_mu(g, m, B1), O.forward_nu(g, v, B2)
    e_u = O.forward_updates(e_m, e_v, B1, B2, EPS, EPS_ROOT, count)
    close(S.forward_mu(T(g), T(m), B1), e_m, dtype, 'forward_mu')
    close(S.forward_nu(T(g), T(v), B2), e_v, dtype, 'forward_nu')
    close(S.forward_updates(T(e_m), T(e_v), B1, B2, EPS, EPS_ROOT, count), e_u, dtype,
          'forward_updates')
    d = draw(dtype, 4099, 4)
    for got, want, name in zip(S.backward_mu(T(d[0]), T(g), T(m), B1), O.backward_mu(d[0], B1),
                               ('d updates', 'd mu')):
        close(got, want, dtype, f'backward_mu {name}')
    for got, want, name in zip(S.backward_nu(T(d[0]), T(g), T(v), B2),
                               O.backward_nu(d[0], g, B2), ('d updates', 'd nu')):
        close(got, want, dtype, f'backward_nu {name}')
    e_m0 = e_m.copy()
    e_m0[::7] = 0  # the skipped elements
    e_u0 = O.forward_updates(e_m0, e_v, B1, B2, EPS, EPS_ROOT, count)
    want = O.backward_updates(d[0], e_u0, e_m0, B1, B2, EPS_ROOT, count)
    got = S.backward_updates(T(d[0]), T(e_u0), T(e_m0), T(e_v), B1, B2, EPS_ROOT, count)
    for a, b, name in zip(got, want, ('d new_mu', 'd new_nu')):
        close(a, b, dtype, f'backward_updates {name}')
        assert np.all(a.numpy()[::7] == 0)
    u, mm, vv = T(g.copy()), T(m.copy()), T(v.copy())
    out = S.forward_(u, mm, vv, B1, B2, EPS, EPS_ROOT, count)
    assert out[0] is u and out[1] is mm and out[2] is vv
    O.forward_inplace(g, m, v, B1, B2, EPS, EPS_ROOT, count)
    for a, b, name in zip((u, mm, vv), (g, m, v), ('updates', 'mu', 'nu')):
        close(a, b, dtype, f'forward_ {name}')


@pytest.mark.gpu
@pytest.mark.parametrize('dtype', [torch.float32, torch.float64])
def test_statement_matches_the_native_op_on_the_gpu(dtype):
    from torchopt_amd._C import adam_op

    npdt = {torch.float32: np.float32, torch.float64: np.float64}[dtype]
    g, m, v = (torch.from_numpy(a).cuda() for a in draw(npdt, 100_003, 5))
    want = adam_op.forward_(g.clone(), m.clone(), v.clone(), B1, B2, EPS, EPS_ROOT, 7)
    got = S.forward_(g.clone(), m.clone(), v.clone(), B1, B2, EPS, EPS_ROOT, 7)
    for a, b, name in zip(got, want, ('updates', 'mu', 'nu')):
        close(a, b.cpu().numpy(), npdt, f'forward_ {name}')
    d = torch.from_numpy(draw(npdt, 100_003, 6)[0]).cuda()
    for a, b in zip(S.backward_updates(d, want[0], want[1], want[2], B1, B2, EPS_ROOT, 7),
                    adam_op.backward_updates(d, want[0], want[1], want[2], B1, B2, EPS_ROOT, 7)):
        close(a, b.cpu().numpy(), npdt, 'backward_updates')
