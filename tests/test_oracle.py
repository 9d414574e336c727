"""The CPU oracle is pinned here, on CPU, before anything is compared with it on the GPU.

Three independent statements of the arithmetic must agree bit for bit:
  1. the golden vectors written by the reference's own compiled CPU op (tests/golden);
  2. the plain-C restatement (oracle/adam_oracle.c) -- the oracle the GPU tests use;
  3. the NumPy one-rounding-per-operation specification (oracle/adam_spec.py);
and, where oracle/_ref has been built, 4. the compiled reference itself on fresh inputs.
Closed forms and invariants that the mathematics fixes come last; each is chosen so that a
plausible slip (dropped term, wrong sign, swapped operand, fused multiply-add, scalar rounded
at the wrong point) breaks it.
"""

from __future__ import annotations

import math

import numpy as np
import pytest

from conftest import assert_bit_equal, hyper_of, load_golden
from oracle import adam_oracle as O
from oracle import adam_spec as S

DTYPES = [np.float32, np.float64]
TAG = {np.float32: 'f32', np.float64: 'f64', np.float16: 'f16', 'bf16': 'bf16'}


def _cases(dtype):
    return sorted(load_golden(TAG[dtype]).items())


def _ids(dtype):
    return [f'{TAG[dtype]}-{name}' for name, _ in _cases(dtype)]


GOLDEN_DTYPES = [np.float32, np.float64, np.float16, 'bf16']
ALL_CASES = [(dt, name, case) for dt in GOLDEN_DTYPES for name, case in _cases(dt)]
ALL_IDS = [f'{TAG[dt]}-{name}' for dt, name, _ in ALL_CASES]


@pytest.mark.parametrize('dtype,name,case', ALL_CASES, ids=ALL_IDS)
@pytest.mark.parametrize('impl', [O, S], ids=['c_oracle', 'numpy_spec'])
def test_against_reference_golden(impl, dtype, name, case):
    if impl is S and dtype == 'bf16':
        pytest.skip('NumPy has no bfloat16; the spec covers float16, float32, float64')
    b1, b2, eps, eps_root, count = hyper_of(case)
    u, mu, nu = case['updates'], case['mu'], case['nu']
    with np.errstate(all='ignore'):
        assert_bit_equal(impl.forward_mu(u, mu, b1), case['new_mu'], 'forward_mu')
        assert_bit_equal(impl.forward_nu(u, nu, b2), case['new_nu'], 'forward_nu')
        assert_bit_equal(
            impl.forward_updates(case['new_mu'], case['new_nu'], b1, b2, eps, eps_root, count),
            case['new_updates'], 'forward_updates')
        iu, im, iv = impl.forward_inplace(u.copy(), mu.copy(), nu.copy(), b1, b2, eps, eps_root,
                                          count)
        assert_bit_equal(iu, case['inplace_updates'], 'forward_ updates')
        assert_bit_equal(im, case['inplace_mu'], 'forward_ mu')
        assert_bit_equal(iv, case['inplace_nu'], 'forward_ nu')
        du, dm = impl.backward_mu(case['dmu'], b1)
        assert_bit_equal(du, case['bmu_dupdates'], 'backward_mu dupdates')
        assert_bit_equal(dm, case['bmu_dmu'], 'backward_mu dmu')
        du, dn = impl.backward_nu(case['dnu'], u, b2)
        assert_bit_equal(du, case['bnu_dupdates'], 'backward_nu dupdates')
        assert_bit_equal(dn, case['bnu_dnu'], 'backward_nu dnu')
        dm, dn = impl.backward_updates(case['dupdates'], case['new_updates'], case['new_mu'],
                                       b1, b2, eps_root, count)
        assert_bit_equal(dm, case['bup_dnew_mu'], 'backward_updates dnew_mu')
        assert_bit_equal(dn, case['bup_dnew_nu'], 'backward_updates dnew_nu')


@pytest.mark.parametrize('dtype', GOLDEN_DTYPES, ids=['f32', 'f64', 'f16', 'bf16'])
def test_golden_internal_consistency(dtype):
    """In the reference's own outputs the fused step equals the three split ops chained."""
    for name, case in _cases(dtype):
        assert_bit_equal(case['inplace_mu'], case['new_mu'], name)
        assert_bit_equal(case['inplace_nu'], case['new_nu'], name)
        assert_bit_equal(case['inplace_updates'], case['new_updates'], name)


def _rand(dtype, n, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(n).astype(dtype), (0.1 * rng.standard_normal(n)).astype(dtype),
            np.abs(0.01 * rng.standard_normal(n)).astype(dtype))


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
@pytest.mark.parametrize('n', [0, 1, 3, 999, 1000, 1001, 4097, 300_007])
def test_c_oracle_equals_numpy_spec(dtype, n):
    """Sizes on both sides of the serial/OpenMP switch; threads must not change a bit."""
    u, mu, nu = _rand(dtype, n, 11 + n)
    rng = np.random.default_rng(n)
    d1, d2, d3 = (rng.standard_normal(n).astype(dtype) for _ in range(3))
    for b1, b2, eps, eps_root, count in [(0.9, 0.999, 1e-8, 0.0, 1), (0.9, 0.999, 1e-8, 1e-8, 5),
                                         (0.8, 0.95, 1e-6, 1e-10, 77)]:
        su, sm, sv = S.forward_inplace(u, mu, nu, b1, b2, eps, eps_root, count)
        ou, om, ov = O.forward_inplace(u.copy(), mu.copy(), nu.copy(), b1, b2, eps, eps_root,
                                       count)
        for a, b, w in ((ou, su, 'u'), (om, sm, 'mu'), (ov, sv, 'nu')):
            assert_bit_equal(a, b, f'forward_ {w}')
        assert_bit_equal(O.forward_mu(u, mu, b1), sm)
        assert_bit_equal(O.forward_nu(u, nu, b2), sv)
        assert_bit_equal(O.forward_updates(sm, sv, b1, b2, eps, eps_root, count), su)
        for a, b in zip(O.backward_mu(d1, b1), S.backward_mu(d1, b1)):
            assert_bit_equal(a, b, 'backward_mu')
        for a, b in zip(O.backward_nu(d2, u, b2), S.backward_nu(d2, u, b2)):
            assert_bit_equal(a, b, 'backward_nu')
        sm0 = sm.copy()
        if n:
            sm0[::5] = 0
        for a, b in zip(O.backward_updates(d3, su, sm0, b1, b2, eps_root, count),
                        S.backward_updates(d3, su, sm0, b1, b2, eps_root, count)):
            assert_bit_equal(a, b, 'backward_updates')


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
def test_c_oracle_equals_compiled_reference(dtype):
    """Fresh inputs, a size that gives the reference several OpenMP threads."""
    ref = O.load_reference()
    if ref is None:
        pytest.skip('oracle/_ref not built (needs the reference sources; `make -C oracle ref`)')
    import torch

    n = 1_000_003
    u, mu, nu = _rand(dtype, n, 5)
    rng = np.random.default_rng(6)
    d1, d2, d3 = (rng.standard_normal(n).astype(dtype) for _ in range(3))
    tn = torch.from_numpy
    op = ref.adam_op
    for b1, b2, eps, eps_root, count in [(0.9, 0.999, 1e-8, 0.0, 10), (0.9, 0.999, 1e-8, 1e-8, 3)]:
        ru, rm, rv = (x.copy() for x in (u, mu, nu))
        op.forward_(tn(ru), tn(rm), tn(rv), b1, b2, eps, eps_root, count)
        ou, om, ov = O.forward_inplace(u.copy(), mu.copy(), nu.copy(), b1, b2, eps, eps_root,
                                       count)
        assert_bit_equal(ou, ru), assert_bit_equal(om, rm), assert_bit_equal(ov, rv)
        assert_bit_equal(O.forward_mu(u, mu, b1), op.forward_mu(tn(u), tn(mu), b1).numpy())
        assert_bit_equal(O.forward_nu(u, nu, b2), op.forward_nu(tn(u), tn(nu), b2).numpy())
        assert_bit_equal(O.forward_updates(rm, rv, b1, b2, eps, eps_root, count),
                         op.forward_updates(tn(rm), tn(rv), b1, b2, eps, eps_root, count).numpy())
        for a, b in zip(O.backward_mu(d1, b1), op.backward_mu(tn(d1), tn(u), tn(mu), b1)):
            assert_bit_equal(a, b.numpy())
        for a, b in zip(O.backward_nu(d2, u, b2), op.backward_nu(tn(d2), tn(u), tn(nu), b2)):
            assert_bit_equal(a, b.numpy())
        rm0 = rm.copy()
        rm0[::9] = 0
        for a, b in zip(O.backward_updates(d3, ru, rm0, b1, b2, eps_root, count),
                        op.backward_updates(tn(d3), tn(ru), tn(rm0), tn(rv), b1, b2, eps_root,
                                            count)):
            assert_bit_equal(a, b.numpy())


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
@pytest.mark.parametrize('maximize', [False, True])
@pytest.mark.parametrize('decay', ['none', 'l2', 'decoupled'])
def test_fused_step_is_the_reference_chain(dtype, maximize, decay):
    """The classic in-place step of the reference is a chain of passes: [neg_],
    [add_(p, alpha=wd)] (alias/utils.py:113-122), forward_, [add_(p, alpha=wd)]
    (transform/add_decayed_weights.py:232-239), mul_(-lr) (transform/scale.py:93-98) and add_
    (update.py:71-74).  Run exactly those calls on CPU tensors -- forward_ from the compiled
    reference where it is built, else from the pinned C oracle -- and compare the one-pass
    oracle with them."""
    import torch

    ref = O.load_reference()
    rng = np.random.default_rng(31)
    wd = 0.0 if decay == 'none' else 0.03
    for n, lr, count, eps_root in [(1, 1e-3, 1, 0.0), (1003, 1e-3, 7, 0.0), (200_003, 0.05, 1000, 1e-8)]:
        g, m, v = _rand(dtype, n, n)
        p = rng.standard_normal(n).astype(dtype)
        tg, tm, tv, tp = (torch.from_numpy(x.copy()) for x in (g, m, v, p))
        if maximize:
            tg.neg_()
        if decay == 'l2':
            tg.add_(tp, alpha=wd)
        if ref is not None:
            ref.adam_op.forward_(tg, tm, tv, 0.9, 0.999, 1e-8, eps_root, count)
        else:
            O.forward_inplace(tg.numpy(), tm.numpy(), tv.numpy(), 0.9, 0.999, 1e-8, eps_root, count)
        if decay == 'decoupled':
            tg.add_(tp, alpha=wd)
        tg.mul_(-lr)
        tp.add_(tg)
        for write_updates in (True, False):
            op, og, om, ov = p.copy(), g.copy(), m.copy(), v.copy()
            O.fused_step(op, og, om, ov, 0.9, 0.999, 1e-8, eps_root, count, lr, maximize,
                         write_updates, wd, decay == 'decoupled')
            assert_bit_equal(op, tp.numpy(), 'params')
            assert_bit_equal(om, tm.numpy(), 'mu')
            assert_bit_equal(ov, tv.numpy(), 'nu')
            assert_bit_equal(og, tg.numpy() if write_updates else g, 'updates')


def test_weight_decay_is_a_fused_multiply_add():
    """Tensor.add_(p, alpha=wd) rounds once; g + round(wd*p) differs on a few percent of random
    float32 inputs, so the distinction is observable and the oracle must be on the fma side."""
    import torch

    rng = np.random.default_rng(2)
    n = 50_000
    g, p = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    torch_way = torch.from_numpy(g.copy()).add_(torch.from_numpy(p), alpha=0.01).numpy()
    two_roundings = g + np.float32(0.01) * p
    assert (torch_way != two_roundings).sum() > 100
    # the oracle's decayed gradient shows in mu after one step from mu = 0 with b1 = 0: mu' = g'
    mu = np.zeros(n, np.float32)
    O.fused_step(p.copy(), g.copy(), mu, np.zeros(n, np.float32), 0.0, 0.0, 1e-8, 0.0, 1, 1e-3,
                 False, False, 0.01, False)
    assert_bit_equal(mu, torch_way)


def test_fused_step_scales_by_the_rounded_learning_rate():
    """In float32 the step is u * float32(-lr), not float32(u * -lr in double): pick lr = 0.1."""
    one = np.ones(8, np.float32)
    p = np.zeros(8, np.float32)
    g = one.copy()
    O.fused_step(p, g, np.zeros(8, np.float32), np.zeros(8, np.float32), 0.9, 0.999, 0.0, 0.0, 1,
                 0.1, False, True)
    u = O.forward_inplace(one.copy(), np.zeros(8, np.float32), np.zeros(8, np.float32), 0.9, 0.999,
                          0.0, 0.0, 1)[0]
    assert_bit_equal(g, u * np.float32(-0.1))
    assert_bit_equal(p, np.float32(0) + u * np.float32(-0.1))


def test_half_conversions_against_numpy_and_torch():
    """The oracle's own float<->half and float->bfloat16 conversions: every half value, every
    midpoint between neighbouring halves (ties to even), the overflow threshold, subnormals."""
    import torch

    L = O.lib()
    halves = np.arange(65536, dtype=np.uint16)
    as_f32 = halves.view(np.float16).astype(np.float32)
    back = np.array([L.oracle_f32_from_f16(int(h)) for h in halves], dtype=np.float32)
    assert_bit_equal(back, as_f32, 'half -> float, all 65536 values')
    fin = np.isfinite(as_f32[:-1]) & np.isfinite(as_f32[1:])
    mids = ((as_f32[:-1].astype(np.float64) + as_f32[1:].astype(np.float64)) / 2)[fin]
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        mids.astype(np.float32),
        np.array([65504, 65519.996, 65520, 65536, 1e30, -65520, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32),
        (rng.standard_normal(20000) * 1e-6).astype(np.float32),
        rng.standard_normal(20000).astype(np.float32),
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    xs = xs[~np.isnan(xs)]
    with np.errstate(all='ignore'):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.oracle_f16_from_f32(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.oracle_bf16_from_f32(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want) and np.array_equal(O.bf16_bits(xs), want)
    assert L.oracle_bf16_from_f32(float('nan')) == 0x7fc0
    assert L.oracle_f16_from_f32(float('nan')) & 0x7fff == 0x7e00


def test_half_division_stays_in_float_until_the_end():
    """mu_hat / (sqrt(.) + eps) with half data: the square root, the sum and the quotient run in
    float and are rounded once.  Rounding the root or the denominator to half first changes
    thousands of results on random data, so the distinction is observable."""
    rng = np.random.default_rng(4)
    n = 20000
    m = (0.1 * rng.standard_normal(n)).astype(np.float16)
    v = np.abs(0.01 * rng.standard_normal(n)).astype(np.float16)
    got = O.forward_updates(m, v, 0.9, 0.999, 1e-3, 1e-4, 5)
    f, h = np.float32, np.float16
    c1, c2 = h(f(1 / (1 - 0.9 ** 5))), h(f(1 / (1 - 0.999 ** 5)))
    mh, vh = m * c1, v * c2
    t = vh + h(f(1e-4))
    kept = (mh.astype(f) / (np.sqrt(t.astype(f)) + f(h(f(1e-3))))).astype(h)
    rounded = mh / (np.sqrt(t) + h(f(1e-3)))
    assert_bit_equal(got, kept)
    assert (kept != rounded).sum() > 100


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
def test_low_precision_oracle_equals_compiled_reference(fmt):
    ref = O.load_reference()
    if ref is None:
        pytest.skip('oracle/_ref not built (needs the reference sources; `make -C oracle ref`)')
    import torch

    tdt = torch.float16 if fmt == 'f16' else torch.bfloat16
    rng = np.random.default_rng(8)
    n = 200_003

    def tens(a):
        return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(tdt)

    def arr(t):
        if fmt == 'bf16':
            return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()
        return t.numpy().copy()

    g, m = tens(rng.standard_normal(n)), tens(0.1 * rng.standard_normal(n))
    v = tens(np.abs(0.01 * rng.standard_normal(n)))
    d1, d2, d3 = (tens(rng.standard_normal(n)) for _ in range(3))
    op = ref.adam_op
    for b1, b2, eps, er, count in [(0.9, 0.999, 1e-3, 0.0, 10), (0.9, 0.999, 1e-3, 1e-4, 3)]:
        tg, tm, tv = g.clone(), m.clone(), v.clone()
        op.forward_(tg, tm, tv, b1, b2, eps, er, count)
        og, om, ov = arr(g), arr(m), arr(v)
        O.forward_inplace(og, om, ov, b1, b2, eps, er, count)
        assert_bit_equal(og, arr(tg)), assert_bit_equal(om, arr(tm)), assert_bit_equal(ov, arr(tv))
        for a, b in zip(O.backward_mu(arr(d1), b1), op.backward_mu(d1, g, m, b1)):
            assert_bit_equal(a, arr(b))
        for a, b in zip(O.backward_nu(arr(d2), arr(g), b2), op.backward_nu(d2, g, v, b2)):
            assert_bit_equal(a, arr(b))
        tm0 = tm.clone()
        tm0[::9] = 0
        for a, b in zip(O.backward_updates(arr(d3), arr(tg), arr(tm0), b1, b2, er, count),
                        op.backward_updates(d3, tg, tm0, tv, b1, b2, er, count)):
            assert_bit_equal(a, arr(b))


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
@pytest.mark.parametrize('maximize', [False, True])
def test_low_precision_fused_step_is_the_reference_chain(fmt, maximize):
    """The classic in-place step on 16-bit tensors, without weight decay: the very calls the
    reference's chains make -- [neg_], forward_ (compiled reference where it is built, else the
    pinned C oracle), mul_(-lr), add_ -- on 16-bit CPU tensors, against the one-pass oracle.  Pins
    how torch treats the Python scalar there: -lr acts as a float, not as a 16-bit value (0.05 is
    not representable in either format)."""
    import torch

    ref = O.load_reference()
    tdt = torch.float16 if fmt == 'f16' else torch.bfloat16
    rng = np.random.default_rng(41)

    def tens(a):
        return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(tdt)

    def arr(t):
        if fmt == 'bf16':
            return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()
        return t.numpy().copy()

    for n, lr, count, eps_root in [(1, 1e-3, 1, 0.0), (1003, 1e-3, 7, 0.0), (200_003, 0.05, 1000, 1e-4)]:
        g, m = tens(rng.standard_normal(n)), tens(0.1 * rng.standard_normal(n))
        v, p = tens(np.abs(0.01 * rng.standard_normal(n))), tens(rng.standard_normal(n))
        tg, tm, tv, tp = g.clone(), m.clone(), v.clone(), p.clone()
        if maximize:
            tg.neg_()
        if ref is not None:
            ref.adam_op.forward_(tg, tm, tv, 0.9, 0.999, 1e-3, eps_root, count)
        else:
            og, om, ov = arr(tg), arr(tm), arr(tv)
            O.forward_inplace(og, om, ov, 0.9, 0.999, 1e-3, eps_root, count)
            for t, a in ((tg, og), (tm, om), (tv, ov)):
                t.copy_(torch.from_numpy(a.view(np.int16)).view(tdt) if fmt == 'bf16'
                        else torch.from_numpy(a))
        tg.mul_(-lr)
        tp.add_(tg)
        for write_updates in (True, False):
            op, og, om, ov = arr(p), arr(g), arr(m), arr(v)
            O.fused_step(op, og, om, ov, 0.9, 0.999, 1e-3, eps_root, count, lr, maximize,
                         write_updates)
            assert_bit_equal(om, arr(tm), 'mu')
            assert_bit_equal(ov, arr(tv), 'nu')
            assert_bit_equal(og, arr(tg) if write_updates else arr(g), 'updates')
            assert_bit_equal(op, arr(tp), 'params')
    with pytest.raises(ValueError, match='no weight decay on 16-bit'):
        O.fused_step(arr(p), arr(g), arr(m), arr(v), 0.9, 0.999, 1e-3, 0.0, 1, 1e-3, False, True,
                     0.01, True)


def test_low_precision_step_keeps_its_learning_rate_in_float():
    """-lr = -0.05 is not representable in float16 or bfloat16: a step scaled by the rounded scalar
    differs from torch's mul_(-0.05) on a fifth of random elements and more, one scaled by the
    float scalar on none -- so the distinction is observable and the oracle is on torch's side."""
    import torch

    rng = np.random.default_rng(5)
    u = rng.standard_normal(200_000).astype(np.float32)
    for tdt in (torch.float16, torch.bfloat16):
        t = torch.from_numpy(u).to(tdt)
        torch_way = t.clone().mul_(-0.05)
        rounded_scalar = (t.float() * torch.tensor(-0.05).to(tdt).float()).to(tdt)
        assert (torch_way != rounded_scalar).sum() > 20_000
        float_scalar = (t.float() * torch.tensor(-0.05, dtype=torch.float32)).to(tdt)
        assert torch.equal(torch_way, float_scalar)


def test_weight_decay_on_16_bit_cpu_tensors_is_not_one_arithmetic():
    """Why the 16-bit step leaves weight decay out: torch.Tensor.add_(p, alpha=wd) on a bfloat16
    CPU tensor rounds alpha to bfloat16 and works in float in its vectorized body, but rounds the
    product to bfloat16 first in its scalar tail -- the same operands give different results
    depending on where in the tensor they lie."""
    import torch

    a = torch.tensor(-0.49609375, dtype=torch.bfloat16)
    b = torch.tensor(1.984375, dtype=torch.bfloat16)
    n = 4096 + 1  # the last element falls into the scalar tail
    ta, tb = a.repeat(n), b.repeat(n)
    out = ta.clone().add_(tb, alpha=0.03)
    body, tail = out[0].item(), out[-1].item()
    if body == tail:
        pytest.skip('this build of torch evaluates body and tail alike')
    assert {body, tail} == {-0.435546875, -0.4375}


# ---------------------------------------------------------------------------------------------
# What the mathematics fixes
# ---------------------------------------------------------------------------------------------


def test_host_scalars_closed_form():
    for b1, b2, er, c in [(0.9, 0.999, 0.0, 1), (0.9, 0.999, 1e-8, 5), (0.5, 0.25, 0.0, 3)]:
        c1, c2, p1, q2 = O.host_scalars(b1, b2, er, c)
        assert c1 == 1.0 / (1.0 - math.pow(b1, c))
        assert c2 == 1.0 / (1.0 - math.pow(b2, c))
        assert p1 == 1.0 - math.pow(b1, c)
        assert q2 == 1.0 / (1.0 - math.pow(b2, c) + er)
    # exactly representable: b = 0.5, count = 3 -> 1/(1 - 1/8) and 7/8
    c1, _, p1, _ = O.host_scalars(0.5, 0.5, 0.0, 3)
    assert p1 == 0.875 and c1 == 1.0 / 0.875
    assert S.host_scalars(0.9, 0.999, 1e-8, 1000) == O.host_scalars(0.9, 0.999, 1e-8, 1000)


def test_fp32_one_minus_beta_is_formed_in_float():
    """1.0f - 0.999f is 9.9998713e-4, not float(1 - 0.999) = 1.00000005e-3: with nu = 0 the
    new nu is exactly that factor times g*g (g = 1)."""
    one = np.ones(4, np.float32)
    zero = np.zeros(4, np.float32)
    out = O.forward_nu(one, zero, 0.999)
    want = np.float32(1) - np.float32(0.999)
    assert out[0] == want and out[0] != np.float32(1.0 - 0.999)
    out = O.forward_mu(one, zero, 0.9)
    assert out[0] == np.float32(1) - np.float32(0.9) and out[0] != np.float32(1.0 - 0.9)


def test_no_fused_multiply_add():
    """b1*m + (1-b1)*g with b1 = 0.5: choose m, g whose products are inexact in float so that a
    fused multiply-add (one rounding) and mul-then-add (two roundings) differ."""
    rng = np.random.default_rng(3)
    m = rng.standard_normal(4096).astype(np.float32)
    g = (-m * np.float32(1 + 2 ** -12)).astype(np.float32)  # near-cancellation
    b1 = 0.7
    out = O.forward_mu(g, m, b1)
    beta = np.float32(b1)
    two_step = (beta * m) + ((np.float32(1) - beta) * g)
    fused = (np.float64(beta) * m.astype(np.float64)
             + np.float64(np.float32(1) - beta) * g.astype(np.float64)).astype(np.float32)
    assert_bit_equal(out, two_step)
    assert np.any(two_step != fused)  # the case does discriminate


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
def test_first_step_from_zero_state_is_sign(dtype):
    """count = 1, mu = nu = 0, eps_root = 0: update = g / (|g| + eps) ~ sign(g)."""
    g = np.array([3.0, -2.0, 0.5, -1e-3, 1e3], dtype)
    z = np.zeros_like(g)
    u, m, v = O.forward_inplace(g.copy(), z.copy(), z.copy(), 0.9, 0.999, 1e-8, 0.0, 1)
    tol = 8 * np.finfo(dtype).eps
    # in float, 1.0f - 0.999f is off from 0.001 by 1.3e-5 relative, and c2 = 1000 undoes it only
    # in exact arithmetic: the step is sign(g) to half of that
    np.testing.assert_allclose(u, g / (np.abs(g) + dtype(1e-8)),
                               rtol=1e-5 if dtype == np.float32 else tol)
    np.testing.assert_allclose(m, (1 - 0.9) * g, rtol=tol)
    np.testing.assert_allclose(v, (1 - 0.999) * g * g, rtol=2e-5 if dtype == np.float32 else tol)


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
def test_forward_matches_high_precision_formula(dtype):
    """Against the textbook formula evaluated in extended precision."""
    u, mu, nu = _rand(dtype, 2000, 21)
    b1, b2, eps, er, c = 0.9, 0.999, 1e-8, 1e-8, 7
    ou, om, ov = O.forward_inplace(u.copy(), mu.copy(), nu.copy(), b1, b2, eps, er, c)
    L = np.longdouble
    beta1, beta2 = L(dtype(b1)), L(dtype(b2))
    m1 = beta1 * L(mu) + (1 - beta1) * L(u)
    v1 = beta2 * L(nu) + (1 - beta2) * L(u) * L(u)
    up = (m1 / (1 - L(b1) ** c)) / (np.sqrt(v1 / (1 - L(b2) ** c) + L(er)) + L(eps))
    e = np.finfo(dtype).eps
    # cancellation in m1 costs absolute, not relative, accuracy
    np.testing.assert_allclose(om.astype(L), m1, rtol=0, atol=4 * e * (np.abs(mu).max() + 1))
    np.testing.assert_allclose(ov.astype(L), v1, rtol=8 * e)
    np.testing.assert_allclose(ou.astype(L), up, rtol=0, atol=64 * e * np.abs(up).max())


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
def test_backward_mu_nu_are_the_analytic_vjps(dtype):
    """d(new_mu)/d(updates) = 1-b1, d/d(mu) = b1; d(new_nu)/d(updates) = 2(1-b2)g, d/d(nu) = b2
    -- checked against central differences of the oracle's own forward in float64."""
    rng = np.random.default_rng(5)
    n = 64
    g, m, v = _rand(np.float64, n, 9)
    ct = rng.standard_normal(n)
    h = 1e-6
    fd_g = (O.forward_mu(g + h, m, 0.9) - O.forward_mu(g - h, m, 0.9)) / (2 * h) * ct
    fd_m = (O.forward_mu(g, m + h, 0.9) - O.forward_mu(g, m - h, 0.9)) / (2 * h) * ct
    du, dm = O.backward_mu(ct.astype(dtype), 0.9)
    tol = 1e-5 if dtype == np.float32 else 1e-8
    np.testing.assert_allclose(du, fd_g, rtol=tol, atol=tol)
    np.testing.assert_allclose(dm, fd_m, rtol=tol, atol=tol)
    fd_g = (O.forward_nu(g + h, v, 0.999) - O.forward_nu(g - h, v, 0.999)) / (2 * h) * ct
    fd_v = (O.forward_nu(g, v + h, 0.999) - O.forward_nu(g, v - h, 0.999)) / (2 * h) * ct
    du, dv = O.backward_nu(ct.astype(dtype), g.astype(dtype), 0.999)
    np.testing.assert_allclose(du, fd_g, rtol=10 * tol, atol=10 * tol)
    np.testing.assert_allclose(dv, fd_v, rtol=tol, atol=tol)


@pytest.mark.parametrize('dtype', DTYPES, ids=['f32', 'f64'])
def test_backward_updates_structure(dtype):
    """The reference's backward of forward_updates is a hand-derived formula, not the exact
    derivative; what is fixed: dnew_mu * new_mu == dupdates * updates (it is d*u/m), the exact
    derivative is recovered when eps = eps_root = 0, zeros of new_mu give exact +0 and NaN does
    not take the zero branch."""
    rng = np.random.default_rng(8)
    n = 512
    b1, b2, c = 0.9, 0.999, 4
    m1 = (0.1 * rng.standard_normal(n)).astype(dtype)
    v1 = np.abs(0.01 * rng.standard_normal(n)).astype(dtype) + dtype(1e-4)
    d = rng.standard_normal(n).astype(dtype)
    u = O.forward_updates(m1, v1, b1, b2, 0.0, 0.0, c)
    dm, dv = O.backward_updates(d, u, m1, b1, b2, 0.0, c)
    e = np.finfo(dtype).eps
    np.testing.assert_allclose(dm * m1, d * u, rtol=8 * e)
    # exact derivative of u = (m c1) / sqrt(v c2):  du/dm = u/m,  du/dv = -u / (2 v)
    np.testing.assert_allclose(dm, d * (u / m1), rtol=8 * e)
    np.testing.assert_allclose(dv, -d * u / (2 * v1), rtol=64 * e)
    m0 = m1.copy()
    m0[:4] = [0.0, -0.0, np.nan, 1.0]
    with np.errstate(all='ignore'):
        dm, dv = O.backward_updates(d, u, m0, b1, b2, 0.0, c)
    for out in (dm, dv):
        assert out[0] == 0 and not np.signbit(out[0])
        assert out[1] == 0 and not np.signbit(out[1])
        assert np.isnan(out[2])


def test_fp32_backward_updates_tail_runs_in_double():
    """Pick values where rounding the tail products in float (instead of one final rounding
    from double) changes the result; the oracle must match the double-tail evaluation."""
    rng = np.random.default_rng(12)
    n = 4096
    d = rng.standard_normal(n).astype(np.float32)
    u = rng.standard_normal(n).astype(np.float32)
    m1 = (0.1 * rng.standard_normal(n)).astype(np.float32) + np.float32(0.5)
    b1, b2, er, c = 0.9, 0.999, 1e-8, 5
    _, dv = O.backward_updates(d, u, m1, b1, b2, er, c)
    _, _, p1, q2 = O.host_scalars(b1, b2, er, c)
    p1, q2 = np.float32(p1), np.float32(q2)
    r = u / m1
    den = r * p1
    head = ((-d) * u) * den
    in_double = (((head.astype(np.float64) * 0.5) * np.float64(q2))
                 * den.astype(np.float64)).astype(np.float32)
    in_float = ((head * np.float32(0.5)) * q2) * den
    assert_bit_equal(dv, in_double)
    assert np.any(in_double != in_float)


def test_thread_policy():
    """min(n/1000, nprocs) threads, serial up to and including n = 1000
    (/root/reference/src/adam_op/adam_op_impl_cpu.cpp:30, 43-46)."""
    import os

    assert O.threads_for(0) == 1 and O.threads_for(1000) == 1
    assert O.threads_for(1001) == 1
    assert O.threads_for(2000) == min(2, os.cpu_count())
    assert O.threads_for(10 ** 9) >= 1
