"""The drop-in boundary, end to end: the reference's OWN extension -- its pybind11 module
(/root/reference/src/extension.cpp), dispatcher (/root/reference/src/adam_op/adam_op.cpp) and CPU
op, compiled unchanged with __USE_CUDA__ -- with torchopt_amd/csrc/adam_op_impl_hip.cpp standing
where its CUDA launchers stood, linked against libtoa_adam.so (`make -C oracle dropin`).  GPU
tensors handed to that module reach this repository's kernels through the reference's own
`tensor.is_cuda()` branch; the results are held to the CPU oracle bit for bit, and the reference's
autograd wrapper logic (accelerated_op/adam_op.py:33-181) is replayed on top of it."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal, hyper_of, load_golden
from oracle import adam_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def ref_ext():
    assert torch.cuda.is_available(), 'these tests need a GPU'
    mod = O.load_dropin()
    if mod is None:
        pytest.skip('oracle/_ref/dropin was not built (needs the reference sources at build time)')
    yield mod.adam_op
    torch.cuda.synchronize()


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:  # bfloat16 bit patterns
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def host(t):
    if t.dtype == torch.bfloat16:
        return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.detach().cpu().numpy()


@pytest.mark.parametrize('tag', ['f32', 'f64', 'f16', 'bf16'])
def test_golden_vectors_through_the_reference_dispatcher(ref_ext, tag):
    for name, case in sorted(load_golden(tag).items()):
        b1, b2, eps, er, c = hyper_of(case)
        g = {k: dev(case[k]) for k in ('updates', 'mu', 'nu', 'dmu', 'dnu', 'dupdates')}
        label = f'{tag}/{name}'
        assert_bit_equal(host(ref_ext.forward_mu(g['updates'], g['mu'], b1)), case['new_mu'], label)
        assert_bit_equal(host(ref_ext.forward_nu(g['updates'], g['nu'], b2)), case['new_nu'], label)
        emu, env, eup = dev(case['new_mu']), dev(case['new_nu']), dev(case['new_updates'])
        assert_bit_equal(host(ref_ext.forward_updates(emu, env, b1, b2, eps, er, c)),
                         case['new_updates'], label)
        du, dm = ref_ext.backward_mu(g['dmu'], g['updates'], g['mu'], b1)
        assert_bit_equal(host(du), case['bmu_dupdates'], label)
        assert_bit_equal(host(dm), case['bmu_dmu'], label)
        du, dn = ref_ext.backward_nu(g['dnu'], g['updates'], g['nu'], b2)
        assert_bit_equal(host(du), case['bnu_dupdates'], label)
        assert_bit_equal(host(dn), case['bnu_dnu'], label)
        dm, dn = ref_ext.backward_updates(g['dupdates'], eup, emu, env, b1, b2, er, c)
        assert_bit_equal(host(dm), case['bup_dnew_mu'], label)
        assert_bit_equal(host(dn), case['bup_dnew_nu'], label)
        out = ref_ext.forward_(g['updates'], g['mu'], g['nu'], b1, b2, eps, er, c)
        assert isinstance(out, list) and out[0] is g['updates'] and out[1] is g['mu']
        assert_bit_equal(host(g['updates']), case['inplace_updates'], label)
        assert_bit_equal(host(g['mu']), case['inplace_mu'], label)
        assert_bit_equal(host(g['nu']), case['inplace_nu'], label)


def test_reference_surface_conventions(ref_ext):
    """Keyword names (with backward_nu's `b1`), count as a 0-dim device tensor, the availability
    probe's aliased call, the other devices' errors: all the reference's own code."""
    a = torch.ones((), device='cuda')
    out = ref_ext.forward_(a, a, a, 0.9, 0.999, 1e-8, 0.0, 1)  # accelerated_op/__init__.py:47
    assert out[0] is a and torch.isfinite(a).all()
    g = torch.randn(1000, device='cuda')
    r = ref_ext.backward_nu(dnu=g, updates=g, nu=g, b1=0.999)
    assert len(r) == 2
    count = torch.tensor(3, device='cuda')
    m, v = 0.1 * torch.randn(1000, device='cuda'), torch.rand(1000, device='cuda')
    got = ref_ext.forward_updates(new_mu=m, new_nu=v, b1=0.9, b2=0.999, eps=1e-8, eps_root=0.0,
                                  count=count)
    want = O.forward_updates(host(m), host(v), 0.9, 0.999, 1e-8, 0.0, 3)
    assert_bit_equal(host(got), want, 'count as a tensor')
    with pytest.raises(RuntimeError, match='Not implemented'):
        ref_ext.forward_mu(torch.ones(2, device='meta'), torch.ones(2, device='meta'), 0.9)
    cpu = ref_ext.forward_mu(torch.ones(4), torch.full((4,), 2.0), 0.9)  # CPU branch untouched
    assert cpu.device.type == 'cpu' and torch.allclose(cpu, torch.full((4,), 1.9))


def test_reference_autograd_wrapper_on_the_dropin(ref_ext):
    """The three autograd Functions exactly as accelerated_op/adam_op.py:36-121 builds them,
    bound to the drop-in module: values and gradients against the oracle's chain."""

    class MuOp(torch.autograd.Function):
        @staticmethod
        def forward(ctx, updates, mu, b1):
            ctx.save_for_backward(updates, mu)
            ctx.b1 = b1
            return ref_ext.forward_mu(updates, mu, b1)

        @staticmethod
        def backward(ctx, dmu):
            updates, mu = ctx.saved_tensors
            r = ref_ext.backward_mu(dmu, updates, mu, ctx.b1)
            return r[0], r[1], None

    class NuOp(torch.autograd.Function):
        @staticmethod
        def forward(ctx, updates, nu, b2):
            ctx.save_for_backward(updates, nu)
            ctx.b2 = b2
            return ref_ext.forward_nu(updates, nu, b2)

        @staticmethod
        def backward(ctx, dnu):
            updates, nu = ctx.saved_tensors
            r = ref_ext.backward_nu(dnu, updates, nu, ctx.b2)
            return r[0], r[1], None

    class UpdatesOp(torch.autograd.Function):
        @staticmethod
        def forward(ctx, new_mu, new_nu, hyper):
            b1, b2, eps, eps_root, count = hyper
            out = ref_ext.forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count)
            ctx.save_for_backward(out, new_mu, new_nu)
            ctx.hyper = hyper
            return out

        @staticmethod
        def backward(ctx, dupdates):
            out, new_mu, new_nu = ctx.saved_tensors
            b1, b2, _, eps_root, count = ctx.hyper
            r = ref_ext.backward_updates(dupdates, out, new_mu, new_nu, b1, b2, eps_root, count)
            return r[0], r[1], None

    rng = np.random.default_rng(8)
    n, b1, b2, eps, er, c = 70_001, 0.9, 0.999, 1e-8, 1e-8, 5
    g = rng.standard_normal(n)
    m = 0.1 * rng.standard_normal(n)
    v = np.abs(0.01 * rng.standard_normal(n))
    d = rng.standard_normal(n)
    tg, tm, tv = (dev(x).requires_grad_(True) for x in (g, m, v))
    new_mu, new_nu = MuOp.apply(tg, tm, b1), NuOp.apply(tg, tv, b2)
    new_u = UpdatesOp.apply(new_mu, new_nu, (b1, b2, eps, er, torch.tensor(c, device='cuda')))
    new_u.backward(dev(d))
    e_mu, e_nu = O.forward_mu(g, m, b1), O.forward_nu(g, v, b2)
    e_u = O.forward_updates(e_mu, e_nu, b1, b2, eps, er, c)
    bm, bv = O.backward_updates(d, e_u, e_mu, b1, b2, er, c)
    gu1, gm = O.backward_mu(bm, b1)
    gu2, gv = O.backward_nu(bv, g, b2)
    assert_bit_equal(host(new_u), e_u, 'new_updates')
    assert_bit_equal(host(tm.grad), gm, 'd mu')
    assert_bit_equal(host(tv.grad), gv, 'd nu')
    assert_bit_equal(host(tg.grad), gu1 + gu2, 'd updates')
