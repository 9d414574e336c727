"""`torch.compile(fullgraph=True)` over code that calls the fused Adam operator: the functions
are registered with `torch.library` (schema, fake implementation), so Dynamo traces through them
without a graph break and the compiled function computes what the eager one does, bit for bit.
The `aot_eager` backend is used: it exercises tracing, functionalisation of the in-place
operators and AOT autograd, and leaves code generation for the surrounding PyTorch ops out."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import AdamOp
from torchopt_amd._C import adam_op
from torchopt_amd.accelerated_op import library  # noqa: F401  (registers the operators)

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()


def host(t):
    return t.detach().cpu().numpy()


def draw(n, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(n).astype(np.float32),
            (0.1 * rng.standard_normal(n)).astype(np.float32),
            np.abs(0.01 * rng.standard_normal(n)).astype(np.float32))


def test_registered_operators_pass_opcheck():
    """torch.library.opcheck: schema (what is mutated), fake implementation against the real one,
    and the AOT dispatch path, for one operator of each kind."""
    g, m, v = (torch.from_numpy(a).cuda() for a in draw(1000, 1))
    ops = torch.ops.torchopt_amd
    torch.library.opcheck(ops.forward_mu.default, (g, m, B1))
    torch.library.opcheck(ops.forward_updates.default, (m, v, B1, B2, EPS, 0.0, 3))
    torch.library.opcheck(ops.backward_nu.default, (g, m, v, B2))
    torch.library.opcheck(ops.forward_.default, (g.clone(), m.clone(), v.clone(), B1, B2, EPS, 0.0, 3))
    torch.library.opcheck(ops.fused_step_multi_.default,
                          ([g.clone()], [g.clone()], [m.clone()], [v.clone()], B1, B2, EPS, 0.0, 3,
                           0.01, False, False, 0.0, False))


def test_inplace_step_compiles_without_graph_breaks():
    op = AdamOp(B1, B2, EPS, eps_root=0.0, inplace=True)

    def step(u, m, v):
        new_m, new_v, new_u = op(m, v, u, 7)
        return new_u * 2.0, new_m, new_v

    compiled = torch.compile(step, fullgraph=True, backend='aot_eager')
    g, m, v = draw(70_001, 2)
    dg, dm, dv = (torch.from_numpy(a).cuda() for a in (g, m, v))
    print('compiled in-place step', flush=True)
    doubled, out_m, out_v = compiled(dg, dm, dv)
    O.forward_inplace(g, m, v, B1, B2, EPS, 0.0, 7)
    assert_bit_equal(host(dg), g, 'updates, overwritten in place')
    assert_bit_equal(host(dm), m, 'mu, overwritten in place')
    assert_bit_equal(host(dv), v, 'nu, overwritten in place')
    assert_bit_equal(host(doubled), g * np.float32(2), 'value computed from the result')


def test_differentiable_step_compiles_with_its_backward():
    op = AdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)

    def loss(u, m, v, w):
        new_m, new_v, new_u = op(m, v, u, 4)
        return (new_u * w).sum() + (new_m * w).sum()

    g, m, v = draw(5000, 3)
    w = np.random.default_rng(4).standard_normal(5000).astype(np.float32)

    def leaves():
        return [torch.from_numpy(a).cuda().requires_grad_(True) for a in (g, m, v)]

    dw = torch.from_numpy(w).cuda()
    eager = leaves()
    loss(*eager, dw).backward()
    traced = leaves()
    print('compiled differentiable step + backward', flush=True)
    torch.compile(loss, fullgraph=True, backend='aot_eager')(*traced, dw).backward()
    for a, b, name in zip(eager, traced, ('updates', 'mu', 'nu')):
        assert_bit_equal(host(b.grad), host(a.grad), f'gradient w.r.t. {name}')
    # and the eager gradients are the oracle's
    e_mu, e_nu = O.forward_mu(g, m, B1), O.forward_nu(g, v, B2)
    e_u = O.forward_updates(e_mu, e_nu, B1, B2, EPS, 1e-8, 4)
    bm, bv = O.backward_updates(w, e_u, e_mu, B1, B2, 1e-8, 4)
    _, gm = O.backward_mu(bm + w, B1)
    assert_bit_equal(host(eager[1].grad), gm, 'gradient w.r.t. mu against the oracle')


def test_optimizer_step_shaped_function_compiles():
    """What FusedAdam(capturable=True).step() does for one group -- advance the device count,
    one fused pass over the list -- as a function of tensors, compiled as one graph and run for
    five steps against the oracle."""
    sizes = [3000, 17, 70_001]
    rng = np.random.default_rng(5)
    hp = [rng.standard_normal(n).astype(np.float32) for n in sizes]
    hm = [np.zeros(n, np.float32) for n in sizes]
    hv = [np.zeros(n, np.float32) for n in sizes]
    params = [torch.from_numpy(a.copy()).cuda() for a in hp]
    mu = [torch.zeros(n, device='cuda') for n in sizes]
    nu = [torch.zeros(n, device='cuda') for n in sizes]
    table = adam_op.bias_rows(torch.float32, B1, B2, 0.0, 1, 32).cuda()
    count = torch.zeros((), dtype=torch.int64, device='cuda')
    ops = torch.ops.torchopt_amd

    def step(params, grads, mu, nu, table, count):
        ops.count_advance_(count)
        ops.fused_step_multi_devcount_(params, grads, mu, nu, B1, B2, EPS, 0.0, table, 1, count,
                                       0.01, False, False, 0.02, True)
        return count + 0

    compiled = torch.compile(step, fullgraph=True, backend='aot_eager')
    for k in range(1, 6):
        fresh = [rng.standard_normal(n).astype(np.float32) for n in sizes]
        grads = [torch.from_numpy(f).cuda() for f in fresh]
        print(f'compiled optimizer step {k}', flush=True)
        seen = compiled(params, grads, mu, nu, table, count)
        assert int(seen) == k == int(count)
        for j, f in enumerate(fresh):
            O.fused_step(hp[j], f, hm[j], hv[j], B1, B2, EPS, 0.0, k, 0.01, False, False, 0.02, True)
            assert_bit_equal(host(params[j]), hp[j], f'step {k} params[{j}]')
            assert_bit_equal(host(mu[j]), hm[j], f'step {k} mu[{j}]')
            assert_bit_equal(host(nu[j]), hv[j], f'step {k} nu[{j}]')


def test_host_count_list_step_compiles():
    sizes = [1000, 5, 4099]
    hs = [draw(n, 20 + k) for k, n in enumerate(sizes)]
    us, ms, vs = ([torch.from_numpy(h[j]).cuda() for h in hs] for j in range(3))

    def step(us, ms, vs):
        torch.ops.torchopt_amd.forward_multi_(us, ms, vs, B1, B2, EPS, 0.0, 2)
        return [u + 1 for u in us]

    print('compiled host-count list step', flush=True)
    plus_one = torch.compile(step, fullgraph=True, backend='aot_eager')(us, ms, vs)
    for k, h in enumerate(hs):
        e = O.forward_inplace(h[0].copy(), h[1].copy(), h[2].copy(), B1, B2, EPS, 0.0, 2)
        assert_bit_equal(host(us[k]), e[0], f'updates[{k}]')
        assert_bit_equal(host(ms[k]), e[1], f'mu[{k}]')
        assert_bit_equal(host(plus_one[k]), e[0] + np.float32(1), f'updates[{k}] + 1')
