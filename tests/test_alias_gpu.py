"""Functional `adam` / `adamw`, `chain`, `apply_updates` and `MetaAdam` on the GPU, pinned the way
the reference pins its accelerated path: against `torch.optim.Adam` / `AdamW` in float64 at 25x
the default tolerance (/root/reference/tests/test_alias.py:207-270, 487-550,
tests/helpers.py:202-229), and the differentiable optimizer against the same inner loop written
with plain differentiable tensor operations."""

from __future__ import annotations

import pytest
import torch

import torchopt_amd as topt

pytestmark = pytest.mark.gpu

TOL = dict(rtol=25 * 1e-7, atol=25 * 1e-7)


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()


def make_models():
    torch.manual_seed(7)

    def net():
        return torch.nn.Sequential(torch.nn.Linear(12, 24), torch.nn.Tanh(),
                                   torch.nn.Linear(24, 3)).to('cuda', torch.float64)

    a, b = net(), net()
    b.load_state_dict(a.state_dict())
    return a, b


def batches(n):
    g = torch.Generator(device='cuda').manual_seed(11)
    for _ in range(n):
        yield (torch.randn(32, 12, device='cuda', dtype=torch.float64, generator=g),
               torch.randn(32, 3, device='cuda', dtype=torch.float64, generator=g))


@pytest.mark.parametrize('inplace', [True, False])
@pytest.mark.parametrize('weight_decay', [0.0, 1e-2])
@pytest.mark.parametrize('maximize', [False, True])
def test_adam_tracks_torch_optim(inplace, weight_decay, maximize):
    model, ref = make_models()
    lr = 1e-2
    base = [p.detach().clone() for p in model.parameters()]
    optim = topt.adam(lr, weight_decay=weight_decay, maximize=maximize)
    params = tuple(model.parameters())
    state = optim.init(params)
    optim_ref = torch.optim.Adam(ref.parameters(), lr, weight_decay=weight_decay,
                                 maximize=maximize)
    for x, y in batches(5):
        loss = ((model(x) - y) ** 2).mean()
        grads = torch.autograd.grad(loss, params)
        updates, state = optim.update(grads, state, params=params, inplace=inplace)
        new = topt.apply_updates(params, updates, inplace=inplace)
        if not inplace:
            with torch.no_grad():
                for p, q in zip(params, new):
                    p.copy_(q)
        optim_ref.zero_grad()
        ((ref(x) - y) ** 2).mean().backward()
        optim_ref.step()
    for p, q, p0 in zip(model.parameters(), ref.parameters(), base):
        torch.testing.assert_close(p - p0, q - p0, **TOL)


@pytest.mark.parametrize('inplace', [True, False])
def test_adamw_tracks_torch_optim(inplace):
    model, ref = make_models()
    lr, wd = 1e-2, 5e-2
    optim = topt.adamw(lr, weight_decay=wd)
    params = tuple(model.parameters())
    state = optim.init(params)
    optim_ref = torch.optim.AdamW(ref.parameters(), lr, weight_decay=wd)
    for x, y in batches(5):
        grads = torch.autograd.grad(((model(x) - y) ** 2).mean(), params)
        updates, state = optim.update(grads, state, params=params, inplace=inplace)
        with torch.no_grad():
            for p, u in zip(params, updates):
                p.add_(u)
        optim_ref.zero_grad()
        ((ref(x) - y) ** 2).mean().backward()
        optim_ref.step()
    for p, q in zip(model.parameters(), ref.parameters()):
        torch.testing.assert_close(p, q, **TOL)


def test_learning_rate_schedule_sees_the_count():
    seen = []

    def schedule(count):
        seen.append(int(count))
        return 0.1 / (1 + int(count))

    optim = topt.adam(schedule)
    p = (torch.ones(4, device='cuda'),)
    state = optim.init(p)
    for _ in range(3):
        u, state = optim.update((torch.ones(4, device='cuda'),), state, params=p, inplace=True)
    assert seen == [0, 1, 2]
    # first step of Adam from zero state is sign(g) = 1: the update is -lr(count)
    torch.testing.assert_close(u[0], torch.full((4,), -0.1 / 3, device='cuda'), rtol=1e-4, atol=0)


def test_chain_state_and_missing_params():
    optim = topt.adam(1e-3, weight_decay=0.1)
    p = (torch.ones(3, device='cuda'),)
    state = optim.init(p)
    assert isinstance(state, tuple) and len(state) == 3
    with pytest.raises(AssertionError, match='Parameters are required'):
        optim.update((torch.ones(3, device='cuda'),), state, inplace=True)
    with pytest.raises(ValueError, match='number of updates and states'):
        optim.update((torch.ones(3, device='cuda'),), state[:2], params=p)


def inner_loop_plain(w, b, x, y, steps, lr, b1, b2, eps, eps_root):
    """The same MetaAdam inner loop with ordinary differentiable tensor operations."""
    mw, vw, mb, vb = (torch.zeros_like(t) for t in (w, w, b, b))
    for t in range(1, steps + 1):
        loss = ((x @ w.t() + b - y) ** 2).mean()
        gw, gb = torch.autograd.grad(loss, (w, b), create_graph=True)
        mw, mb = b1 * mw + (1 - b1) * gw, b1 * mb + (1 - b1) * gb
        vw, vb = b2 * vw + (1 - b2) * gw * gw, b2 * vb + (1 - b2) * gb * gb
        c1, c2 = 1 / (1 - b1 ** t), 1 / (1 - b2 ** t)
        w = w - lr * (mw * c1) / (torch.sqrt(vw * c2 + eps_root) + eps)
        b = b - lr * (mb * c1) / (torch.sqrt(vb * c2 + eps_root) + eps)
    return w, b


@pytest.mark.parametrize('eps,er,rtol,atol', [(0.0, 0.0, 1e-8, 1e-11), (1e-8, 1e-8, 5e-3, 1e-5)],
                         ids=['exact-when-eps-is-zero', 'reference-approximation'])
def test_meta_adam_outer_gradient(eps, er, rtol, atol):
    """Two inner steps of MetaAdam on a linear model, then an outer loss on the adapted
    parameters, differentiated back to the initial parameters and to a learnable input scale.
    The reference's backward of the update uses 1/(sqrt(v)+eps) where the exact derivative has
    1/sqrt(v), and 1/(1-b2^t+eps_root) for the bias correction (adam_op_impl_cpu.cpp:309-329):
    with eps = eps_root = 0 it is the exact derivative and must agree to rounding; otherwise it
    is off by up to eps/sqrt(v) per element, by design."""
    torch.manual_seed(5)
    dt = torch.float64
    lin = torch.nn.Linear(6, 4).to('cuda', dt)
    w0, b0 = lin.weight, lin.bias
    scale = torch.tensor(1.3, device='cuda', dtype=dt, requires_grad=True)
    x = torch.randn(20, 6, device='cuda', dtype=dt)
    y = torch.randn(20, 4, device='cuda', dtype=dt)
    xo = torch.randn(20, 6, device='cuda', dtype=dt)
    yo = torch.randn(20, 4, device='cuda', dtype=dt)
    lr, b1, b2 = 0.05, 0.9, 0.999

    opt = topt.MetaAdam(lin, lr, (b1, b2), eps, eps_root=er)
    for _ in range(2):
        opt.step(((lin(x * scale) - y) ** 2).mean())
    assert lin.weight.grad_fn is not None  # parameters were replaced by differentiable results
    outer = ((lin(xo) - yo) ** 2).mean()
    got = torch.autograd.grad(outer, (w0, b0, scale))

    w, b = inner_loop_plain(w0, b0, x * scale, y, 2, lr, b1, b2, eps, er)
    outer_ref = ((xo @ w.t() + b - yo) ** 2).mean()
    want = torch.autograd.grad(outer_ref, (w0, b0, scale))
    torch.testing.assert_close(lin.weight, w, rtol=1e-9, atol=1e-12)
    for g, r in zip(got, want):
        torch.testing.assert_close(g, r, rtol=rtol, atol=atol)
    counts = opt.state_dict()[0][1].count
    assert [int(c) for c in counts] == [2, 2]


def test_meta_adamw_and_unused_parameters():
    """A parameter the loss does not touch gets no gradient (allow_unused) and stays put."""
    torch.manual_seed(2)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.used = torch.nn.Linear(5, 2)
            self.unused = torch.nn.Linear(5, 2)

        def forward(self, x):
            return self.used(x)

    net = Net().to('cuda')
    before = net.unused.weight
    opt = topt.MetaAdamW(net, 1e-2, weight_decay=0.1)
    x = torch.randn(8, 5, device='cuda')
    opt.step(net(x).pow(2).mean())
    assert net.unused.weight is before and net.used.weight.grad_fn is not None
    opt.step(net(x).pow(2).mean())
    st = opt.state_dict()[0][1]
    assert [int(c) for c in st.count] == [2, 2, 0, 0]


def test_func_optimizer_inner_loop_matches_plain_autograd():
    """`FuncOptimizer(adam(...)).step(loss, params)` on a dict of parameters: two differentiable
    steps, outer gradient against the hand-written inner loop (eps = eps_root = 0, where the
    op's backward is the exact derivative)."""
    torch.manual_seed(9)
    dt = torch.float64
    w0 = torch.randn(4, 6, device='cuda', dtype=dt, requires_grad=True)
    b0 = torch.randn(4, device='cuda', dtype=dt, requires_grad=True)
    x = torch.randn(20, 6, device='cuda', dtype=dt)
    y = torch.randn(20, 4, device='cuda', dtype=dt)
    lr, b1, b2 = 0.05, 0.9, 0.999
    opt = topt.FuncOptimizer(topt.adam(lr, (b1, b2), 0.0))
    params = {'w': w0, 'b': b0, 'frozen': None}
    for _ in range(2):
        loss = ((x @ params['w'].t() + params['b'] - y) ** 2).mean()
        params = opt.step(loss, params)
    assert set(params) == {'w', 'b', 'frozen'} and params['frozen'] is None
    outer = (params['w'] ** 2).sum() + (params['b'] ** 2).sum()
    got = torch.autograd.grad(outer, (w0, b0))
    w, b = inner_loop_plain(w0, b0, x, y, 2, lr, b1, b2, 0.0, 0.0)
    want = torch.autograd.grad((w ** 2).sum() + (b ** 2).sum(), (w0, b0))
    torch.testing.assert_close(params['w'], w, rtol=1e-9, atol=1e-12)
    for g, r in zip(got, want):
        torch.testing.assert_close(g, r, rtol=1e-8, atol=1e-11)
    with pytest.raises(TypeError):
        topt.FuncOptimizer(object())


@pytest.mark.parametrize('inplace', [True, False])
def test_adamw_mask_decays_only_the_chosen_leaves(inplace):
    """`mask` as the reference's adamw takes it (alias/adamw.py:62): weights decay, biases do
    not -- against torch.optim.AdamW with two parameter groups."""
    model, ref = make_models()
    lr, wd = 1e-2, 5e-2
    params = tuple(model.parameters())
    mask = lambda ps: tuple(p.dim() > 1 for p in ps)  # noqa: E731
    optim = topt.adamw(lr, weight_decay=wd, mask=mask, use_accelerated_op=True)
    state = optim.init(params)
    optim_ref = torch.optim.AdamW([
        {'params': [p for p in ref.parameters() if p.dim() > 1], 'weight_decay': wd},
        {'params': [p for p in ref.parameters() if p.dim() <= 1], 'weight_decay': 0.0}], lr)
    for x, y in batches(4):
        grads = torch.autograd.grad(((model(x) - y) ** 2).mean(), params)
        updates, state = optim.update(grads, state, params=params, inplace=inplace)
        with torch.no_grad():
            for p, u in zip(params, updates):
                p.add_(u)
        optim_ref.zero_grad()
        ((ref(x) - y) ** 2).mean().backward()
        optim_ref.step()
    for p, q in zip(model.parameters(), ref.parameters()):
        torch.testing.assert_close(p, q, **TOL)


@pytest.mark.parametrize('inplace', [True, False])
@pytest.mark.parametrize('make', [lambda: topt.adam(0.01, weight_decay=0.1, maximize=True),
                                  lambda: topt.adamw(0.01, weight_decay=0.1),
                                  lambda: topt.adam(lambda c: 0.01 / (1 + c))],
                         ids=['adam', 'adamw', 'schedule'])
def test_dict_trees_are_matched_by_name_through_the_whole_chain(make, inplace):
    """Parameters, gradients and state as flat dicts whose insertion orders differ: every
    transformation of the chain and `apply_updates` pair leaves by name (the reference's pytree
    library sorts dict keys), so the run equals the same run on tuples."""
    torch.manual_seed(4)
    names = ['c', 'a', 'd', 'b']
    shapes = [(5, 3), (7,), (2, 2, 2), (300,)]
    values = [torch.randn(s, device='cuda', dtype=torch.float64) for s in shapes]
    pd = {n: v.clone() for n, v in zip(names, values)}
    pt = tuple(v.clone() for v in values)
    od, ot = make(), make()
    sd, st = od.init(pd), ot.init(pt)
    for step in range(3):
        grads = [torch.randn(s, device='cuda', dtype=torch.float64) for s in shapes]
        order = [2, 0, 3, 1] if step % 2 else [0, 1, 2, 3]
        gd = {names[k]: grads[k].clone() for k in order}
        ud, sd = od.update(gd, sd, params=pd, inplace=inplace)
        ut, st = ot.update(tuple(g.clone() for g in grads), st, params=pt, inplace=inplace)
        pd = topt.apply_updates(pd, ud, inplace=inplace)
        pt = topt.apply_updates(pt, ut, inplace=inplace)
        assert sorted(pd) == sorted(names)
        for k, n in enumerate(names):
            assert torch.equal(ud[n], ut[k]), (step, n, 'update')
            assert torch.equal(pd[n], pt[k]), (step, n, 'parameter')
