"""The one-pass optimizer step (Adam, scale by -lr, add to the parameters) against the CPU
oracle of the reference's three-pass chain, against the unfused chain run on the GPU, and
through the `FusedAdam` optimizer."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import FusedAdam, FusedAdamW
from torchopt_amd._C import adam_op
from torchopt_amd.transform import scale_by_accelerated_adam

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def rand4(dtype, n, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(n).astype(dtype), rng.standard_normal(n).astype(dtype),
            (0.1 * rng.standard_normal(n)).astype(dtype),
            np.abs(0.01 * rng.standard_normal(n)).astype(dtype))


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
@pytest.mark.parametrize('maximize', [False, True])
@pytest.mark.parametrize('write_updates', [False, True])
def test_single_tensor_against_oracle(dtype, maximize, write_updates):
    for k, n in enumerate([1, 3, 255, 256, 257, 1025, 65537, (1 << 20) + 3]):
        lr, count, eps_root = (1e-3, 1, 0.0) if k % 2 else (0.05, 1000, 1e-8)
        p, g, m, v = rand4(dtype, n, 200 + n)
        gp, gg, gm, gv = dev(p), dev(g), dev(m), dev(v)
        r = adam_op.fused_step_(gp, gg, gm, gv, B1, B2, EPS, eps_root, count, lr,
                                maximize=maximize, write_updates=write_updates)
        assert r[0] is gp and r[1] is gg
        O.fused_step(p, g, m, v, B1, B2, EPS, eps_root, count, lr, maximize, write_updates)
        assert_bit_equal(host(gp), p, f'n={n} params')
        assert_bit_equal(host(gm), m, f'n={n} mu')
        assert_bit_equal(host(gv), v, f'n={n} nu')
        assert_bit_equal(host(gg), g, f'n={n} updates (untouched unless write_updates)')


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
@pytest.mark.parametrize('decoupled', [False, True], ids=['l2', 'decoupled'])
def test_weight_decay_against_oracle(dtype, decoupled):
    for k, n in enumerate([1, 257, 65537, (1 << 20) + 3]):
        p, g, m, v = rand4(dtype, n, 500 + n)
        gp, gg, gm, gv = dev(p), dev(g), dev(m), dev(v)
        adam_op.fused_step_(gp, gg, gm, gv, B1, B2, EPS, 1e-8, 4, 0.01, maximize=bool(k % 2),
                            write_updates=True, weight_decay=0.05, decoupled=decoupled)
        O.fused_step(p, g, m, v, B1, B2, EPS, 1e-8, 4, 0.01, bool(k % 2), True, 0.05, decoupled)
        for t, want, what in ((gp, p, 'params'), (gg, g, 'updates'), (gm, m, 'mu'), (gv, v, 'nu')):
            assert_bit_equal(host(t), want, f'n={n} {what}')


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
@pytest.mark.parametrize('decay', [None, 'l2', 'decoupled'])
def test_operands_over_the_whole_exponent_range(dtype, decay):
    """Operands drawn uniformly over the finite bit patterns of the type (every exponent equally
    likely, denormals and near-overflow values included): the step's fused multiply-adds,
    division and root under underflow and overflow; whole-tile kernel and ragged tail."""
    n = (1 << 22) + 37
    rng = np.random.default_rng(21)
    it = np.uint32 if dtype is np.float32 else np.uint64
    top = int(np.array(np.inf, dtype).view(it))

    def draw(nonneg=False):
        bits = rng.integers(0, top, size=n, dtype=it)
        if not nonneg:
            bits |= rng.integers(0, 2, size=n, dtype=it) << it(8 * bits.itemsize - 1)
        return bits.view(dtype)

    p, g, m, v = draw(), draw(), draw(), draw(nonneg=True)
    wd, decoupled = (0.0, False) if decay is None else (0.05, decay == 'decoupled')
    gp, gg, gm, gv = dev(p), dev(g), dev(m), dev(v)
    adam_op.fused_step_(gp, gg, gm, gv, B1, B2, EPS, 1e-8, 4, 0.01, maximize=True,
                        write_updates=True, weight_decay=wd, decoupled=decoupled)
    with np.errstate(all='ignore'):
        O.fused_step(p, g, m, v, B1, B2, EPS, 1e-8, 4, 0.01, True, True, wd, decoupled)
    for t, want, what in ((gp, p, 'params'), (gg, g, 'updates'), (gm, m, 'mu'), (gv, v, 'nu')):
        assert_bit_equal(host(t), want, f'whole exponent range, decay {decay}: {what}')


@pytest.mark.parametrize('decay', ['l2', 'decoupled'])
def test_weight_decay_equals_the_unfused_chain_on_the_gpu(decay):
    """With PyTorch's own GPU kernels for the neighbours (add_ with alpha, mul_, add_)."""
    n, lr, wd, count = (1 << 21) + 1, 1e-3, 0.02, 9
    g = torch.Generator(device='cuda').manual_seed(8)
    p, u = (torch.randn(n, device='cuda', generator=g) for _ in range(2))
    m = torch.randn(n, device='cuda', generator=g).mul_(0.1)
    v = torch.randn(n, device='cuda', generator=g).mul_(0.01).abs_()
    p2, u2, m2, v2 = p.clone(), u.clone(), m.clone(), v.clone()
    if decay == 'l2':
        u.add_(p, alpha=wd)
    adam_op.forward_(u, m, v, B1, B2, EPS, 0.0, count)
    if decay == 'decoupled':
        u.add_(p, alpha=wd)
    u.mul_(-lr)
    p.add_(u)
    adam_op.fused_step_(p2, u2, m2, v2, B1, B2, EPS, 0.0, count, lr, write_updates=True,
                        weight_decay=wd, decoupled=decay == 'decoupled')
    assert torch.equal(p, p2) and torch.equal(u, u2) and torch.equal(m, m2) and torch.equal(v, v2)


@pytest.mark.parametrize('dtype', [torch.float32, torch.float64], ids=['f32', 'f64'])
def test_equals_the_unfused_chain_on_the_gpu(dtype):
    """forward_ then Tensor.mul_(-lr) then Tensor.add_ -- the reference's three passes, with
    PyTorch's own GPU kernels for the last two -- give the same bits as the one-pass step."""
    n, lr, count = (1 << 22) + 5, 3e-4, 12
    g = torch.Generator(device='cuda').manual_seed(5)
    p = torch.randn(n, device='cuda', dtype=dtype, generator=g)
    u = torch.randn(n, device='cuda', dtype=dtype, generator=g)
    m = torch.randn(n, device='cuda', dtype=dtype, generator=g).mul_(0.1)
    v = torch.randn(n, device='cuda', dtype=dtype, generator=g).mul_(0.01).abs_()
    p2, u2, m2, v2 = p.clone(), u.clone(), m.clone(), v.clone()
    adam_op.forward_(u, m, v, B1, B2, EPS, 0.0, count)
    u.mul_(-lr)
    p.add_(u)
    adam_op.fused_step_(p2, u2, m2, v2, B1, B2, EPS, 0.0, count, lr, write_updates=True)
    assert torch.equal(p, p2) and torch.equal(u, u2) and torch.equal(m, m2) and torch.equal(v, v2)


def test_multi_tensor_with_ragged_members_and_counts():
    sizes = [1000, 0, 17, 300_001, 256, 5] + [33] * 100  # crosses one kernel-argument table
    counts = [(k % 3) + 1 for k in range(len(sizes))]
    hs = [rand4(np.float32, n, 300 + k) for k, n in enumerate(sizes)]
    ds = [[dev(a) for a in h] for h in hs]
    r = adam_op.fused_step_multi_([d[0] for d in ds], [d[1] for d in ds], [d[2] for d in ds],
                                  [d[3] for d in ds], B1, B2, EPS, 1e-8, counts, 0.01,
                                  maximize=True, write_updates=False)
    assert r[0][0] is ds[0][0]
    for k, (h, d) in enumerate(zip(hs, ds)):
        O.fused_step(h[0], h[1], h[2], h[3], B1, B2, EPS, 1e-8, counts[k], 0.01, True, False)
        for j, what in enumerate(('params', 'updates', 'mu', 'nu')):
            assert_bit_equal(host(d[j]), h[j], f'tensor {k} {what}')


@pytest.mark.parametrize('maximize', [False, True])
def test_fused_adam_equals_the_transformation_chain(maximize):
    """FusedAdam.step() against scale_by_accelerated_adam -> mul_(-lr) -> add_ on clones, over
    several steps with a parameter whose gradient is missing on some steps."""
    torch.manual_seed(3)
    lr = 2e-3
    shapes = [(64, 32), (64,), (10, 64), (10,), ()]
    params = [torch.randn(s, device='cuda', requires_grad=True) for s in shapes]
    twins = [p.detach().clone() for p in params]
    opt = FusedAdam(params, lr, eps_root=1e-8, maximize=maximize)
    chain = scale_by_accelerated_adam(B1, B2, EPS, eps_root=1e-8)
    state = chain.init(tuple(twins))
    for step in range(6):
        opt.zero_grad(set_to_none=True)
        grads = [torch.randn(s, device='cuda') for s in shapes]
        if step in (1, 4):
            grads[3] = None
        for p, g in zip(params, grads):
            p.grad = None if g is None else g.clone()
        opt.step()
        # p.grad is left alone by the fused step
        assert all(p.grad is None or torch.equal(p.grad, g) for p, g in zip(params, grads))
        ups = tuple(None if g is None else (g.neg() if maximize else g.clone()) for g in grads)
        ups, state = chain.update(ups, state, params=tuple(twins), inplace=True)
        for t, u in zip(twins, ups):
            if u is not None:
                t.add_(u.mul_(-lr))
        for k, (p, t) in enumerate(zip(params, twins)):
            assert torch.equal(p.detach(), t), f'step {step} param {k}'
    st = opt.state_dict()[0]
    assert [int(c) for c in st.count] == [6, 6, 6, 4, 6]
    for a, b in zip(st.mu, state.mu):
        assert torch.equal(a, b)
    # the state round-trips and can be handed to the transformation
    opt.load_state_dict(opt.state_dict())
    chain.update(tuple(torch.randn(s, device='cuda') for s in shapes), st, inplace=True)


@pytest.mark.parametrize('cls,ref_cls,wd', [(FusedAdam, torch.optim.Adam, 0.0),
                                            (FusedAdam, torch.optim.Adam, 0.05),
                                            (FusedAdamW, torch.optim.AdamW, 0.05)])
def test_fused_adam_tracks_torch_optim_adam(cls, ref_cls, wd):
    torch.manual_seed(0)
    net = torch.nn.Sequential(torch.nn.Linear(16, 32), torch.nn.ReLU(),
                              torch.nn.Linear(32, 4)).to('cuda', torch.float64)
    ref = torch.nn.Sequential(torch.nn.Linear(16, 32), torch.nn.ReLU(),
                              torch.nn.Linear(32, 4)).to('cuda', torch.float64)
    ref.load_state_dict(net.state_dict())
    a = cls(net.parameters(), 1e-2, weight_decay=wd)
    b = ref_cls(ref.parameters(), 1e-2, weight_decay=wd)
    for _ in range(10):
        x = torch.randn(32, 16, device='cuda', dtype=torch.float64)
        y = torch.randn(32, 4, device='cuda', dtype=torch.float64)
        for model, opt in ((net, a), (ref, b)):
            opt.zero_grad()
            loss = ((model(x) - y) ** 2).mean()
            loss.backward()
            opt.step()
    for p, q in zip(net.parameters(), ref.parameters()):
        torch.testing.assert_close(p, q, rtol=25e-7, atol=25e-7)


def test_fused_adam_one_go_path_equals_the_general_path():
    """`step()` takes every parameter in one call when all have gradients and have stepped
    together, and sorts them into buckets otherwise.  A run that moves between the two (a
    gradient missing on the third step, everything present again afterwards) against a run held
    on the general path throughout: parameters, moments and step numbers bit for bit."""
    torch.manual_seed(5)
    shapes = [(300,), (17, 9), (4096,), (1,)]
    base = [torch.randn(s, device='cuda') for s in shapes]
    runs = []
    for general_only in (False, True):
        ps = [b.clone().requires_grad_(True) for b in base]
        opt = FusedAdam(ps, 0.01, eps_root=1e-8)
        gen = torch.Generator(device='cuda').manual_seed(9)
        for step in range(6):
            if general_only:
                opt._uniform = [False] * len(opt._uniform)
            for k, p in enumerate(ps):
                p.grad = torch.randn(p.shape, device='cuda', generator=gen)
                if step == 2 and k == 1:
                    p.grad = None
            opt.step()
        (state,) = opt.state_dict()
        runs.append((ps, state))
    (pa, sa), (pb, sb) = runs
    assert [int(c) for c in sa.count] == [int(c) for c in sb.count] == [6, 5, 6, 6]
    for a, b in zip(list(pa) + list(sa.mu) + list(sa.nu), list(pb) + list(sb.mu) + list(sb.nu)):
        assert torch.equal(a, b)


def test_fused_adam_reads_gradients_in_any_layout():
    """`p.grad` may be channels-last, expanded or a strided slice while the parameter is
    contiguous: the step only reads it, so it is brought to the parameter's memory order."""
    torch.manual_seed(11)
    ps = [torch.randn(4, 3, 5, 5, device='cuda'), torch.randn(6, 40, device='cuda'),
          torch.randn(33, device='cuda')]
    grads = [torch.randn(4, 3, 5, 5, device='cuda').contiguous(memory_format=torch.channels_last),
             torch.tensor(0.25, device='cuda').expand(6, 40),
             torch.randn(66, device='cuda')[::2]]
    a = [p.clone().requires_grad_(True) for p in ps]
    b = [p.clone().requires_grad_(True) for p in ps]
    opt_a, opt_b = FusedAdam(a, lr=0.01), FusedAdam(b, lr=0.01)
    for _ in range(3):
        for p, q, g in zip(a, b, grads):
            p.grad, q.grad = g, g.contiguous()
        opt_a.step()
        opt_b.step()
    for p, q in zip(a, b):
        assert torch.equal(p, q)
    # the single-tensor entry point likewise
    p1, p2 = ps[0].clone(), ps[0].clone()
    m, v = torch.zeros_like(p1), torch.zeros_like(p1)
    adam_op.fused_step_(p1, grads[0], m, v, B1, B2, EPS, 0.0, 1, 0.01)
    adam_op.fused_step_(p2, grads[0].contiguous(), torch.zeros_like(p2), torch.zeros_like(p2), B1,
                        B2, EPS, 0.0, 1, 0.01)
    assert torch.equal(p1, p2)
    with pytest.raises(RuntimeError):  # a gradient that must be overwritten has to be dense
        adam_op.fused_step_(p1, torch.tensor(0.25, device='cuda').expand(4, 3, 5, 5), m, v, B1,
                            B2, EPS, 0.0, 2, 0.01, write_updates=True)


def test_fused_adam_with_a_learning_rate_schedule():
    """The schedule sees the number of steps already taken (0 on the first step); checked step
    by step against the oracle with the same host-computed rate, and loosely against
    `torch.optim.Adam` under a `LambdaLR`."""
    schedule = lambda count: 0.05 / (1.0 + 0.5 * count)  # noqa: E731
    rng = np.random.default_rng(21)
    p0 = rng.standard_normal(3001).astype(np.float32)
    p = dev(p0).requires_grad_(True)
    q = dev(p0).requires_grad_(True)
    opt = FusedAdam([p], lr=schedule)
    ref = torch.optim.Adam([q], lr=1.0)
    sched = torch.optim.lr_scheduler.LambdaLR(ref, schedule)
    hp, hm, hv = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    for step in range(4):
        g = rng.standard_normal(3001).astype(np.float32)
        p.grad, q.grad = dev(g), dev(g)
        opt.step()
        ref.step()
        sched.step()
        O.fused_step(hp, g.copy(), hm, hv, B1, B2, EPS, 0.0, step + 1, schedule(step),
                     write_updates=False)
        assert_bit_equal(host(p), hp, f'step {step}')
    np.testing.assert_allclose(host(p), host(q), rtol=2e-5, atol=1e-6)


def test_fused_adamw_mask():
    """Biases exempt from the decay: against torch.optim.AdamW with two parameter groups."""
    torch.manual_seed(4)
    net = torch.nn.Sequential(torch.nn.Linear(7, 5), torch.nn.Tanh(), torch.nn.Linear(5, 3)).cuda()
    ref = torch.nn.Sequential(torch.nn.Linear(7, 5), torch.nn.Tanh(), torch.nn.Linear(5, 3)).cuda()
    ref.load_state_dict(net.state_dict())
    opt = FusedAdamW(net.parameters(), lr=1e-2, weight_decay=0.1,
                     mask=lambda ps: [p.dim() > 1 for p in ps])
    opt_ref = torch.optim.AdamW([
        {'params': [p for p in ref.parameters() if p.dim() > 1], 'weight_decay': 0.1},
        {'params': [p for p in ref.parameters() if p.dim() <= 1], 'weight_decay': 0.0}], lr=1e-2)
    for _ in range(4):
        x = torch.randn(16, 7, device='cuda')
        for model, o in ((net, opt), (ref, opt_ref)):
            o.zero_grad()
            model(x).pow(2).mean().backward()
            o.step()
    for p, q in zip(net.parameters(), ref.parameters()):
        torch.testing.assert_close(p, q, rtol=2e-5, atol=1e-6)


# ---- float16 / bfloat16 -----------------------------------------------------------------------
# The 16-bit step has no weight decay: Tensor.add_(p, alpha=wd) on 16-bit CPU tensors is not one
# arithmetic (tests/test_oracle.py shows body and tail of one call disagreeing), so there is no
# result to be identical to and the library refuses the combination.

TDT = {'f16': torch.float16, 'bf16': torch.bfloat16}


def rand4_16(fmt, n, seed):
    """(params, updates, mu, nu) as host arrays in the oracle's format for `fmt` (NumPy float16,
    or uint16 bit patterns for bfloat16) and as GPU tensors."""
    rng = np.random.default_rng(seed)
    raw = (rng.standard_normal(n), rng.standard_normal(n), 0.1 * rng.standard_normal(n),
           np.abs(0.01 * rng.standard_normal(n)))
    ts = [torch.from_numpy(a.astype(np.float32)).to(TDT[fmt]) for a in raw]
    return [bits16(t, fmt) for t in ts], [t.cuda() for t in ts]


def bits16(t, fmt):
    t = t.detach().cpu().contiguous()
    if fmt == 'bf16':
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
@pytest.mark.parametrize('maximize', [False, True])
@pytest.mark.parametrize('write_updates', [False, True])
def test_16_bit_single_tensor_against_oracle(fmt, maximize, write_updates):
    # sizes on both sides of the whole-tile kernel's threshold, ragged tails, odd element counts
    for k, n in enumerate([1, 3, 511, 512, 513, 4099, 65537, (1 << 22) + 7]):
        lr, count, eps_root = (1e-3, 1, 0.0) if k % 2 else (0.05, 1000, 1e-4)
        h, d = rand4_16(fmt, n, 900 + n)
        print(f'fused_step_ {fmt} n={n} maximize={maximize} write_updates={write_updates}',
              flush=True)
        adam_op.fused_step_(d[0], d[1], d[2], d[3], B1, B2, 1e-3, eps_root, count, lr,
                            maximize=maximize, write_updates=write_updates)
        O.fused_step(h[0], h[1], h[2], h[3], B1, B2, 1e-3, eps_root, count, lr, maximize,
                     write_updates)
        for j, what in enumerate(('params', 'updates', 'mu', 'nu')):
            assert_bit_equal(bits16(d[j], fmt), h[j], f'{fmt} n={n} {what}')


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
@pytest.mark.parametrize('operand', [0, 1, 2, 3], ids=['params', 'updates', 'mu', 'nu'])
@pytest.mark.parametrize('maximize', [False, True])
@pytest.mark.parametrize('lr', [0.05, 1e-3])
def test_16_bit_every_bit_pattern_of_one_operand(fmt, operand, maximize, lr):
    """All 65 536 values of the type (every denormal, infinity and NaN) in one operand, the
    others random, through the element-wise kernel (65 536 elements) and the whole-tile kernel
    (the same 128 times over): every conversion, rounding and sign case, the sign flip of
    `maximize` included.  (This is the test that caught float16 steps rounded once where the CPU
    rounds twice: parameter 0x09ae, direction 0x85d2, lr 0.05.)"""
    for repeat in (1, 128):
        n = (1 << 16) * repeat
        h, d = rand4_16(fmt, n, 500 + operand)
        every = torch.arange(n, dtype=torch.int32).to(torch.int16).view(TDT[fmt])
        d[operand] = every.cuda()
        h[operand] = bits16(every, fmt)
        print(f'fused_step_ {fmt} every pattern in operand {operand} x {repeat} '
              f'maximize={maximize} lr={lr}', flush=True)
        adam_op.fused_step_(d[0], d[1], d[2], d[3], B1, B2, 1e-3, 1e-4, 3, lr,
                            maximize=maximize, write_updates=True)
        with np.errstate(all='ignore'):
            O.fused_step(h[0], h[1], h[2], h[3], B1, B2, 1e-3, 1e-4, 3, lr, maximize, True)
        for j, what in enumerate(('params', 'updates', 'mu', 'nu')):
            assert_bit_equal(bits16(d[j], fmt), h[j], f'{fmt} all {operand} x {repeat} {what}')


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
@pytest.mark.parametrize('lr', [0.05, 1e-4, 1e-5, 2.5e-6])
def test_16_bit_steps_down_to_the_denormal_range(fmt, lr):
    """Small learning rates put float16 steps below 6.1e-5, the type's denormal range (with
    lr = 1e-4 nine steps in ten are denormal); the float multiplication by -lr and the rounding
    to 16 bits must stay two roundings there as everywhere, as on the CPU (a handful of
    elements per run tell the difference).  Whole tiles and the element-wise kernel of short
    and ragged tensors."""
    for n in (1, 5, 777, (1 << 18), (1 << 18) + 13):
        h, d = rand4_16(fmt, n, 4242 + n)
        print(f'fused_step_ {fmt} n={n} lr={lr}', flush=True)
        adam_op.fused_step_(d[0], d[1], d[2], d[3], B1, B2, 1e-3, 1e-4, 3, lr,
                            maximize=False, write_updates=True)
        with np.errstate(all='ignore'):
            O.fused_step(h[0], h[1], h[2], h[3], B1, B2, 1e-3, 1e-4, 3, lr, False, True)
        for j, what in enumerate(('params', 'updates', 'mu', 'nu')):
            assert_bit_equal(bits16(d[j], fmt), h[j], f'{fmt} n={n} lr={lr} {what}')


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
def test_16_bit_step_equals_the_unfused_chain(fmt):
    """forward_ in place on the GPU, then PyTorch's own mul_(-lr) and add_ -- its CPU kernels,
    which round the float product and then convert (PyTorch's GPU mul_ on this platform may
    round a float16 product once: 0x85d2 * -0.05 gives 0x4b there and 0x4a on the CPU)."""
    n, lr, count = (1 << 21) + 5, 0.05, 9
    h, d = rand4_16(fmt, n, 77)
    p, g, m, v = (t.clone() for t in d)
    adam_op.forward_(g, m, v, B1, B2, 1e-3, 0.0, count)
    p, g = p.cpu(), g.cpu()
    g.mul_(-lr)
    p.add_(g)
    adam_op.fused_step_(d[0], d[1], d[2], d[3], B1, B2, 1e-3, 0.0, count, lr, write_updates=True)
    for got, want, what in zip(d, (p, g, m, v), ('params', 'updates', 'mu', 'nu')):
        assert_bit_equal(bits16(got, fmt), bits16(want, fmt), f'{fmt} {what}')


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
def test_16_bit_list_with_ragged_members_and_counts(fmt):
    sizes = [864, 9216, 33, 4001, 5, 0, 70_001, 1 << 20]
    counts = [1, 1, 2, 7, 7, 3, 1000, 2]
    pairs = [rand4_16(fmt, n, 40 + k) for k, n in enumerate(sizes)]
    hs, ds = [p[0] for p in pairs], [p[1] for p in pairs]
    print(f'fused_step_multi_ {fmt} ragged list', flush=True)
    adam_op.fused_step_multi_([d[0] for d in ds], [d[1] for d in ds], [d[2] for d in ds],
                              [d[3] for d in ds], B1, B2, 1e-3, 1e-4, counts, 0.01,
                              maximize=True, write_updates=True)
    for k, (h, d) in enumerate(zip(hs, ds)):
        O.fused_step(h[0], h[1], h[2], h[3], B1, B2, 1e-3, 1e-4, counts[k], 0.01, True, True)
        for j, what in enumerate(('params', 'updates', 'mu', 'nu')):
            assert_bit_equal(bits16(d[j], fmt), h[j], f'{fmt} tensor {k} {what}')


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
def test_16_bit_step_refuses_weight_decay(fmt):
    _, d = rand4_16(fmt, 1000, 3)
    before = [t.clone() for t in d]
    for decoupled in (False, True):
        with pytest.raises(RuntimeError, match='weight decay for float32 and float64 only'):
            adam_op.fused_step_(d[0], d[1], d[2], d[3], B1, B2, 1e-3, 0.0, 1, 0.01,
                                weight_decay=0.01, decoupled=decoupled)
        with pytest.raises(RuntimeError, match='weight decay for float32 and float64 only'):
            adam_op.fused_step_multi_([d[0]], [d[1]], [d[2]], [d[3]], B1, B2, 1e-3, 0.0, 1, 0.01,
                                      weight_decay=0.01, decoupled=decoupled)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(d, before)), 'a refused call touched its tensors'


@pytest.mark.parametrize('fmt', ['f16', 'bf16'])
@pytest.mark.parametrize('capturable', [False, True])
def test_fused_adam_on_16_bit_parameters(fmt, capturable):
    """Five optimizer steps on 16-bit parameters, host-counted and with the count on the device,
    against the oracle step by step."""
    shapes = [(300, 7), (5,), (64, 64, 3)]
    rng = np.random.default_rng(21)
    tdt = TDT[fmt]
    params = [torch.from_numpy(rng.standard_normal(s).astype(np.float32)).to(tdt).cuda()
              .requires_grad_(True) for s in shapes]
    hp = [bits16(p, fmt).reshape(-1) for p in params]
    hm = [np.zeros_like(a) for a in hp]
    hv = [np.zeros_like(a) for a in hp]
    opt = FusedAdam(params, lr=0.01, eps=1e-3, eps_root=1e-4, capturable=capturable)
    for step in range(1, 6):
        grads = [torch.from_numpy(rng.standard_normal(s).astype(np.float32)).to(tdt) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = g.cuda()
        opt.step()
        for k, g in enumerate(grads):
            O.fused_step(hp[k], bits16(g, fmt).reshape(-1), hm[k], hv[k], B1, B2, 1e-3, 1e-4, step,
                         0.01)
            assert_bit_equal(bits16(params[k], fmt).reshape(-1), hp[k],
                             f'{fmt} step {step} params[{k}]')
