"""The entry points only enqueue kernels (no allocation, no copy, no synchronisation, tables in
kernel arguments), so a HIP graph can capture them.  Each captured step is replayed several
times with eager work and synchronisations in between, and every replay is checked against the
same steps run eagerly and against the oracle."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd._C import adam_op

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()


def host(t):
    return t.detach().cpu().numpy()


def test_inplace_multi_step_under_graph_replay():
    sizes = [5000, 17, 70_001, 256, 1]
    rng = np.random.default_rng(0)
    h_mu = [np.zeros(n, np.float32) for n in sizes]
    h_nu = [np.zeros(n, np.float32) for n in sizes]
    mu = [torch.zeros(n, device='cuda') for n in sizes]
    nu = [torch.zeros(n, device='cuda') for n in sizes]
    grads = [torch.zeros(n, device='cuda') for n in sizes]  # static input buffers
    count = 3  # fixed in the captured call: a graph freezes the scalars it was captured with

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream, as torch asks
        adam_op.forward_multi_([g.clone() for g in grads], [m.clone() for m in mu],
                               [v.clone() for v in nu], B1, B2, EPS, 0.0, count)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        adam_op.forward_multi_(grads, mu, nu, B1, B2, EPS, 0.0, count)

    for replay in range(4):
        fresh = [rng.standard_normal(n).astype(np.float32) for n in sizes]
        for g, f in zip(grads, fresh):
            g.copy_(torch.from_numpy(f))  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k, f in enumerate(fresh):
            O.forward_inplace(f, h_mu[k], h_nu[k], B1, B2, EPS, 0.0, count)
            assert_bit_equal(host(grads[k]), f, f'replay {replay} updates[{k}]')
            assert_bit_equal(host(mu[k]), h_mu[k], f'replay {replay} mu[{k}]')
            assert_bit_equal(host(nu[k]), h_nu[k], f'replay {replay} nu[{k}]')
        # an eager call between replays must not disturb the captured one
        adam_op.forward_mu(grads[0], mu[0], B1)


def test_split_ops_and_fused_step_under_graph_replay():
    n = 100_003
    rng = np.random.default_rng(1)
    g = torch.zeros(n, device='cuda', dtype=torch.float64)
    m = torch.from_numpy(0.1 * rng.standard_normal(n)).cuda()
    v = torch.from_numpy(np.abs(0.01 * rng.standard_normal(n))).cuda()
    p = torch.from_numpy(rng.standard_normal(n)).cuda()
    hm, hv, hp = host(m).copy(), host(v).copy(), host(p).copy()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        adam_op.forward_updates(adam_op.forward_mu(g, m, B1), adam_op.forward_nu(g, v, B2), B1, B2,
                                EPS, 1e-8, 2)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        new_m = adam_op.forward_mu(g, m, B1)  # outputs come from the graph's private pool
        new_v = adam_op.forward_nu(g, v, B2)
        new_u = adam_op.forward_updates(new_m, new_v, B1, B2, EPS, 1e-8, 2)
        adam_op.fused_step_(p, g, m, v, B1, B2, EPS, 1e-8, 2, 0.01)

    for replay in range(3):
        f = rng.standard_normal(n)
        g.copy_(torch.from_numpy(f))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        e_m, e_v = O.forward_mu(f, hm, B1), O.forward_nu(f, hv, B2)
        assert_bit_equal(host(new_m), e_m, f'replay {replay} forward_mu')
        assert_bit_equal(host(new_v), e_v, f'replay {replay} forward_nu')
        assert_bit_equal(host(new_u), O.forward_updates(e_m, e_v, B1, B2, EPS, 1e-8, 2),
                         f'replay {replay} forward_updates')
        O.fused_step(hp, f.copy(), hm, hv, B1, B2, EPS, 1e-8, 2, 0.01, False, False)
        assert_bit_equal(host(p), hp, f'replay {replay} params')
        assert_bit_equal(host(m), hm, f'replay {replay} mu')
        assert_bit_equal(host(g), f, f'replay {replay} gradient left alone')


def test_concurrent_callers_on_their_own_streams():
    """The library keeps no per-call state: threads launching on separate streams at the same
    time (as autograd's worker threads do for the backward ops) get independent, correct
    results."""
    import threading

    rng = np.random.default_rng(3)
    n, rounds = 200_003, 25
    jobs = []
    for k in range(4):
        g = rng.standard_normal(n).astype(np.float32)
        m = (0.1 * rng.standard_normal(n)).astype(np.float32)
        v = np.abs(0.01 * rng.standard_normal(n)).astype(np.float32)
        jobs.append({'host': (g, m, v), 'count': k + 1, 'out': None, 'err': None})

    def worker(job):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                dev = [torch.from_numpy(a).cuda() for a in job['host']]
                for _ in range(rounds):  # out-of-place ops: same inputs, same outputs, every time
                    mu1 = adam_op.forward_mu(dev[0], dev[1], 0.9)
                    nu1 = adam_op.forward_nu(dev[0], dev[2], 0.999)
                    up = adam_op.forward_updates(mu1, nu1, 0.9, 0.999, 1e-8, 0.0, job['count'])
                stream.synchronize()
                job['out'] = (mu1.cpu().numpy(), nu1.cpu().numpy(), up.cpu().numpy())
        except Exception as exc:  # noqa: BLE001
            job['err'] = exc

    threads = [threading.Thread(target=worker, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for k, job in enumerate(jobs):
        assert job['err'] is None, job['err']
        g, m, v = job['host']
        e_mu, e_nu = O.forward_mu(g, m, 0.9), O.forward_nu(g, v, 0.999)
        e_up = O.forward_updates(e_mu, e_nu, 0.9, 0.999, 1e-8, 0.0, job['count'])
        for got, want, what in zip(job['out'], (e_mu, e_nu, e_up), ('mu', 'nu', 'updates')):
            assert_bit_equal(got, want, f'thread {k} {what}')


# ------------------------------------------------------------------ the step number on the device


def capture(fn, warm):
    """torch's capture protocol: warm up on a side stream, then capture `fn`."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        warm()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return graph


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
def test_device_count_rows_and_clamping(dtype):
    """forward_devcount_ eagerly: the step number is whatever the device tensor holds; below the
    table's first step the first row serves, beyond its last step the last row."""
    from torchopt_amd._C import adam_op as A

    tdt = torch.from_numpy(np.zeros(1, dtype)).dtype
    rng = np.random.default_rng(4)
    n = 70_001
    first, rows = 3, 5  # steps 3..7
    table = A.bias_rows(tdt, B1, B2, 1e-8, first, rows).cuda()
    count = torch.zeros((), dtype=torch.int64, device='cuda')
    for step, served in ((1, 3), (3, 3), (5, 5), (7, 7), (12, 7)):
        g = rng.standard_normal(n).astype(dtype)
        m = (0.1 * rng.standard_normal(n)).astype(dtype)
        v = np.abs(0.01 * rng.standard_normal(n)).astype(dtype)
        dg, dm, dv = (torch.from_numpy(a).cuda() for a in (g, m, v))
        count.fill_(step)
        print(f'forward_devcount_ step {step} (row of step {served})', flush=True)
        A.forward_devcount_(dg, dm, dv, B1, B2, EPS, 1e-8, table, first, count)
        O.forward_inplace(g, m, v, B1, B2, EPS, 1e-8, served)
        assert_bit_equal(host(dg), g, f'step {step} updates')
        assert_bit_equal(host(dm), m, f'step {step} mu')
        assert_bit_equal(host(dv), v, f'step {step} nu')


def test_a_settled_table_is_exact_for_every_later_step():
    """bias_rows_needed: once b^count is below half an ulp of 1 the corrections stop changing, so
    a table that long serves any later step exactly."""
    from torchopt_amd._C import adam_op as A

    b1, b2 = 0.5, 0.6
    rows = A.bias_rows_needed(b1, b2, 1, 10_000)
    assert 60 < rows < 200
    assert A.bias_rows_needed(b1, b2, 1, rows - 1) == 0  # one row fewer is not enough
    table = A.bias_rows(torch.float64, b1, b2, 0.0, 1, rows).cuda()
    assert torch.equal(table[-1], table[-1] * 0 + 1)  # the fixed point: no correction at all
    assert not torch.equal(table[-2], table[-1])
    rng = np.random.default_rng(6)
    n = 5000
    count = torch.zeros((), dtype=torch.int64, device='cuda')
    for step in (rows - 1, rows, rows + 1, rows + 12_345, 2 ** 40):
        g = rng.standard_normal(n)
        m = 0.1 * rng.standard_normal(n)
        v = np.abs(0.01 * rng.standard_normal(n))
        dg, dm, dv = (torch.from_numpy(a).cuda() for a in (g, m, v))
        count.fill_(step)
        A.forward_devcount_(dg, dm, dv, b1, b2, EPS, 0.0, table, 1, count)
        O.forward_inplace(g, m, v, b1, b2, EPS, 0.0, step)
        assert_bit_equal(host(dg), g, f'step {step} updates')


def test_one_captured_graph_serves_ten_steps():
    """The list step with its count on the device, captured ONCE together with the kernel that
    advances the count: replay k is step k, bit-equal to the oracle run with counts 1..10."""
    from torchopt_amd._C import adam_op as A

    sizes = [5000, 17, 70_001, 256, 1, 256 * 9000 + 3]
    rng = np.random.default_rng(10)
    h_mu = [np.zeros(n, np.float32) for n in sizes]
    h_nu = [np.zeros(n, np.float32) for n in sizes]
    mu = [torch.zeros(n, device='cuda') for n in sizes]
    nu = [torch.zeros(n, device='cuda') for n in sizes]
    grads = [torch.zeros(n, device='cuda') for n in sizes]
    table = A.bias_rows(torch.float32, B1, B2, 0.0, 1, 64).cuda()
    count = torch.zeros((), dtype=torch.int64, device='cuda')

    def one_step():
        A.count_advance_(count)
        A.forward_multi_devcount_(grads, mu, nu, B1, B2, EPS, 0.0, table, 1, count)

    def warm():
        c = count.clone()
        A.count_advance_(c)
        A.forward_multi_devcount_([g.clone() for g in grads], [m.clone() for m in mu],
                                  [v.clone() for v in nu], B1, B2, EPS, 0.0, table, 1, c)

    print('capturing count_advance_ + forward_multi_devcount_', flush=True)
    graph = capture(one_step, warm)
    assert int(count) == 0  # capture runs nothing
    for step in range(1, 11):
        fresh = [rng.standard_normal(n).astype(np.float32) for n in sizes]
        for g, f in zip(grads, fresh):
            g.copy_(torch.from_numpy(f))  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(count) == step
        for k, f in enumerate(fresh):
            O.forward_inplace(f, h_mu[k], h_nu[k], B1, B2, EPS, 0.0, step)
            assert_bit_equal(host(grads[k]), f, f'step {step} updates[{k}]')
            assert_bit_equal(host(mu[k]), h_mu[k], f'step {step} mu[{k}]')
            assert_bit_equal(host(nu[k]), h_nu[k], f'step {step} nu[{k}]')
        A.forward_mu(grads[0], mu[0], B1)  # an eager call between replays


@pytest.mark.parametrize('kind', ['adam', 'adamw'])
def test_capturable_optimizer_in_one_graph(kind):
    """FusedAdam(capturable=True).step() captured once and replayed ten times against the same
    optimizer stepped eagerly with host-side counts, and against the oracle."""
    import torchopt_amd

    cls = torchopt_amd.FusedAdam if kind == 'adam' else torchopt_amd.FusedAdamW
    shapes = [(300, 7), (5,), (64, 64, 3), (1,)]
    rng = np.random.default_rng(12)
    init = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    p_graph = [torch.from_numpy(a.copy()).cuda().requires_grad_(True) for a in init]
    p_eager = [torch.from_numpy(a.copy()).cuda().requires_grad_(True) for a in init]
    for p in p_graph + p_eager:
        p.grad = torch.zeros_like(p)
    opt_graph = cls(p_graph, lr=0.01, weight_decay=0.02, eps_root=1e-8, capturable=True)
    opt_eager = cls(p_eager, lr=0.01, weight_decay=0.02, eps_root=1e-8)
    opt_graph.init_state()

    def warm():
        scratch = cls([p.detach().clone().requires_grad_(True) for p in p_graph], lr=0.01,
                      weight_decay=0.02, eps_root=1e-8, capturable=True)
        for q in scratch.param_groups[0]:
            q.grad = torch.zeros_like(q)
        scratch.step()

    print(f'capturing {cls.__name__}(capturable=True).step()', flush=True)
    graph = capture(opt_graph.step, warm)
    hp = [a.copy() for a in init]
    hm = [np.zeros_like(a) for a in init]
    hv = [np.zeros_like(a) for a in init]
    for step in range(1, 11):
        fresh = [rng.standard_normal(s).astype(np.float32) for s in shapes]
        for pg, pe, f in zip(p_graph, p_eager, fresh):
            pg.grad.copy_(torch.from_numpy(f))
            pe.grad.copy_(torch.from_numpy(f))
        torch.cuda.synchronize()
        graph.replay()
        opt_eager.step()
        torch.cuda.synchronize()
        for k, f in enumerate(fresh):
            O.fused_step(hp[k].reshape(-1), f.reshape(-1).copy(), hm[k].reshape(-1),
                         hv[k].reshape(-1), B1, B2, EPS, 1e-8, step, 0.01, False, False, 0.02,
                         kind == 'adamw')
            assert_bit_equal(host(p_graph[k]), hp[k], f'{kind} step {step} params[{k}] (graph)')
            assert_bit_equal(host(p_eager[k]), hp[k], f'{kind} step {step} params[{k}] (eager)')
    state = opt_graph.state_dict()[0]
    assert all(int(c) == 10 for c in state.count)
    assert_bit_equal(host(state.mu[0]), hm[0], 'mu after ten replays')
    # the same optimizer keeps going eagerly, from the device's count
    for pg, f in zip(p_graph, fresh):
        pg.grad.copy_(torch.from_numpy(f))
    opt_graph.step()
    for k, f in enumerate(fresh):
        O.fused_step(hp[k].reshape(-1), f.reshape(-1).copy(), hm[k].reshape(-1),
                     hv[k].reshape(-1), B1, B2, EPS, 1e-8, 11, 0.01, False, False, 0.02,
                     kind == 'adamw')
        assert_bit_equal(host(p_graph[k]), hp[k], f'{kind} eager step 11 params[{k}]')


def test_host_counted_steps_refuse_capture():
    """A captured step whose count lives on the host would replay one step number for ever:
    FusedAdam.step() without capturable=True and the transformation's update() say so instead."""
    import torchopt_amd
    from torchopt_amd.transform import scale_by_accelerated_adam

    p = torch.zeros(1000, device='cuda', requires_grad=True)
    p.grad = torch.ones_like(p)
    opt = torchopt_amd.FusedAdam([p], lr=0.1)
    opt.step()
    transform = scale_by_accelerated_adam()
    state = transform.init((p.detach(),))
    transform.update((p.grad.clone(),), state)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match='capturable=True'):
        with torch.cuda.graph(graph):
            opt.step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match='cannot be captured'):
        with torch.cuda.graph(graph):
            transform.update((p.grad,), state)
    torch.cuda.synchronize()
    opt.step()  # and the optimizer is fine afterwards
    torch.cuda.synchronize()
