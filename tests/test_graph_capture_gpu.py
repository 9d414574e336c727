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
