"""Long lists through device-resident plans: one launch over a table in device memory, cached per
stream and list.  Results must equal the oracle's per tensor, whether the plan was just written,
found in the cache, rewritten for another list, shared by no one (two streams) or not used at
all (stream capture, plans switched off)."""

from __future__ import annotations

import ctypes
import threading

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from test_multi_tensor_gpu import check_lists, make_lists, run_all_multi, to_dev
from torchopt_amd import _lib
from torchopt_amd._C import adam_op

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8


@pytest.fixture(autouse=True)
def _defaults():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    lib = _lib.load()
    yield
    lib.toa_adam_set_plan_mode(0)
    torch.cuda.synchronize()


def ragged_sizes(num, seed):
    rng = np.random.default_rng(seed)
    sizes = [int(x) for x in rng.integers(0, 3000, size=num)]
    sizes[0], sizes[1], sizes[2], sizes[3] = 0, 1, 255, 257
    sizes[num // 3] = 300_001  # many tiles, so the tile groups of the plan are larger than one
    sizes[num // 2] = 256 * 700
    sizes[-1] = 100_003
    return sizes


def step_and_check(g, h, count, what):
    adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, count)
    for k in range(len(h['updates'])):
        O.forward_inplace(h['updates'][k], h['mu'][k], h['nu'][k], B1, B2, EPS, 0.0, count)
    check_lists(g['updates'], h['updates'], f'{what} updates')
    check_lists(g['mu'], h['mu'], f'{what} mu')
    check_lists(g['nu'], h['nu'], f'{what} nu')


@pytest.mark.parametrize('mode', [0, 1, 2])
@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
def test_all_ops_over_a_long_list(mode, dtype):
    """400 ragged tensors through every multi-tensor op: plans by default, several launches with
    plans switched off, and plans forced."""
    _lib.load().toa_adam_set_plan_mode(mode)
    print(f'all multi ops, 400 tensors, plan mode {mode}', flush=True)
    run_all_multi(dtype, ragged_sizes(400, 3), 17, 1e-8, 3)


def test_short_lists_through_forced_plans():
    _lib.load().toa_adam_set_plan_mode(2)
    print('all multi ops, short lists, plans forced', flush=True)
    run_all_multi(np.float32, [5, 0, 70_001, 256, 1], 4, 0.0, 2)
    run_all_multi(np.float32, [1000, 17, 5000, 256, 3, 70_000, 999, 1], 9, 0.0,
                  [1, 5, 1, 1000, 5, 2, 1000, 7])  # a plan per distinct count


def test_cached_plan_then_another_list_then_the_first_again():
    sizes = ragged_sizes(300, 5)
    h1, h2 = make_lists(np.float32, sizes, 1), make_lists(np.float32, sizes[::-1], 2)
    g1, g2 = to_dev(h1), to_dev(h2)
    print('plan written, reused, replaced', flush=True)
    for step in range(1, 4):  # written on the first step, found in the cache afterwards
        step_and_check(g1, h1, step, f'list 1 step {step}')
    step_and_check(g2, h2, 1, 'list 2')
    step_and_check(g1, h1, 4, 'list 1 again')
    # a list that differs from a cached one in a single pointer must not be taken for it
    spare = torch.from_numpy(h1['updates'][7].copy()).cuda()
    hs = h1['updates'][7].copy()
    g1['updates'][7], h1['updates'][7] = spare, hs
    step_and_check(g1, h1, 5, 'list 1 with one array elsewhere')
    # more lists than a stream keeps plans for: the oldest is rewritten
    others = []
    for k in range(18):  # a stream keeps 16
        s = ragged_sizes(130 + k, 20 + k)
        others.append((to_dev(make_lists(np.float32, s, 30 + k)), make_lists(np.float32, s, 30 + k)))
    for k, (g, h) in enumerate(others):
        step_and_check(g, h, 2, f'other list {k}')
    step_and_check(g1, h1, 6, 'list 1 after its plan was evicted')
    assert _lib.load().toa_adam_release_plans() == 0
    step_and_check(g1, h1, 7, 'list 1 after the plans were released')


def test_long_list_under_graph_capture_keeps_its_tables_in_the_launches():
    """A captured launch must not depend on memory a later call may rewrite: under capture a long
    list takes one launch per kernel-argument table, and replays stay right while eager calls
    with other long lists run in between."""
    sizes = ragged_sizes(250, 8)
    rng = np.random.default_rng(0)
    h = make_lists(np.float32, sizes, 6)
    g = to_dev(h)
    other_h = make_lists(np.float32, ragged_sizes(270, 9), 7)
    other_g = to_dev(other_h)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        adam_op.forward_multi_([t.clone() for t in g['updates']], [t.clone() for t in g['mu']],
                               [t.clone() for t in g['nu']], B1, B2, EPS, 0.0, 3)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    print('long list captured', flush=True)
    with torch.cuda.graph(graph):
        adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, 3)
    for replay in range(3):
        for k, n in enumerate(sizes):
            fresh = rng.standard_normal(n).astype(np.float32)
            g['updates'][k].copy_(torch.from_numpy(fresh))
            h['updates'][k] = fresh
        step_and_check(other_g, other_h, replay + 1, f'eager list between replays {replay}')
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k in range(len(sizes)):
            O.forward_inplace(h['updates'][k], h['mu'][k], h['nu'][k], B1, B2, EPS, 0.0, 3)
        check_lists(g['updates'], h['updates'], f'replay {replay} updates')
        check_lists(g['mu'], h['mu'], f'replay {replay} mu')
        check_lists(g['nu'], h['nu'], f'replay {replay} nu')


def test_two_streams_each_with_its_own_plans():
    jobs = []
    for k in range(3):
        sizes = ragged_sizes(200 + 10 * k, 40 + k)
        jobs.append({'h': make_lists(np.float32, sizes, 50 + k), 'err': None, 'out': None})

    def worker(job):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                g = to_dev(job['h'])
                for step in range(1, 6):
                    adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, step)
                stream.synchronize()
                job['out'] = {k: [t.cpu().numpy() for t in g[k]] for k in ('updates', 'mu', 'nu')}
        except Exception as exc:  # noqa: BLE001
            job['err'] = exc

    print('three threads, three streams, long lists', flush=True)
    threads = [threading.Thread(target=worker, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for j, job in enumerate(jobs):
        assert job['err'] is None, job['err']
        h = job['h']
        for step in range(1, 6):
            for k in range(len(h['updates'])):
                O.forward_inplace(h['updates'][k], h['mu'][k], h['nu'][k], B1, B2, EPS, 0.0, step)
        for key in ('updates', 'mu', 'nu'):
            for k, (got, want) in enumerate(zip(job['out'][key], h[key])):
                assert_bit_equal(got, want, f'thread {j} {key}[{k}]')


def test_fused_step_and_one_pass_ops_over_a_long_list():
    sizes = ragged_sizes(333, 11)
    rng = np.random.default_rng(12)
    h = make_lists(np.float64, sizes, 13)
    params = [rng.standard_normal(n) for n in sizes]
    g = to_dev(h)
    gp = [torch.from_numpy(p).cuda() for p in params]
    print('forward_all_multi, backward_all_multi, fused_step_multi_ over 333 tensors', flush=True)
    new_mu, new_nu, new_u = adam_op.forward_all_multi(g['updates'], g['mu'], g['nu'], B1, B2, EPS,
                                                      1e-8, 4)
    e_mu = [O.forward_mu(u, m, B1) for u, m in zip(h['updates'], h['mu'])]
    e_nu = [O.forward_nu(u, v, B2) for u, v in zip(h['updates'], h['nu'])]
    e_u = [O.forward_updates(m, v, B1, B2, EPS, 1e-8, 4) for m, v in zip(e_mu, e_nu)]
    check_lists(new_mu, e_mu, 'forward_all new_mu')
    check_lists(new_u, e_u, 'forward_all new_updates')
    du, dm, dn = adam_op.backward_all_multi(g['dupdates'], g['dmu'], g['dnu'], new_u, new_mu,
                                            g['updates'], B1, B2, 1e-8, 4)
    for k in range(len(sizes)):
        bm, bv = O.backward_updates(h['dupdates'][k], e_u[k], e_mu[k], B1, B2, 1e-8, 4)
        gu1, gm = O.backward_mu(h['dmu'][k] + bm, B1)
        gu2, gv = O.backward_nu(h['dnu'][k] + bv, h['updates'][k], B2)
        assert_bit_equal(dm[k].cpu().numpy(), gm, f'backward_all dmu[{k}]')
        assert_bit_equal(dn[k].cpu().numpy(), gv, f'backward_all dnu[{k}]')
        assert_bit_equal(du[k].cpu().numpy(), gu1 + gu2, f'backward_all dupdates[{k}]')
    adam_op.fused_step_multi_(gp, g['updates'], g['mu'], g['nu'], B1, B2, EPS, 1e-8, 4, 0.01,
                              weight_decay=0.02, decoupled=True)
    for k in range(len(sizes)):
        O.fused_step(params[k], h['updates'][k], h['mu'][k], h['nu'][k], B1, B2, EPS, 1e-8, 4,
                     0.01, False, False, 0.02, True)
    check_lists(gp, params, 'fused step params')
    check_lists(g['mu'], h['mu'], 'fused step mu')
    check_lists(g['nu'], h['nu'], 'fused step nu')


def test_a_remembered_call_is_only_taken_for_the_very_same_arguments():
    """A plan remembers the last call it served and serves a byte-for-byte repeat with one launch.
    Anything else -- one size changed under the same pointers, another op over the same lists,
    another schedule, a capturing stream -- must go the long way and still be right."""
    lib = _lib.load()
    sizes = ragged_sizes(200, 11)
    h = make_lists(np.float32, sizes, 3)
    g = to_dev(h)
    print('remembered calls: repeat, size change, other op, other schedule, capture', flush=True)
    for step in (1, 2, 3):  # 1 writes the plan, 2 and 3 are repeats
        step_and_check(g, h, step, f'repeat {step}')

    # the same arrays, one tensor shorter by a few elements: views of the same storage
    k = len(sizes) // 3
    short = sizes[k] - 1000
    gs = {name: list(g[name]) for name in ('updates', 'mu', 'nu')}
    hs = {name: list(h[name]) for name in ('updates', 'mu', 'nu')}
    keep = {name: h[name][k][short:].copy() for name in hs}
    for name in gs:
        gs[name][k] = g[name][k][:short]
        hs[name][k] = h[name][k][:short]
    step_and_check(gs, hs, 4, 'one tensor shorter')
    for name in keep:  # the tail beyond the shorter length was not touched
        assert_bit_equal(g[name][k][short:].cpu().numpy(), keep[name], f'{name} beyond the new length')
    step_and_check(g, h, 5, 'full length again')

    # another op over the same three lists plus parameters
    hp = [np.random.default_rng(50 + i).standard_normal(n).astype(np.float32)
          for i, n in enumerate(sizes)]
    gp = [torch.from_numpy(a).cuda() for a in hp]
    adam_op.fused_step_multi_(gp, g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, 6, 0.01,
                              write_updates=True)
    for i in range(len(sizes)):
        O.fused_step(hp[i], h['updates'][i], h['mu'][i], h['nu'][i], B1, B2, EPS, 0.0, 6, 0.01)
    check_lists(gp, hp, 'fused step params')
    check_lists(g['updates'], h['updates'], 'fused step updates')
    step_and_check(g, h, 7, 'in-place step after the fused one')

    for schedule in (2, 1, 0):
        lib.toa_adam_set_schedule(schedule)
        step_and_check(g, h, 8 + schedule, f'schedule {schedule}')
        step_and_check(g, h, 12 + schedule, f'schedule {schedule}, repeat')
    lib.toa_adam_set_schedule(0)

    # a capturing stream must not lean on the remembered plan
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, 20)  # warm, eager
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, 21)
    torch.cuda.synchronize()
    for i in range(len(sizes)):
        O.forward_inplace(h['updates'][i], h['mu'][i], h['nu'][i], B1, B2, EPS, 0.0, 20)
    assert lib.toa_adam_release_plans() == 0  # the replay below must not need any plan
    graph.replay()
    torch.cuda.synchronize()
    for i in range(len(sizes)):
        O.forward_inplace(h['updates'][i], h['mu'][i], h['nu'][i], B1, B2, EPS, 0.0, 21)
    check_lists(g['updates'], h['updates'], 'replayed capture updates')
    check_lists(g['mu'], h['mu'], 'replayed capture mu')


@pytest.mark.parametrize('sizes_of', ['ragged', 'one_tile_or_less', 'a_giant_among_thousands'])
def test_thousands_of_small_tensors_start_from_the_finer_index(sizes_of):
    """More records than twice the cells of the launch's coarse index: the plan carries a finer
    index in device memory and waves start from that.  Checked like every other list, over two
    steps (plan written, then found in the cache and the call remembered)."""
    rng = np.random.default_rng(11)
    if sizes_of == 'ragged':
        sizes = [int(x) for x in rng.integers(0, 3000, size=6000)]
    elif sizes_of == 'one_tile_or_less':
        sizes = [int(x) for x in rng.integers(1, 257, size=4000)]
    else:
        sizes = [int(x) for x in rng.integers(1, 600, size=5000)]
        sizes[2500] = 256 * 40_000 + 17  # shifts the index to coarser entries
    h = make_lists(np.float32, sizes, 12)
    g = to_dev(h)
    print(f'{len(sizes)} small tensors ({sizes_of}) through a plan with a finer index', flush=True)
    for step in (1, 2, 3):
        step_and_check(g, h, step, f'{sizes_of} step {step}')
