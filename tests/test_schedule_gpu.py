"""The two memory schedules of the in-place step -- plain (all loads, then all stores) and staged
(load g | load mu | store mu', load nu | store nu', store u') -- against the CPU oracle, bit for
bit, on tensors large enough to take the bandwidth-bound kernels; the fallback to the plain
schedule when the arrays of a tensor overlap; lists whose arrays lie 16 MiB apart (the layout that
collides in DRAM and makes a list pick the staged schedule by itself); the load orders of the
staged program and the per-call-site choice among them.  Correctness only: nothing here
asserts a speed."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import _lib

pytestmark = pytest.mark.gpu

B1, B2 = 0.9, 0.999
CODE = {'f32': _lib.TOA_F32, 'f64': _lib.TOA_F64, 'f16': _lib.TOA_F16, 'bf16': _lib.TOA_BF16}
TORCH = {'f32': torch.float32, 'f64': torch.float64, 'f16': torch.float16, 'bf16': torch.bfloat16}
# elements per 1 KiB tile, times more tiles than one round of workgroups (8192), plus a ragged tail
BIG = {'f32': 256 * 9000 + 77, 'f64': 128 * 9000 + 5, 'f16': 512 * 9000 + 301, 'bf16': 512 * 9000 + 301}


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    lib = _lib.load()
    yield
    lib.toa_adam_set_schedule(0)
    lib.toa_adam_set_waves_per_cu(0)
    lib.toa_adam_set_load_order(-1)
    lib.toa_adam_set_tuning(1)
    torch.cuda.synchronize()


def draw(tag, n, seed):
    rng = np.random.default_rng(seed)

    def fmt(x):
        if tag == 'bf16':
            return O.bf16_bits(x.astype(np.float32))
        return x.astype({'f32': np.float32, 'f64': np.float64, 'f16': np.float16}[tag])

    return [fmt(rng.standard_normal(n)), fmt(0.1 * rng.standard_normal(n)),
            fmt(np.abs(0.01 * rng.standard_normal(n)))]


def dev(a, tag):
    a = np.ascontiguousarray(a)
    if tag == 'bf16':
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def host(t, tag):
    if tag == 'bf16':
        return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.detach().cpu().numpy()


@pytest.mark.parametrize('tag', ['f32', 'f64', 'f16', 'bf16'])
@pytest.mark.parametrize('schedule', [0, 1, 2])
def test_both_schedules_match_the_oracle(tag, schedule):
    lib = _lib.load()
    n = BIG[tag]
    eps, eps_root, count = (1e-8, 1e-8, 7) if tag in ('f32', 'f64') else (1e-3, 0.0, 7)
    u, m, v = draw(tag, n, 11)
    want = O.forward_inplace(u.copy(), m.copy(), v.copy(), B1, B2, eps, eps_root, count)
    du, dm, dv = (dev(a, tag) for a in (u, m, v))
    assert lib.toa_adam_set_schedule(schedule) in (0, 1, 2)
    print(f'forward_inplace {tag} n={n} schedule={schedule}', flush=True)
    rc = lib.toa_adam_forward_inplace(CODE[tag], du.data_ptr(), dm.data_ptr(), dv.data_ptr(), n,
                                      B1, B2, eps, eps_root, count,
                                      torch.cuda.current_stream().cuda_stream)
    lib.toa_adam_set_schedule(0)
    assert rc == 0, lib.toa_adam_error_string(rc)
    for got, exp, name in zip((du, dm, dv), want, ('updates', 'mu', 'nu')):
        assert_bit_equal(host(got, tag), exp, f'{tag} schedule {schedule} {name}')


@pytest.mark.parametrize('levels', [(14, 16, 18, 21, 25, 32)])
def test_staged_schedule_at_every_residency_level(levels):
    """The level only bounds how many workgroups share a compute unit; results cannot depend on it."""
    lib = _lib.load()
    n = BIG['f32']
    u, m, v = draw('f32', n, 12)
    want = O.forward_inplace(u.copy(), m.copy(), v.copy(), B1, B2, 1e-8, 0.0, 1000)
    for w in levels:
        du, dm, dv = (dev(a, 'f32') for a in (u, m, v))
        lib.toa_adam_set_waves_per_cu(w)
        print(f'forward_inplace f32 n={n} staged waves={w}', flush=True)
        rc = lib.toa_adam_forward_inplace(CODE['f32'], du.data_ptr(), dm.data_ptr(),
                                          dv.data_ptr(), n, B1, B2, 1e-8, 0.0, 1000,
                                          torch.cuda.current_stream().cuda_stream)
        lib.toa_adam_set_waves_per_cu(0)
        assert rc == 0, lib.toa_adam_error_string(rc)
        for got, exp, name in zip((du, dm, dv), want, ('updates', 'mu', 'nu')):
            assert_bit_equal(host(got, 'f32'), exp, f'waves {w} {name}')


@pytest.mark.parametrize('tag', ['f32', 'f64', 'f16', 'bf16'])
def test_every_load_order_of_the_staged_step_matches_the_oracle(tag):
    """Which moment the staged program handles first, and whether it loads it before the
    gradient, moves the rate with the placement of the arrays and nothing else: all four orders
    (the 16-bit types have one, whatever is asked for), at the three residency levels around the default,
    give the oracle's bits -- through the host-counted and the device-counted entry point."""
    lib = _lib.load()
    n = BIG[tag]
    eps, eps_root, count = (1e-8, 1e-8, 7) if tag in ('f32', 'f64') else (1e-3, 0.0, 7)
    u, m, v = draw(tag, n, 21)
    want = O.forward_inplace(u.copy(), m.copy(), v.copy(), B1, B2, eps, eps_root, count)
    stream = torch.cuda.current_stream().cuda_stream
    rows = 4
    table = torch.empty(rows, 4, dtype=TORCH[tag])
    assert lib.toa_adam_bias_rows(CODE[tag], B1, B2, eps_root, count - 1, rows,
                                  table.data_ptr()) == 0
    table = table.cuda()
    step = torch.tensor(count, dtype=torch.int64, device='cuda')
    lib.toa_adam_set_schedule(2)
    try:
        for order in range(4):
            for waves in (16, 18, 21):
                lib.toa_adam_set_load_order(order)
                lib.toa_adam_set_waves_per_cu(waves)
                for devcount in (False, True):
                    du, dm, dv = (dev(a, tag) for a in (u, m, v))
                    print(f'forward_inplace {tag} n={n} staged order={order} waves={waves} '
                          f'devcount={devcount}', flush=True)
                    if devcount:
                        rc = lib.toa_adam_forward_inplace_devcount(
                            CODE[tag], du.data_ptr(), dm.data_ptr(), dv.data_ptr(), n, B1, B2, eps,
                            eps_root, table.data_ptr(), count - 1, rows, step.data_ptr(), stream)
                    else:
                        rc = lib.toa_adam_forward_inplace(
                            CODE[tag], du.data_ptr(), dm.data_ptr(), dv.data_ptr(), n, B1, B2, eps,
                            eps_root, count, stream)
                    assert rc == 0, lib.toa_adam_error_string(rc)
                    for got, exp, name in zip((du, dm, dv), want, ('updates', 'mu', 'nu')):
                        assert_bit_equal(host(got, tag), exp,
                                         f'{tag} order {order} waves {waves} {name}')
    finally:
        lib.toa_adam_set_schedule(0)
        lib.toa_adam_set_load_order(-1)
        lib.toa_adam_set_waves_per_cu(0)


@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_the_load_order_is_chosen_per_call_site_and_changes_no_bit(tag):
    """A call site of 64 MiB per array is explored over its first 30 launches (four load orders and the
    plain schedule, six rounds) and then keeps one of them; forty steps on it give the bits of forty steps with tuning
    off (order 0 throughout) -- and, for the first of them, the oracle's.  With tuning off, under
    a forced order or below the size limit no site is recorded."""
    lib = _lib.load()
    esize = {'f32': 4, 'f64': 8}[tag]
    n = (64 << 20) // esize + 1000  # whole tiles of 64 MiB and a ragged tail
    u, m, v = draw(tag, n, 31)
    first = O.forward_inplace(u.copy(), m.copy(), v.copy(), B1, B2, 1e-8, 1e-8, 1)
    stream = torch.cuda.current_stream().cuda_stream
    code = CODE[tag]

    def steps(arrays, count):
        for k in range(count):
            rc = lib.toa_adam_forward_inplace(code, *[a.data_ptr() for a in arrays], n, B1, B2,
                                              1e-8, 1e-8, k + 1, stream)
            assert rc == 0, lib.toa_adam_error_string(rc)

    tuned = [dev(a, tag) for a in (u, m, v)]
    plain = [dev(a, tag) for a in (u, m, v)]
    site = lambda arrays: lib.toa_adam_tuned_load_order(code, *[a.data_ptr() for a in arrays], n)

    lib.toa_adam_set_tuning(0)
    print(f'forward_inplace {tag} n={n} forty steps, tuning off', flush=True)
    steps(plain, 40)
    torch.cuda.synchronize()
    assert site(plain) == -1
    lib.toa_adam_set_tuning(1)
    assert site(tuned) == -1
    print(f'forward_inplace {tag} n={n} first step of a tuned site', flush=True)
    steps(tuned, 1)
    torch.cuda.synchronize()
    for got, exp, name in zip(tuned, first, ('updates', 'mu', 'nu')):
        assert_bit_equal(host(got, tag), exp, f'{tag} first tuned step {name}')
    print(f'forward_inplace {tag} n={n} thirty-nine more steps of the tuned site', flush=True)
    for k in range(1, 40):
        rc = lib.toa_adam_forward_inplace(code, *[a.data_ptr() for a in tuned], n, B1, B2, 1e-8,
                                          1e-8, k + 1, stream)
        assert rc == 0
        if k in (5, 29):
            assert site(tuned) == -1 or k == 29  # exploring: nothing is decided before 30 launches
    torch.cuda.synchronize()
    assert site(tuned) in (0, 1, 2, 3, 4)  # every sample is back: decided
    for a, b, name in zip(tuned, plain, ('updates', 'mu', 'nu')):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), f'{tag} tuned != untuned {name}'
    # no site for a forced order, a forced level, or arrays below the limit
    others = [dev(a, tag) for a in (u, m, v)]
    lib.toa_adam_set_load_order(2)
    steps(others, 2)
    lib.toa_adam_set_load_order(-1)
    lib.toa_adam_set_waves_per_cu(18)
    steps(others, 2)
    lib.toa_adam_set_waves_per_cu(0)
    torch.cuda.synchronize()
    assert site(others) == -1
    small = [t[:BIG[tag]] for t in others]
    rc = lib.toa_adam_forward_inplace(code, *[a.data_ptr() for a in small], BIG[tag], B1, B2, 1e-8,
                                      1e-8, 1, stream)
    assert rc == 0
    assert lib.toa_adam_tuned_load_order(code, *[a.data_ptr() for a in small], BIG[tag]) == -1


@pytest.mark.parametrize('alias', ['mu is nu', 'all three'])
def test_overlapping_arrays_keep_the_plain_schedule(alias):
    """The reference's CPU loop reads an element of all three arrays and then writes mu, nu,
    updates in that order (adam_op_impl_cpu.cpp:47-61), so with aliased arrays the last write
    wins.  The staged schedule would read nu after writing mu; the library must notice the overlap
    and keep the plain schedule, whose result is the reference's."""
    lib = _lib.load()
    n = BIG['f32']
    rng = np.random.default_rng(5)
    buf = (np.abs(0.05 * rng.standard_normal(n)) + 1e-3).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    dbuf, dg = dev(buf, 'f32'), dev(g, 'f32')
    if alias == 'mu is nu':
        O.forward_inplace(g, buf, buf, B1, B2, 1e-8, 0.0, 3)  # same array twice, as on the GPU
        pu = dg.data_ptr()
    else:
        O.forward_inplace(buf, buf, buf, B1, B2, 1e-8, 0.0, 3)
        pu = dbuf.data_ptr()
    lib.toa_adam_set_schedule(2)  # staged wherever it is legal: here it is not
    print(f'forward_inplace f32 n={n} aliased: {alias}', flush=True)
    rc = lib.toa_adam_forward_inplace(CODE['f32'], pu, dbuf.data_ptr(), dbuf.data_ptr(), n, B1,
                                      B2, 1e-8, 0.0, 3, torch.cuda.current_stream().cuda_stream)
    lib.toa_adam_set_schedule(0)
    assert rc == 0, lib.toa_adam_error_string(rc)
    assert_bit_equal(host(dbuf, 'f32'), buf, f'aliased ({alias}) state')
    if alias == 'mu is nu':
        assert_bit_equal(host(dg, 'f32'), g, f'aliased ({alias}) updates')


@pytest.mark.parametrize('schedule', [0, 1, 2])
def test_list_with_colliding_arrays(schedule):
    """Leaves whose three arrays lie exactly 16 MiB apart (GPT-2-medium's 4096 x 1024 float32
    weights allocated side by side): the list picks the staged schedule by itself."""
    lib = _lib.load()
    S, K = 4 << 20, 3  # 16 MiB arrays, three leaves; plus one small ragged leaf elsewhere
    rng = np.random.default_rng(8)
    arena = (np.abs(0.05 * rng.standard_normal(3 * S * K)) + 1e-3).astype(np.float32)
    small = [a.astype(np.float32) for a in draw('f32', 70_001, 9)]
    d_arena = dev(arena, 'f32')
    d_small = [dev(a, 'f32') for a in small]
    base = d_arena.data_ptr()
    pu = [base + 4 * (3 * k) * S for k in range(K)] + [d_small[0].data_ptr()]
    pm = [p + 4 * S for p in pu[:K]] + [d_small[1].data_ptr()]
    pv = [p + 8 * S for p in pu[:K]] + [d_small[2].data_ptr()]
    ns = [S] * K + [70_001]
    num = K + 1
    arr = lambda ps: (ctypes.c_void_p * num)(*ps)
    lib.toa_adam_set_schedule(schedule)
    print(f'forward_inplace_multi f32 colliding list schedule={schedule}', flush=True)
    rc = lib.toa_adam_forward_inplace_multi(CODE['f32'], num, arr(pu), arr(pm), arr(pv),
                                            (ctypes.c_size_t * num)(*ns), B1, B2, 1e-8, 0.0, None,
                                            4, torch.cuda.current_stream().cuda_stream)
    lib.toa_adam_set_schedule(0)
    assert rc == 0, lib.toa_adam_error_string(rc)
    got = host(d_arena, 'f32')
    for k in range(K):
        u, m, v = (arena[(3 * k + a) * S:(3 * k + a + 1) * S].copy() for a in range(3))
        O.forward_inplace(u, m, v, B1, B2, 1e-8, 0.0, 4)
        for a, exp, name in zip(range(3), (u, m, v), ('updates', 'mu', 'nu')):
            assert_bit_equal(got[(3 * k + a) * S:(3 * k + a + 1) * S], exp, f'leaf {k} {name}')
    O.forward_inplace(small[0], small[1], small[2], B1, B2, 1e-8, 0.0, 4)
    for t, exp, name in zip(d_small, small, ('updates', 'mu', 'nu')):
        assert_bit_equal(host(t, 'f32'), exp, f'small leaf {name}')


@pytest.mark.parametrize('tag', ['f32', 'f64', 'f16', 'bf16'])
@pytest.mark.parametrize('schedule', [1, 2])
def test_forward_all_both_schedules(tag, schedule):
    """The one-pass differentiable forward equals forward_mu, forward_nu, forward_updates."""
    lib = _lib.load()
    n = BIG[tag]
    eps, eps_root, count = (1e-8, 1e-8, 3) if tag in ('f32', 'f64') else (1e-3, 0.0, 3)
    u, m, v = draw(tag, n, 21)
    e_mu, e_nu = O.forward_mu(u, m, B1), O.forward_nu(u, v, B2)
    e_u = O.forward_updates(e_mu, e_nu, B1, B2, eps, eps_root, count)
    du, dm, dv = (dev(a, tag) for a in (u, m, v))
    outs = [torch.empty_like(du) for _ in range(3)]
    lib.toa_adam_set_schedule(schedule)
    print(f'forward_all {tag} n={n} schedule={schedule}', flush=True)
    rc = lib.toa_adam_forward_all(CODE[tag], du.data_ptr(), dm.data_ptr(), dv.data_ptr(), n, B1,
                                  B2, eps, eps_root, count, outs[0].data_ptr(),
                                  outs[1].data_ptr(), outs[2].data_ptr(),
                                  torch.cuda.current_stream().cuda_stream)
    lib.toa_adam_set_schedule(0)
    assert rc == 0, lib.toa_adam_error_string(rc)
    for got, exp, name in zip(outs, (e_mu, e_nu, e_u), ('new_mu', 'new_nu', 'new_updates')):
        assert_bit_equal(host(got, tag), exp, f'{tag} schedule {schedule} {name}')
    for got, exp, name in zip((du, dm, dv), (u, m, v), ('updates', 'mu', 'nu')):
        assert_bit_equal(host(got, tag), exp, f'{tag} schedule {schedule} input {name} untouched')


@pytest.mark.parametrize('tag', ['f32', 'f64'])
@pytest.mark.parametrize('schedule', [0, 1, 2])
@pytest.mark.parametrize('variant', ['adam', 'adam maximize', 'adam + L2', 'adamw', 'adamw maximize'])
def test_fused_step_both_schedules(tag, schedule, variant):
    lib = _lib.load()
    n = BIG[tag]
    wd = 0.0 if variant.startswith('adam') and '+' not in variant and 'w' not in variant else 0.02
    decoupled, maximize = 'adamw' in variant, 'maximize' in variant
    write_updates = variant in ('adam', 'adamw maximize')
    rng = np.random.default_rng(31)
    np_t = {'f32': np.float32, 'f64': np.float64}[tag]
    p = rng.standard_normal(n).astype(np_t)
    g, m, v = draw(tag, n, 32)
    dp, dg, dm, dv = (dev(a, tag) for a in (p, g, m, v))
    O.fused_step(p, g, m, v, B1, B2, 1e-8, 1e-8, 9, 0.01, maximize, write_updates, wd, decoupled)
    lib.toa_adam_set_schedule(schedule)
    print(f'fused_step {tag} n={n} schedule={schedule} {variant}', flush=True)
    rc = lib.toa_adam_fused_step(CODE[tag], dp.data_ptr(), dg.data_ptr(), dm.data_ptr(),
                                 dv.data_ptr(), n, B1, B2, 1e-8, 1e-8, 9, 0.01, wd, int(decoupled),
                                 int(maximize), int(write_updates),
                                 torch.cuda.current_stream().cuda_stream)
    lib.toa_adam_set_schedule(0)
    assert rc == 0, lib.toa_adam_error_string(rc)
    for got, exp, name in zip((dp, dg, dm, dv), (p, g, m, v), ('params', 'updates', 'mu', 'nu')):
        assert_bit_equal(host(got, tag), exp, f'{tag} schedule {schedule} {variant} {name}')


def test_fused_step_list_takes_the_staged_schedule():
    """A ragged list through toa_adam_fused_step_multi (lists are staged for this op)."""
    lib = _lib.load()
    sizes = [BIG['f32'], 5, 0, 70_001, 256 * 8200]
    rng = np.random.default_rng(41)
    host_lists = []
    for k, n in enumerate(sizes):
        g, m, v = draw('f32', n, 42 + k)
        host_lists.append([rng.standard_normal(n).astype(np.float32), g, m, v])
    dev_lists = [[dev(a, 'f32') for a in leaf] for leaf in host_lists]
    num = len(sizes)
    col = lambda j: (ctypes.c_void_p * num)(*[leaf[j].data_ptr() for leaf in dev_lists])
    print('fused_step_multi f32 ragged list', flush=True)
    rc = lib.toa_adam_fused_step_multi(CODE['f32'], num, col(0), col(1), col(2), col(3),
                                       (ctypes.c_size_t * num)(*sizes), B1, B2, 1e-8, 0.0, None, 2,
                                       1e-3, 0.01, 1, 0, 1, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.toa_adam_error_string(rc)
    for k, (h, d) in enumerate(zip(host_lists, dev_lists)):
        O.fused_step(h[0], h[1], h[2], h[3], B1, B2, 1e-8, 0.0, 2, 1e-3, False, True, 0.01, True)
        for got, exp, name in zip(d, h, ('params', 'updates', 'mu', 'nu')):
            assert_bit_equal(host(got, 'f32'), exp, f'leaf {k} {name}')


@pytest.mark.parametrize('tag', ['f32', 'f64', 'f16'])
@pytest.mark.parametrize('schedule', [1, 2])
@pytest.mark.parametrize('outside', ['both', 'mu only', 'none'])
def test_backward_all_both_schedules(tag, schedule, outside):
    """The one-pass backward equals backward_updates, autograd's additions, backward_mu and
    backward_nu, whichever order the wave issues its memory operations in."""
    lib = _lib.load()
    n = BIG[tag]
    eps, eps_root, count = (1e-8, 1e-8, 3) if tag in ('f32', 'f64') else (1e-3, 1e-4, 3)
    g, m, v = draw(tag, n, 51)
    d_u, d_m, d_v = draw(tag, n, 52)
    e_mu, e_nu = O.forward_mu(g, m, B1), O.forward_nu(g, v, B2)
    e_u = O.forward_updates(e_mu, e_nu, B1, B2, eps, eps_root, count)
    bm, bv = O.backward_updates(d_u, e_u, e_mu, B1, B2, eps_root, count)
    has_m, has_v = outside in ('both', 'mu only'), outside == 'both'
    # the sums autograd forms where a gradient reaches new_mu / new_nu from outside as well
    from torchopt_amd._C import adam_op as A

    def plus(a, b):  # a + b in the element type's own arithmetic, on the GPU
        return host(dev(a, tag) + dev(b, tag), tag)

    tot_m = plus(d_m, bm) if has_m else bm
    tot_v = plus(d_v, bv) if has_v else bv
    gu1, gm = O.backward_mu(tot_m, B1)
    gu2, gv = O.backward_nu(tot_v, g, B2)
    want_du = plus(gu1, gu2)
    t = {k: dev(a, tag) for k, a in (('du', d_u), ('nu_', e_u), ('nm', e_mu), ('g', g),
                                     ('dm', d_m), ('dv', d_v))}
    outs = [torch.empty_like(t['g']) for _ in range(3)]
    lib.toa_adam_set_schedule(schedule)
    print(f'backward_all {tag} n={n} schedule={schedule} outside gradients: {outside}', flush=True)
    rc = lib.toa_adam_backward_all(CODE[tag], t['du'].data_ptr(), t['nu_'].data_ptr(),
                                   t['nm'].data_ptr(), t['g'].data_ptr(),
                                   t['dm'].data_ptr() if has_m else None,
                                   t['dv'].data_ptr() if has_v else None, n, B1, B2, eps_root,
                                   count, outs[0].data_ptr(), outs[1].data_ptr(),
                                   outs[2].data_ptr(), torch.cuda.current_stream().cuda_stream)
    lib.toa_adam_set_schedule(0)
    assert rc == 0, lib.toa_adam_error_string(rc)
    assert_bit_equal(host(outs[1], tag), gm, f'{tag} {outside} d(mu)')
    assert_bit_equal(host(outs[2], tag), gv, f'{tag} {outside} d(nu)')
    assert_bit_equal(host(outs[0], tag), want_du, f'{tag} {outside} d(updates)')
    del A


def test_fc_weight_list_parity_on_the_colliding_layout():
    """64 leaves of 4096 x 1024 float32 (GPT-2-medium's fc weight, 16 MiB), the gradient, mu and nu
    lists each contiguous: every leaf's arrays lie 1 GiB = 64 x 16 MiB apart and meet in the same
    DRAM banks, so the list picks the staged schedule by itself.  Results equal the oracle's bit
    for bit.  (What the layout costs in time is held by tests/test_perf_gates.py, under its own
    marker.)"""
    lib = _lib.load()
    leaf, K = 4096 * 1024, 64
    total = leaf * K
    stream = torch.cuda.current_stream().cuda_stream
    g, m, v = draw('f32', total, 61)
    ns = (ctypes.c_size_t * K)(*([leaf] * K))
    arena = torch.empty(3 * total, device='cuda', dtype=torch.float32)
    lists = [arena[j * total:(j + 1) * total] for j in range(3)]
    ptrs = [(ctypes.c_void_p * K)(*[t.data_ptr() + 4 * leaf * k for k in range(K)])
            for t in lists]
    for t, a in zip(lists, (g, m, v)):
        t.copy_(torch.from_numpy(a))
    print('forward_inplace_multi f32, 64 leaves of 16 MiB, lists contiguous', flush=True)
    rc = lib.toa_adam_forward_inplace_multi(CODE['f32'], K, ptrs[0], ptrs[1], ptrs[2], ns, B1, B2,
                                            1e-8, 0.0, None, 7, stream)
    assert rc == 0, lib.toa_adam_error_string(rc)
    got = [host(t, 'f32') for t in lists]
    O.forward_inplace(g, m, v, B1, B2, 1e-8, 0.0, 7)  # leaves share the scalars: one flat pass
    for a, exp, name in zip(got, (g, m, v), ('updates', 'mu', 'nu')):
        assert_bit_equal(a, exp, f'colliding layout {name}')
