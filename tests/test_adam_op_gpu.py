"""Parity of the HIP path with the CPU oracle, on a real MI355X.

Every comparison is bit for bit (NaNs compared as NaNs): the kernels follow the reference's
rounding sequence, so the stated tolerance -- 2 ulp for float32, 1e-12 relative for float64 --
is met with zero slack.  `assert_parity` states that tolerance and then the stronger claim.

Two routes into the kernels are exercised: the raw C ABI (ctypes on libtoa_adam.so with device
pointers) and the Python surface `torchopt_amd._C.adam_op` that callers of the reference's
`torchopt._C.adam_op` would import instead.
"""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal, hyper_of, load_golden, ulp_distance
from oracle import adam_oracle as O
from torchopt_amd import _lib
from torchopt_amd._C import adam_op

pytestmark = pytest.mark.gpu

NP = {'f32': np.float32, 'f64': np.float64}
CODE = {'f32': _lib.TOA_F32, 'f64': _lib.TOA_F64}
HYPERS = [(0.9, 0.999, 1e-8, 0.0, 10), (0.9, 0.999, 1e-8, 1e-8, 5), (0.8, 0.95, 1e-6, 1e-10, 77)]
SIZES = [1, 2, 3, 4, 5, 7, 255, 256, 1023, 1024, 1025, 4095, 4096, 4097, 8191, 12289, 65537,
         1 << 20, (1 << 20) + 3,
         (1 << 22) + 777]  # whole tiles to the branch-free kernel, the ragged tail to the general one


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    _lib.load()
    yield
    torch.cuda.synchronize()


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy()


def assert_parity(got: np.ndarray, want: np.ndarray, what: str):
    """The contract (<= 2 ulp float32, <= 1e-12 relative float64), then bit equality."""
    d = ulp_distance(got, want)
    if got.dtype == np.float32:
        assert d.max(initial=0) <= 2, f'{what}: {d.max()} ulp'
    else:
        with np.errstate(all='ignore'):
            fin = np.isfinite(want) & (want != 0)
            rel = np.abs(got[fin] - want[fin]) / np.abs(want[fin])
        assert rel.max(initial=0) <= 1e-12, f'{what}: rel {rel.max()}'
        assert d.max(initial=0) <= 2, f'{what}: {d.max()} ulp'
    assert_bit_equal(got, want, what)


def rand(dtype, n, seed):
    rng = np.random.default_rng(seed)
    return {
        'updates': rng.standard_normal(n).astype(dtype),
        'mu': (0.1 * rng.standard_normal(n)).astype(dtype),
        'nu': np.abs(0.01 * rng.standard_normal(n)).astype(dtype),
        'dmu': rng.standard_normal(n).astype(dtype),
        'dnu': rng.standard_normal(n).astype(dtype),
        'dupdates': rng.standard_normal(n).astype(dtype),
    }


# ------------------------------------------------------------------ the two routes to the GPU


class CAbi:
    """Raw C ABI on device pointers; outputs allocated here."""

    def __init__(self, tag):
        self.code = CODE[tag]
        self.lib = _lib.load()
        self.stream = torch.cuda.current_stream().cuda_stream

    def _ok(self, rc):
        assert rc == 0, self.lib.toa_adam_error_string(rc)

    def forward_(self, u, m, v, b1, b2, eps, er, c):
        self._ok(self.lib.toa_adam_forward_inplace(self.code, u.data_ptr(), m.data_ptr(),
                                                   v.data_ptr(), u.numel(), b1, b2, eps, er, c,
                                                   self.stream))
        return u, m, v

    def forward_mu(self, u, m, b1):
        out = torch.empty_like(m)
        self._ok(self.lib.toa_adam_forward_mu(self.code, u.data_ptr(), m.data_ptr(), u.numel(),
                                              b1, out.data_ptr(), self.stream))
        return out

    def forward_nu(self, u, v, b2):
        out = torch.empty_like(v)
        self._ok(self.lib.toa_adam_forward_nu(self.code, u.data_ptr(), v.data_ptr(), u.numel(),
                                              b2, out.data_ptr(), self.stream))
        return out

    def forward_updates(self, m, v, b1, b2, eps, er, c):
        out = torch.empty_like(m)
        self._ok(self.lib.toa_adam_forward_updates(self.code, m.data_ptr(), v.data_ptr(),
                                                   m.numel(), b1, b2, eps, er, c,
                                                   out.data_ptr(), self.stream))
        return out

    def backward_mu(self, d, u, m, b1):
        o1, o2 = torch.empty_like(d), torch.empty_like(d)
        self._ok(self.lib.toa_adam_backward_mu(self.code, d.data_ptr(), d.numel(), b1,
                                               o1.data_ptr(), o2.data_ptr(), self.stream))
        return o1, o2

    def backward_nu(self, d, u, v, b2):
        o1, o2 = torch.empty_like(d), torch.empty_like(d)
        self._ok(self.lib.toa_adam_backward_nu(self.code, d.data_ptr(), u.data_ptr(), d.numel(),
                                               b2, o1.data_ptr(), o2.data_ptr(), self.stream))
        return o1, o2

    def backward_updates(self, d, u, m, v, b1, b2, er, c):
        o1, o2 = torch.empty_like(d), torch.empty_like(d)
        self._ok(self.lib.toa_adam_backward_updates(self.code, d.data_ptr(), u.data_ptr(),
                                                    m.data_ptr(), d.numel(), b1, b2, er, c,
                                                    o1.data_ptr(), o2.data_ptr(), self.stream))
        return o1, o2


class Module:
    """The drop-in Python module."""

    def __init__(self, tag):
        pass

    forward_ = staticmethod(adam_op.forward_)
    forward_mu = staticmethod(adam_op.forward_mu)
    forward_nu = staticmethod(adam_op.forward_nu)
    forward_updates = staticmethod(adam_op.forward_updates)
    backward_mu = staticmethod(adam_op.backward_mu)
    backward_nu = staticmethod(adam_op.backward_nu)
    backward_updates = staticmethod(adam_op.backward_updates)


ROUTES = {'cabi': CAbi, 'module': Module}


def check_all_seven(route, inp, hyper, label, exp=None):
    """Run the seven functions on the GPU and compare with `exp` (golden arrays) or the oracle."""
    b1, b2, eps, er, c = hyper
    u, m, v = inp['updates'], inp['mu'], inp['nu']
    with np.errstate(all='ignore'):
        if exp is None:
            ou, om, ov = O.forward_inplace(u.copy(), m.copy(), v.copy(), b1, b2, eps, er, c)
            exp = {
                'new_mu': O.forward_mu(u, m, b1), 'new_nu': O.forward_nu(u, v, b2),
                'inplace_updates': ou, 'inplace_mu': om, 'inplace_nu': ov,
            }
            exp['new_updates'] = O.forward_updates(exp['new_mu'], exp['new_nu'], b1, b2, eps, er,
                                                   c)
            exp['bmu_dupdates'], exp['bmu_dmu'] = O.backward_mu(inp['dmu'], b1)
            exp['bnu_dupdates'], exp['bnu_dnu'] = O.backward_nu(inp['dnu'], u, b2)
            exp['bup_dnew_mu'], exp['bup_dnew_nu'] = O.backward_updates(
                inp['dupdates'], exp['new_updates'], exp['new_mu'], b1, b2, er, c)
    g = {k: dev(a) for k, a in inp.items()}
    new_mu = route.forward_mu(g['updates'], g['mu'], b1)
    new_nu = route.forward_nu(g['updates'], g['nu'], b2)
    assert_parity(host(new_mu), exp['new_mu'], f'{label} forward_mu')
    assert_parity(host(new_nu), exp['new_nu'], f'{label} forward_nu')
    # inputs must be untouched by the out-of-place ops
    assert_bit_equal(host(g['updates']), u, f'{label} forward_mu/nu clobbered updates')
    assert_bit_equal(host(g['mu']), m, f'{label} forward_mu clobbered mu')
    emu, env = dev(exp['new_mu']), dev(exp['new_nu'])
    new_u = route.forward_updates(emu, env, b1, b2, eps, er, c)
    assert_parity(host(new_u), exp['new_updates'], f'{label} forward_updates')
    iu, im, iv = g['updates'].clone(), g['mu'].clone(), g['nu'].clone()
    r = route.forward_(iu, im, iv, b1, b2, eps, er, c)
    assert r[0] is iu and r[1] is im and r[2] is iv
    assert_parity(host(iu), exp['inplace_updates'], f'{label} forward_ updates')
    assert_parity(host(im), exp['inplace_mu'], f'{label} forward_ mu')
    assert_parity(host(iv), exp['inplace_nu'], f'{label} forward_ nu')
    du, dm = route.backward_mu(g['dmu'], g['updates'], g['mu'], b1)
    assert_parity(host(du), exp['bmu_dupdates'], f'{label} backward_mu dupdates')
    assert_parity(host(dm), exp['bmu_dmu'], f'{label} backward_mu dmu')
    du, dn = route.backward_nu(g['dnu'], g['updates'], g['nu'], b2)
    assert_parity(host(du), exp['bnu_dupdates'], f'{label} backward_nu dupdates')
    assert_parity(host(dn), exp['bnu_dnu'], f'{label} backward_nu dnu')
    dm, dn = route.backward_updates(g['dupdates'], dev(exp['new_updates']), emu, env, b1, b2, er,
                                    c)
    assert_parity(host(dm), exp['bup_dnew_mu'], f'{label} backward_updates dnew_mu')
    assert_parity(host(dn), exp['bup_dnew_nu'], f'{label} backward_updates dnew_nu')


# ------------------------------------------------------------------------------------ tests


@pytest.mark.parametrize('via', ['cabi', 'module'])
@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_golden_vectors(tag, via):
    """The reference CPU op's own outputs, including the special-value grid."""
    route = ROUTES[via](tag)
    for name, case in sorted(load_golden(tag).items()):
        inp = {k: case[k] for k in ('updates', 'mu', 'nu', 'dmu', 'dnu', 'dupdates')}
        check_all_seven(route, inp, hyper_of(case), f'{tag}/{name}', exp=case)


@pytest.mark.parametrize('via', ['cabi', 'module'])
@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_sizes_against_oracle(tag, via):
    """Lengths around every boundary of the kernels: vector width, workgroup, tile, grid."""
    route = ROUTES[via](tag)
    for k, n in enumerate(SIZES):
        hyper = HYPERS[k % len(HYPERS)]
        check_all_seven(route, rand(NP[tag], n, 1000 + n), hyper, f'{tag}/n={n}')


@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_operands_over_the_whole_exponent_range(tag):
    """Operands drawn uniformly over the finite BIT PATTERNS of the type -- every exponent equally
    likely, denormals and values next to overflow included -- so that the division, the root and
    the long product of backward_updates meet underflow, overflow and gradual underflow at
    random; whole-tile kernel and ragged tail."""
    route = ROUTES['module'](tag)
    n = (1 << 22) + 37
    rng = np.random.default_rng(20)
    it, ft = (np.uint32, np.float32) if tag == 'f32' else (np.uint64, np.float64)
    top = int(np.array(np.inf, ft).view(it))  # patterns below it: the finite non-negative values

    def draw(nonneg=False):
        bits = rng.integers(0, top, size=n, dtype=it)
        if not nonneg:
            bits |= rng.integers(0, 2, size=n, dtype=it) << it(8 * bits.itemsize - 1)
        return bits.view(ft)

    inp = {'updates': draw(), 'mu': draw(), 'nu': draw(nonneg=True), 'dmu': draw(),
           'dnu': draw(), 'dupdates': draw()}
    for hyper in ((0.9, 0.999, 1e-8, 0.0, 1), (0.9, 0.999, 1e-8, 1e-8, 4)):
        check_all_seven(route, inp, hyper, f'{tag}/whole exponent range {hyper}')


@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_zero_mu_branch_and_specials_in_backward_updates(tag):
    dtype = NP[tag]
    inp = rand(dtype, 5000, 3)
    b1, b2, eps, er, c = HYPERS[1]
    new_mu = O.forward_mu(inp['updates'], inp['mu'], b1)
    new_nu = O.forward_nu(inp['updates'], inp['nu'], b2)
    new_u = O.forward_updates(new_mu, new_nu, b1, b2, eps, er, c)
    new_mu[::3] = 0.0
    new_mu[1::7] = -0.0
    new_mu[5::11] = np.nan
    new_mu[6::13] = np.inf
    new_u[2::17] = np.inf
    with np.errstate(all='ignore'):
        em, en = O.backward_updates(inp['dupdates'], new_u, new_mu, b1, b2, er, c)
    gm, gn = adam_op.backward_updates(dev(inp['dupdates']), dev(new_u), dev(new_mu), dev(new_nu),
                                      b1, b2, er, c)
    assert_parity(host(gm), em, 'dnew_mu')
    assert_parity(host(gn), en, 'dnew_nu')
    zeros = new_mu == 0  # both signs of zero
    assert zeros.sum() > 1000
    for out in (host(gm), host(gn)):
        assert np.all(out[zeros] == 0) and not np.any(np.signbit(out[zeros]))


@pytest.mark.parametrize('tag', ['f32', 'f64'])
@pytest.mark.parametrize('offset', [1, 2, 3])
def test_misaligned_pointers(tag, offset):
    """Views that start off a 16-byte boundary take the element-wise path; same results."""
    dtype = NP[tag]
    n = 70001
    inp = rand(dtype, n + 4, 50 + offset)
    b1, b2, eps, er, c = HYPERS[0]
    cut = {k: a[offset:offset + n] for k, a in inp.items()}
    ou, om, ov = O.forward_inplace(cut['updates'].copy(), cut['mu'].copy(), cut['nu'].copy(), b1,
                                   b2, eps, er, c)
    full = {k: dev(a) for k, a in inp.items()}
    gu, gm, gv = (full[k][offset:offset + n] for k in ('updates', 'mu', 'nu'))
    # (two doubles are 16 bytes: that offset stays on the vector path, with a shifted base)
    assert (gu.data_ptr() % 16 != 0) == (offset * gu.element_size() % 16 != 0)
    adam_op.forward_(gu, gm, gv, b1, b2, eps, er, c)
    assert_parity(host(gu), ou, 'updates')
    assert_parity(host(gm), om, 'mu')
    assert_parity(host(gv), ov, 'nu')
    # nothing outside the view was written
    for k in ('updates', 'mu', 'nu'):
        h = host(full[k])
        assert_bit_equal(h[:offset], inp[k][:offset], 'head guard')
        assert_bit_equal(h[offset + n:], inp[k][offset + n:], 'tail guard')
    # only one operand misaligned: mu aligned, updates not
    mu_al = dev(cut['mu'])
    out = adam_op.forward_mu(full['dmu'][offset:offset + n], mu_al, b1)
    assert_parity(host(out), O.forward_mu(cut['dmu'], cut['mu'], b1), 'mixed alignment')


def test_tail_guard_aligned():
    """The vector path must not write past n when n is not a multiple of the vector width."""
    for tag in ('f32', 'f64'):
        dtype = NP[tag]
        for n in (1, 5, 4097, 12291):
            inp = rand(dtype, n + 8, n)
            full = {k: dev(a) for k, a in inp.items()}
            adam_op.forward_(full['updates'][:n], full['mu'][:n], full['nu'][:n], *HYPERS[0])
            for k in ('updates', 'mu', 'nu'):
                assert_bit_equal(host(full[k])[n:], inp[k][n:], f'{tag} n={n} {k} tail')


def test_stride_loop_when_tiles_exceed_the_grid_cap():
    """Tensors with more tiles than the launch cap are covered by the kernels' stride loop; with
    the cap lowered to a handful of workgroups the same code runs on a small input."""
    lib = _lib.load()
    prev = lib.toa_adam_set_max_grid(7)
    try:
        for tag in ('f32', 'f64'):
            route = ROUTES['module'](tag)
            check_all_seven(route, rand(NP[tag], 100_003, 17), HYPERS[1], f'{tag}/cap=7')
        sizes = [5000, 3, 70_001, 256]
        hs = [rand(np.float32, n, 60 + k) for k, n in enumerate(sizes)]
        ds = [{k: dev(a) for k, a in h.items()} for h in hs]
        adam_op.forward_multi_([d['updates'] for d in ds], [d['mu'] for d in ds],
                               [d['nu'] for d in ds], *HYPERS[0])
        for k, (h, d) in enumerate(zip(hs, ds)):
            eu, em, ev = O.forward_inplace(h['updates'], h['mu'], h['nu'], *HYPERS[0])
            assert_parity(host(d['updates']), eu, f'multi cap=7 updates[{k}]')
            assert_parity(host(d['nu']), ev, f'multi cap=7 nu[{k}]')
    finally:
        lib.toa_adam_set_max_grid(prev)


@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_one_pass_forward_and_backward_against_oracle_chain(tag):
    """forward_all / backward_all through the module and through the raw C ABI, against the
    oracle's separate functions composed with the additions autograd performs between them."""
    dtype = NP[tag]
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    np.seterr(all='ignore')  # the last case overflows on purpose
    for k, n in enumerate([1, 5, 257, 4099, 300_001, (1 << 22) + 37]):
        b1, b2, eps, er, c = HYPERS[k % 3]
        inp = rand(dtype, n, 900 + n)
        if n > (1 << 22):  # the staged whole-tile kernels, on operands of every exponent
            rng = np.random.default_rng(22)
            it = np.uint32 if tag == 'f32' else np.uint64
            top = int(np.array(np.inf, dtype).view(it))
            for key in inp:
                bits = rng.integers(0, top, size=n, dtype=it)
                if key != 'nu':
                    bits |= rng.integers(0, 2, size=n, dtype=it) << it(8 * bits.itemsize - 1)
                inp[key] = bits.view(dtype)
        g = {key: dev(a) for key, a in inp.items()}
        e_mu, e_nu = O.forward_mu(inp['updates'], inp['mu'], b1), O.forward_nu(inp['updates'],
                                                                              inp['nu'], b2)
        e_u = O.forward_updates(e_mu, e_nu, b1, b2, eps, er, c)
        new_mu, new_nu, new_u = adam_op.forward_all(g['updates'], g['mu'], g['nu'], b1, b2, eps,
                                                    er, c)
        assert_parity(host(new_mu), e_mu, f'n={n} forward_all new_mu')
        assert_parity(host(new_nu), e_nu, f'n={n} forward_all new_nu')
        assert_parity(host(new_u), e_u, f'n={n} forward_all new_updates')
        bm, bv = O.backward_updates(inp['dupdates'], e_u, e_mu, b1, b2, er, c)
        for has_m, has_v in [(False, False), (True, False), (False, True), (True, True)]:
            tot_m = inp['dmu'] + bm if has_m else bm
            tot_v = inp['dnu'] + bv if has_v else bv
            du1, dmu = O.backward_mu(tot_m, b1)
            du2, dnu = O.backward_nu(tot_v, inp['updates'], b2)
            got = adam_op.backward_all(g['dupdates'], g['dmu'] if has_m else None,
                                       g['dnu'] if has_v else None, new_u, new_mu, g['updates'],
                                       b1, b2, er, c)
            label = f'n={n} backward_all dm={has_m} dv={has_v}'
            assert_parity(host(got[0]), du1 + du2, f'{label} dupdates')
            assert_parity(host(got[1]), dmu, f'{label} dmu')
            assert_parity(host(got[2]), dnu, f'{label} dnu')
            outs = [torch.empty_like(new_mu) for _ in range(3)]
            rc = lib.toa_adam_backward_all(
                CODE[tag], g['dupdates'].data_ptr(), new_u.data_ptr(), new_mu.data_ptr(),
                g['updates'].data_ptr(), g['dmu'].data_ptr() if has_m else None,
                g['dnu'].data_ptr() if has_v else None, n, b1, b2, er, c, outs[0].data_ptr(),
                outs[1].data_ptr(), outs[2].data_ptr(), stream)
            assert rc == 0
            for a, b in zip(outs, got):
                bits = torch.int32 if tag == 'f32' else torch.int64  # NaNs included
                assert torch.equal(a.view(bits), b.view(bits)), \
                    f'{label}: C ABI and module disagree'


def test_empty_tensors():
    for dt in (torch.float32, torch.float64):
        e = torch.empty(0, device='cuda', dtype=dt)
        r = adam_op.forward_(e, e.clone(), e.clone(), 0.9, 0.999, 1e-8, 0.0, 1)
        assert r[0] is e
        assert adam_op.forward_mu(e, e, 0.9).shape == (0,)
        assert adam_op.forward_nu(e, e, 0.9).shape == (0,)
        assert adam_op.forward_updates(e, e, 0.9, 0.999, 1e-8, 0.0, 1).shape == (0,)
        assert [t.shape for t in adam_op.backward_mu(e, e, e, 0.9)] == [(0,), (0,)]
        assert [t.shape for t in adam_op.backward_nu(e, e, e, 0.9)] == [(0,), (0,)]
        assert [t.shape for t in adam_op.backward_updates(e, e, e, e, 0.9, 0.999, 0.0, 1)] == \
            [(0,), (0,)]
        e2 = torch.empty(3, 0, 5, device='cuda', dtype=dt)
        assert adam_op.forward_mu(e2, e2, 0.9).shape == (3, 0, 5)
    torch.cuda.synchronize()


def test_fully_aliased_scalar_like_the_availability_probe():
    """The reference's probe passes one 0-dim tensor as mu, nu and updates (n = 1)."""
    t = torch.tensor(1.0, device='cuda')
    r = adam_op.forward_(t, t, t, 0.9, 0.999, 1e-8, 0.0, 1)
    assert r[0] is t and torch.isfinite(t).item()
    # stores land in the order mu, nu, updates, so the survivor is the update
    one = np.ones(1, np.float32)
    ou, _, _ = O.forward_inplace(one.copy(), one.copy(), one.copy(), 0.9, 0.999, 1e-8, 0.0, 1)
    assert host(t).reshape(1)[0] == ou[0]


def test_count_accepts_int_and_zero_dim_tensors():
    inp = rand(np.float32, 1000, 1)
    want = O.forward_updates(inp['mu'], inp['nu'], 0.9, 0.999, 1e-8, 0.0, 6)
    for count in (6, np.int64(6), torch.tensor(6), torch.tensor(6, device='cuda'),
                  torch.zeros(1, dtype=torch.int64, device='cuda').squeeze_() + 6):
        got = adam_op.forward_updates(dev(inp['mu']), dev(inp['nu']), 0.9, 0.999, 1e-8, 0.0, count)
        assert_parity(host(got), want, f'count={type(count).__name__}')
    with pytest.raises(TypeError):
        adam_op.forward_updates(dev(inp['mu']), dev(inp['nu']), 0.9, 0.999, 1e-8, 0.0, 1.5)
    with pytest.raises(TypeError):
        adam_op.forward_updates(dev(inp['mu']), dev(inp['nu']), 0.9, 0.999, 1e-8, 0.0, -1)


def test_keyword_names_match_the_registered_ones():
    """adam_op.cpp:157-214, including backward_nu's fourth keyword being spelled b1."""
    inp = {k: dev(a) for k, a in rand(np.float64, 100, 2).items()}
    adam_op.forward_(updates=inp['updates'].clone(), mu=inp['mu'].clone(), nu=inp['nu'].clone(),
                     b1=0.9, b2=0.999, eps=1e-8, eps_root=0.0, count=1)
    adam_op.forward_mu(updates=inp['updates'], mu=inp['mu'], b1=0.9)
    adam_op.forward_nu(updates=inp['updates'], nu=inp['nu'], b2=0.999)
    adam_op.forward_updates(new_mu=inp['mu'], new_nu=inp['nu'], b1=0.9, b2=0.999, eps=1e-8,
                            eps_root=0.0, count=1)
    adam_op.backward_mu(dmu=inp['dmu'], updates=inp['updates'], mu=inp['mu'], b1=0.9)
    adam_op.backward_nu(dnu=inp['dnu'], updates=inp['updates'], nu=inp['nu'], b1=0.999)
    adam_op.backward_updates(dupdates=inp['dupdates'], updates=inp['updates'], new_mu=inp['mu'],
                             new_nu=inp['nu'], b1=0.9, b2=0.999, eps_root=0.0, count=1)
    torch.cuda.synchronize()


def test_return_conventions():
    """Lists for the array-returning ops, fresh tensors from the split ops, shapes from donors."""
    inp = {k: dev(a).reshape(4, 25) for k, a in rand(np.float32, 100, 2).items()}
    r = adam_op.forward_(inp['updates'].clone(), inp['mu'].clone(), inp['nu'].clone(), 0.9, 0.999,
                         1e-8, 0.0, 1)
    assert isinstance(r, list) and len(r) == 3
    m = adam_op.forward_mu(inp['updates'], inp['mu'], 0.9)
    assert m.shape == (4, 25) and m.data_ptr() != inp['mu'].data_ptr()
    r = adam_op.backward_mu(inp['dmu'], inp['updates'], inp['mu'], 0.9)
    assert isinstance(r, list) and len(r) == 2 and r[0].shape == (4, 25)
    r = adam_op.backward_updates(inp['dupdates'], inp['updates'], inp['mu'], inp['nu'], 0.9,
                                 0.999, 0.0, 1)
    assert isinstance(r, list) and len(r) == 2 and not r[0].requires_grad


def test_noncontiguous_grads_and_dense_layouts():
    """Incoming grads are made contiguous (adam_op.cpp:107,123,143); dense but permuted state
    (same strides everywhere) is processed in memory order."""
    dtype = np.float64
    base = rand(dtype, 6 * 50, 4)
    dmu_t = dev(base['dmu']).reshape(50, 6).t()  # shape (6, 50), non-contiguous
    upd = dev(base['updates']).reshape(6, 50)
    mu = dev(base['mu']).reshape(6, 50)
    du, dm = adam_op.backward_mu(dmu_t, upd, mu, 0.9)
    edu, edm = O.backward_mu(np.ascontiguousarray(base['dmu'].reshape(50, 6).T).ravel(), 0.9)
    assert_parity(host(du).ravel(), edu, 'dupdates')
    assert_parity(host(dm).ravel(), edm, 'dmu')
    # permuted-dense state: all three share strides
    u_p, m_p, v_p = (dev(base[k]).reshape(50, 6).t() for k in ('updates', 'mu', 'nu'))
    ou, om, ov = O.forward_inplace(base['updates'].copy(), base['mu'].copy(), base['nu'].copy(),
                                   *HYPERS[0])
    adam_op.forward_(u_p, m_p, v_p, *HYPERS[0])
    assert_parity(host(u_p.t()).ravel(), ou, 'permuted updates')
    assert_parity(host(m_p.t()).ravel(), om, 'permuted mu')
    # strided (not dense) state is refused rather than silently mis-indexed
    big = dev(rand(dtype, 200, 5)['mu'])
    with pytest.raises(RuntimeError):
        adam_op.forward_(big[::2], big[::2].clone(), big[::2].clone(), *HYPERS[0])


def test_error_paths_on_gpu_tensors():
    a = torch.ones(8, device='cuda')
    with pytest.raises(RuntimeError, match='not implemented for'):
        adam_op.forward_mu(a.int(), a.int(), 0.9)
    with pytest.raises(RuntimeError, match='unsupported dtype'):  # 16-bit: no weight decay
        adam_op.fused_step_(a.half(), a.half(), a.half(), a.half(), 0.9, 0.999, 1e-8, 0.0, 1, 1e-3,
                            weight_decay=0.01)
    with pytest.raises(RuntimeError, match='scalar type'):
        adam_op.forward_mu(a, a.double(), 0.9)
    with pytest.raises(RuntimeError, match='size mismatch'):
        adam_op.forward_mu(a, a[:4], 0.9)
    with pytest.raises(RuntimeError):
        adam_op.forward_mu(a, a.cpu(), 0.9)
    with pytest.raises(RuntimeError, match='Not implemented'):
        adam_op.forward_mu(a.cpu(), a, 0.9)
    lib = _lib.load()
    assert lib.toa_adam_forward_mu(7, a.data_ptr(), a.data_ptr(), 8, 0.9, a.data_ptr(), None) == -1
    assert lib.toa_adam_forward_mu(0, None, a.data_ptr(), 8, 0.9, a.data_ptr(), None) == -2
    torch.cuda.synchronize()


def test_runs_on_the_current_stream():
    """Work is enqueued on PyTorch's current stream: a side stream's result is ordered after
    that stream's earlier work without any extra synchronisation."""
    n = 1 << 22
    inp = rand(np.float32, n, 77)
    want = O.forward_mu(inp['updates'], inp['mu'], 0.9)
    side = torch.cuda.Stream()
    u = torch.empty(n, device='cuda')
    m = dev(inp['mu'])
    src = dev(inp['updates'])
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(20):  # keep the side stream busy, then write the real operand last
            u.copy_(src * 0)
        u.copy_(src)
        out = adam_op.forward_mu(u, m, 0.9)
    side.synchronize()
    assert_parity(host(out), want, 'side stream')


@pytest.mark.parametrize('tag', ['f32', 'f64'])
def test_fused_equals_split_chain_on_gpu(tag):
    """forward_ is bit-identical to forward_updates(forward_mu, forward_nu) (same expressions)."""
    n = (1 << 22) + 1
    g = {k: dev(a) for k, a in rand(NP[tag], n, 9).items()}
    b1, b2, eps, er, c = HYPERS[1]
    m1 = adam_op.forward_mu(g['updates'], g['mu'], b1)
    v1 = adam_op.forward_nu(g['updates'], g['nu'], b2)
    u1 = adam_op.forward_updates(m1, v1, b1, b2, eps, er, c)
    adam_op.forward_(g['updates'], g['mu'], g['nu'], b1, b2, eps, er, c)
    assert torch.equal(g['updates'], u1) and torch.equal(g['mu'], m1) and torch.equal(g['nu'], v1)


def test_repeated_steps_track_the_oracle():
    """Ten consecutive in-place steps with a growing count and fresh gradients."""
    n = 50_001
    rng = np.random.default_rng(123)
    mu = np.zeros(n, np.float32)
    nu = np.zeros(n, np.float32)
    gmu, gnu = dev(mu), dev(nu)
    for step in range(1, 11):
        g = rng.standard_normal(n).astype(np.float32)
        gg = dev(g)
        O.forward_inplace(g, mu, nu, 0.9, 0.999, 1e-8, 0.0, step)
        adam_op.forward_(gg, gmu, gnu, 0.9, 0.999, 1e-8, 0.0, step)
        assert_parity(host(gg), g, f'step {step} updates')
    assert_parity(host(gmu), mu, 'mu after 10 steps')
    assert_parity(host(gnu), nu, 'nu after 10 steps')


def test_every_residency_override_launches():
    """toa_adam_set_waves_per_cu reserves dynamic LDS to bound residency (2..32 workgroups per
    compute unit; up to 55 040 bytes).  Every level must launch and give the oracle's result."""
    lib = _lib.load()
    n = 70_001
    try:
        for waves in range(2, 33):
            a = rand(np.float32, n, 900 + waves)
            want = O.forward_inplace(a['updates'].copy(), a['mu'].copy(), a['nu'].copy(), 0.9,
                                     0.999, 1e-8, 0.0, 3)
            u, m, v = dev(a['updates']), dev(a['mu']), dev(a['nu'])
            lib.toa_adam_set_waves_per_cu(waves)
            print(f'forward_inplace f32 n={n} waves override {waves}', flush=True)
            rc = lib.toa_adam_forward_inplace(CODE['f32'], u.data_ptr(), m.data_ptr(),
                                              v.data_ptr(), n, 0.9, 0.999, 1e-8, 0.0, 3,
                                              torch.cuda.current_stream().cuda_stream)
            assert rc == 0, (waves, lib.toa_adam_error_string(rc))
            for got, exp, name in zip((u, m, v), want, ('updates', 'mu', 'nu')):
                assert_parity(host(got), exp, f'waves {waves} {name}')
        assert lib.toa_adam_set_waves_per_cu(1) == 32  # one per CU is not served: back to defaults
        assert lib.toa_adam_set_waves_per_cu(0) == 0
    finally:
        lib.toa_adam_set_waves_per_cu(0)
