"""float16 and bfloat16 tensors through the GPU op against the CPU oracle and the golden vectors
of the reference CPU op (which serves at::Half / at::BFloat16 with per-operation rounding,
/root/reference/include/common.h:26-31).  Bit for bit."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal, hyper_of, load_golden
from oracle import adam_oracle as O
from torchopt_amd import AdamOp
from torchopt_amd._C import adam_op

pytestmark = pytest.mark.gpu

TORCH = {'f16': torch.float16, 'bf16': torch.bfloat16}


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()


def dev(a, tag):
    """NumPy float16 array, or uint16 bfloat16 bit patterns, to a GPU tensor of that type."""
    a = np.ascontiguousarray(a)
    if tag == 'bf16':
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def host(t, tag):
    if tag == 'bf16':
        return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.detach().cpu().numpy()


def draw(tag, n, seed):
    rng = np.random.default_rng(seed)

    def fmt(x):
        return O.bf16_bits(x.astype(np.float32)) if tag == 'bf16' else x.astype(np.float16)

    return {'updates': fmt(rng.standard_normal(n)), 'mu': fmt(0.1 * rng.standard_normal(n)),
            'nu': fmt(np.abs(0.01 * rng.standard_normal(n))), 'dmu': fmt(rng.standard_normal(n)),
            'dnu': fmt(rng.standard_normal(n)), 'dupdates': fmt(rng.standard_normal(n))}


def check_all_seven(tag, inp, hyper, label, exp=None):
    b1, b2, eps, er, c = hyper
    u, m, v = inp['updates'], inp['mu'], inp['nu']
    if exp is None:
        ou, om, ov = O.forward_inplace(u.copy(), m.copy(), v.copy(), b1, b2, eps, er, c)
        exp = {'new_mu': O.forward_mu(u, m, b1), 'new_nu': O.forward_nu(u, v, b2),
               'inplace_updates': ou, 'inplace_mu': om, 'inplace_nu': ov}
        exp['new_updates'] = O.forward_updates(exp['new_mu'], exp['new_nu'], b1, b2, eps, er, c)
        exp['bmu_dupdates'], exp['bmu_dmu'] = O.backward_mu(inp['dmu'], b1)
        exp['bnu_dupdates'], exp['bnu_dnu'] = O.backward_nu(inp['dnu'], u, b2)
        exp['bup_dnew_mu'], exp['bup_dnew_nu'] = O.backward_updates(
            inp['dupdates'], exp['new_updates'], exp['new_mu'], b1, b2, er, c)
    g = {k: dev(a, tag) for k, a in inp.items()}

    def same(t, key):
        assert_bit_equal(host(t, tag), exp[key], f'{label} {key}')

    same(adam_op.forward_mu(g['updates'], g['mu'], b1), 'new_mu')
    same(adam_op.forward_nu(g['updates'], g['nu'], b2), 'new_nu')
    emu, env = dev(exp['new_mu'], tag), dev(exp['new_nu'], tag)
    same(adam_op.forward_updates(emu, env, b1, b2, eps, er, c), 'new_updates')
    iu, im, iv = g['updates'].clone(), g['mu'].clone(), g['nu'].clone()
    adam_op.forward_(iu, im, iv, b1, b2, eps, er, c)
    same(iu, 'inplace_updates'), same(im, 'inplace_mu'), same(iv, 'inplace_nu')
    du, dm = adam_op.backward_mu(g['dmu'], g['updates'], g['mu'], b1)
    same(du, 'bmu_dupdates'), same(dm, 'bmu_dmu')
    du, dn = adam_op.backward_nu(g['dnu'], g['updates'], g['nu'], b2)
    same(du, 'bnu_dupdates'), same(dn, 'bnu_dnu')
    dm, dn = adam_op.backward_updates(g['dupdates'], dev(exp['new_updates'], tag), emu, env, b1,
                                      b2, er, c)
    same(dm, 'bup_dnew_mu'), same(dn, 'bup_dnew_nu')


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_golden_vectors(tag):
    for name, case in sorted(load_golden(tag).items()):
        inp = {k: case[k] for k in ('updates', 'mu', 'nu', 'dmu', 'dnu', 'dupdates')}
        check_all_seven(tag, inp, hyper_of(case), f'{tag}/{name}', exp=case)


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_sizes_against_oracle(tag):
    """Eight elements per 128-bit access, 512 per tile: sizes around those boundaries."""
    hypers = [(0.9, 0.999, 1e-3, 0.0, 10), (0.9, 0.999, 1e-3, 1e-4, 5), (0.8, 0.95, 1e-2, 1e-3, 77)]
    for k, n in enumerate([1, 7, 8, 9, 511, 512, 513, 4095, 4097, 65537, (1 << 20) + 5,
                           (1 << 23) + 777]):  # the last: whole-tile kernel plus a ragged tail
        check_all_seven(tag, draw(tag, n, 700 + n), hypers[k % 3], f'{tag}/n={n}')


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
@pytest.mark.parametrize('operand', ['updates', 'mu', 'nu', 'dmu', 'dnu', 'dupdates'])
def test_every_bit_pattern_of_one_operand(tag, operand):
    """All 65 536 values of the type (every denormal, infinity and NaN included) in one operand,
    the others drawn at random: every conversion and rounding case of that operand's paths."""
    n = 1 << 16
    inp = draw(tag, n, 900 + len(operand))
    every = np.arange(n, dtype=np.uint16)
    inp[operand] = every if tag == 'bf16' else every.view(np.float16)
    with np.errstate(all='ignore'):
        check_all_seven(tag, inp, (0.9, 0.999, 1e-3, 1e-4, 3), f'{tag}/all {operand}')


@pytest.mark.parametrize('hyper', [(0.9, 0.999, 1e-8, 0.0, 1), (0.9, 0.999, 1e-3, 1e-4, 7),
                                   (0.8, 0.95, 1e-2, 1e-3, 1000), (0.0, 0.5, 0.0, 0.0, 3)],
                         ids=['default', 'eps_root', 'late', 'degenerate'])
@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_quick_route_equals_exact_route_for_every_pair(tag, hyper):
    """The 16-bit update takes a quick route (1-ulp root and reciprocal) wherever the quotient
    is provably far from a rounding boundary and the exact chain elsewhere.  All 2^32 pairs of
    (new_mu, new_nu) bit patterns: the 16-byte aligned call (quick route with exact repeats)
    against the same data one element off alignment (element-wise path, always the exact chain),
    and a slice of it against the CPU oracle."""
    b1, b2, eps, er, count = hyper
    dt = TORCH[tag]
    every = torch.arange(65536, dtype=torch.int32, device='cuda').to(torch.int16)
    rows = 4096  # new_nu patterns per chunk
    n = rows * 65536
    mu = every.repeat(rows).view(dt)
    off_mu = torch.empty(n + 8, dtype=dt, device='cuda')[1:n + 1]
    off_nu = torch.empty(n + 8, dtype=dt, device='cuda')[1:n + 1]
    off_mu.copy_(mu)
    assert mu.data_ptr() % 16 == 0 and off_mu.data_ptr() % 16 == 2
    for chunk in range(65536 // rows):
        nu = every[chunk * rows:(chunk + 1) * rows].repeat_interleave(65536).view(dt)
        off_nu.copy_(nu)
        quick = adam_op.forward_updates(mu, nu, b1, b2, eps, er, count)
        exact = adam_op.forward_updates(off_mu, off_nu, b1, b2, eps, er, count)
        # NaN signs and payloads are not part of the contract: every NaN counts as one value
        nan = torch.tensor(0x7fff, dtype=torch.int16, device='cuda')
        qb = torch.where(quick.isnan(), nan, quick.view(torch.int16))
        eb = torch.where(exact.isnan(), nan, exact.view(torch.int16))
        if not torch.equal(qb, eb):
            bad = (qb != eb).nonzero()[0].item()
            raise AssertionError(
                f'chunk {chunk}: new_mu {mu.view(torch.int16)[bad].item() & 0xffff:#06x} new_nu '
                f'{nu.view(torch.int16)[bad].item() & 0xffff:#06x}: quick '
                f'{quick.view(torch.int16)[bad].item() & 0xffff:#06x} exact '
                f'{exact.view(torch.int16)[bad].item() & 0xffff:#06x}')
        if chunk in (3, 4):  # positive normal new_nu of everyday magnitude: tie to the oracle
            k = 1 << 24
            with np.errstate(all='ignore'):
                want = O.forward_updates(host(mu[:k], tag), host(nu[:k], tag), b1, b2, eps, er,
                                         count)
            assert_bit_equal(host(quick[:k], tag), want, f'chunk {chunk} against the oracle')
        del nu, quick, exact, qb, eb
    torch.cuda.empty_cache()


def _as_one_nan(t):
    nan = torch.tensor(0x7fff, dtype=torch.int16, device=t.device)
    return torch.where(t.isnan(), nan, t.view(torch.int16))


def _first_moment_in_float(mu, g, b1):
    """b1*mu + (1-b1)*g the way c10::Half / c10::BFloat16 compute it -- every operation in
    float, each result rounded to the 16-bit type -- with PyTorch's own kernels, one operation
    and one conversion per kernel, so no instruction can merge an operation with its rounding."""
    dt = mu.dtype
    one_minus = float(torch.tensor(1.0, dtype=dt) - torch.tensor(b1, dtype=dt))
    a = (mu.float() * b1).to(dt)
    b = (g.float() * one_minus).to(dt)
    return (a.float() + b.float()).to(dt)


def _first_moment(op, mu, g, b1):
    """new_mu from the element-wise kernel (forward_mu, whose float16 operations the compiler
    may merge with their roundings) or from the kernels that compute in pairs (forward_ in
    place: packed half instructions for float16, one rounding instruction per pair for
    bfloat16)."""
    if op == 'forward_mu':
        return adam_op.forward_mu(g, mu, b1)
    new_mu = mu.clone()
    adam_op.forward_(g.clone(), new_mu, torch.ones_like(mu), b1, 0.999, 1e-3, 0.0, 1)
    return new_mu


@pytest.mark.parametrize('op', ['forward_mu', 'forward_'])
@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_sums_equal_float_sums_rounded_for_every_pair(tag, op):
    """float16 pairs are added with v_pk_add_f16, and single values by whatever the compiler
    makes of widen-add-convert.  That both are the float addition rounded to float16 (what the
    reference computes) for EVERY pair of operands: the first moment with b1 = 0.5 is
    0.5*mu + 0.5*g, whose two halvings are exact for all but the smallest values, over all
    2^32 (mu, g) pairs, against the same expression evaluated in float by separate PyTorch
    kernels.  bfloat16, which adds in float and rounds with one instruction, likewise."""
    dt = TORCH[tag]
    every = torch.arange(65536, dtype=torch.int32, device='cuda').to(torch.int16)
    rows = 1024
    mu = every.repeat(rows).view(dt)
    for chunk in range(65536 // rows):
        g = every[chunk * rows:(chunk + 1) * rows].repeat_interleave(65536).view(dt)
        got = _as_one_nan(_first_moment(op, mu, g, 0.5))
        want = _as_one_nan(_first_moment_in_float(mu, g, 0.5))
        if not torch.equal(got, want):
            bad = (got != want).nonzero()[0].item()
            raise AssertionError(
                f'mu {mu.view(torch.int16)[bad].item() & 0xffff:#06x} g '
                f'{g.view(torch.int16)[bad].item() & 0xffff:#06x}: got '
                f'{got[bad].item() & 0xffff:#06x} want {want[bad].item() & 0xffff:#06x}')
        del g, got, want
    torch.cuda.empty_cache()


@pytest.mark.parametrize('op', ['forward_mu', 'forward_'])
@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_products_equal_float_products_rounded_for_every_pair(tag, op):
    """... and v_pk_mul_f16 (or the compiler's widen-multiply-convert) the float multiplication
    rounded to 16 bits: b1*mu for values of b1 in [0, 1) (every 5th bit pattern, all of them
    around the powers of two, every denormal) times every mu, with a zero gradient."""
    dt = TORCH[tag]
    every = torch.arange(65536, dtype=torch.int32, device='cuda').to(torch.int16)
    mu = every.view(dt)
    g = torch.zeros(65536, dtype=dt, device='cuda')
    one, binade = (0x3c00, 0x0400) if tag == 'f16' else (0x3f80, 0x0080)
    patterns = sorted(p for p in set(range(0, one, 5))
                      | {p + d for p in range(binade, one, binade) for d in range(-3, 4)}
                      | set(range(0, binade + 16))  # the denormal values of b1, all of them
                      if p < one)
    for pattern in patterns:
        b1 = float(torch.tensor(pattern, dtype=torch.int16).view(dt))
        got = _as_one_nan(_first_moment(op, mu, g, b1))
        want = _as_one_nan(_first_moment_in_float(mu, g, b1))
        if not torch.equal(got, want):
            bad = (got != want).nonzero()[0].item()
            raise AssertionError(f'b1 {pattern:#06x} mu {bad:#06x}: got '
                                 f'{got[bad].item() & 0xffff:#06x} want '
                                 f'{want[bad].item() & 0xffff:#06x}')


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_misaligned_views(tag):
    n = 30_001
    inp = draw(tag, n + 8, 5)
    for off in (1, 3, 4, 7):
        cut = {k: a[off:off + n].copy() for k, a in inp.items()}
        e = O.forward_inplace(cut['updates'], cut['mu'], cut['nu'], 0.9, 0.999, 1e-3, 0.0, 4)
        full = {k: dev(inp[k], tag) for k in ('updates', 'mu', 'nu')}
        views = [full[k][off:off + n] for k in ('updates', 'mu', 'nu')]
        adam_op.forward_(*views, 0.9, 0.999, 1e-3, 0.0, 4)
        for t, want, k in zip(views, e, ('updates', 'mu', 'nu')):
            assert_bit_equal(host(t, tag), want, f'offset {off} {k}')
            h = host(full[k], tag)
            assert_bit_equal(h[:off], inp[k][:off], 'head guard')
            assert_bit_equal(h[off + n:], inp[k][off + n:], 'tail guard')


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
def test_multi_tensor_and_autograd(tag):
    sizes = [864, 9216, 32, 4000, 5, 0, 70_001]
    hs = [draw(tag, n, 40 + k) for k, n in enumerate(sizes)]
    us, ms, vs = ([dev(h[key], tag) for h in hs] for key in ('updates', 'mu', 'nu'))
    adam_op.forward_multi_(us, ms, vs, 0.9, 0.999, 1e-3, 1e-4, 3)
    for k, h in enumerate(hs):
        eu, em, ev = O.forward_inplace(h['updates'].copy(), h['mu'].copy(), h['nu'].copy(), 0.9,
                                       0.999, 1e-3, 1e-4, 3)
        assert_bit_equal(host(us[k], tag), eu, f'multi updates[{k}]')
        assert_bit_equal(host(vs[k], tag), ev, f'multi nu[{k}]')
    # differentiable chain on one leaf
    h = hs[1]
    g, m, v = (dev(h[key], tag).requires_grad_(True) for key in ('updates', 'mu', 'nu'))
    new_mu, new_nu, new_u = AdamOp(0.9, 0.999, 1e-3, eps_root=1e-4, inplace=False)(m, v, g, 2)
    new_u.backward(dev(h['dupdates'], tag))
    e_mu, e_nu = O.forward_mu(h['updates'], h['mu'], 0.9), O.forward_nu(h['updates'], h['nu'], 0.999)
    e_u = O.forward_updates(e_mu, e_nu, 0.9, 0.999, 1e-3, 1e-4, 2)
    assert_bit_equal(host(new_u, tag), e_u, 'forward chain')
    bm, bv = O.backward_updates(h['dupdates'], e_u, e_mu, 0.9, 0.999, 1e-4, 2)
    _, gm = O.backward_mu(bm, 0.9)
    _, gv = O.backward_nu(bv, h['updates'], 0.999)
    assert_bit_equal(host(m.grad, tag), gm, 'd mu')
    assert_bit_equal(host(v.grad, tag), gv, 'd nu')


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
@pytest.mark.parametrize('operand', ['updates', 'mu', 'nu', 'dmu', 'dnu', 'dupdates'])
def test_one_pass_ops_equal_the_seven_for_every_bit_pattern(tag, operand):
    """forward_all / backward_all (one pass per direction) against the seven ops they fuse, with
    every value of the type in one operand: the element-wise kernels (65 536 elements) and the
    whole-tile ones (128 times that).  The seven are pinned to the oracle above; here GPU
    results are compared with GPU results, NaNs as one value."""
    b1, b2, eps, er, c = 0.9, 0.999, 1e-3, 1e-4, 3
    for repeat in (1, 128):
        n = 65536 * repeat
        inp = draw(tag, n, 1200 + len(operand))
        g = {k: dev(a, tag) for k, a in inp.items()}
        every = torch.arange(n, dtype=torch.int32, device='cuda').to(torch.int16)
        g[operand] = every.view(TORCH[tag])
        new_mu = adam_op.forward_mu(g['updates'], g['mu'], b1)
        new_nu = adam_op.forward_nu(g['updates'], g['nu'], b2)
        new_u = adam_op.forward_updates(new_mu, new_nu, b1, b2, eps, er, c)
        got = adam_op.forward_all(g['updates'], g['mu'], g['nu'], b1, b2, eps, er, c)
        for a, b, what in zip(got, (new_mu, new_nu, new_u), ('new_mu', 'new_nu', 'new_updates')):
            assert torch.equal(_as_one_nan(a), _as_one_nan(b)), f'{tag} x{repeat} {what}'
        bm, bv = adam_op.backward_updates(g['dupdates'], new_u, new_mu, new_nu, b1, b2, er, c)
        for has_m, has_v in [(False, False), (True, False), (False, True), (True, True)]:
            tot_m = g['dmu'] + bm if has_m else bm
            tot_v = g['dnu'] + bv if has_v else bv
            du1, dmu = adam_op.backward_mu(tot_m, g['updates'], g['mu'], b1)
            du2, dnu = adam_op.backward_nu(tot_v, g['updates'], g['nu'], b2)
            got = adam_op.backward_all(g['dupdates'], g['dmu'] if has_m else None,
                                       g['dnu'] if has_v else None, new_u, new_mu, g['updates'],
                                       b1, b2, er, c)
            for a, b, what in zip(got, (du1 + du2, dmu, dnu), ('dupdates', 'dmu', 'dnu')):
                assert torch.equal(_as_one_nan(a), _as_one_nan(b)), \
                    f'{tag} x{repeat} dm={has_m} dv={has_v} {what}'


@pytest.mark.parametrize('tag', ['f16', 'bf16'])
@pytest.mark.parametrize('eps', [-1e-3, -0.25, -4.0, float('nan')])
def test_negative_eps_takes_the_exact_chain(tag, eps):
    """The quick route's error bound assumes root + eps does not cancel.  The raw ops accept a
    negative (or NaN) eps, so those must go through the exact chain: the aligned call (quick
    route where allowed) against the same data one element off alignment (always exact) and
    against the CPU oracle, over every new_mu pattern and a spread of new_nu values."""
    dt = TORCH[tag]
    every = torch.arange(65536, dtype=torch.int32, device='cuda').to(torch.int16)
    nus = torch.tensor([0.0, 1e-6, 2.5e-4, 1e-3, 0.0625, 0.25, 1.0, 4.0, 15.9, 16.0, 16.1, 300.0],
                       device='cuda').to(dt)
    rows = nus.numel()
    n = rows * 65536
    mu = every.repeat(rows).view(dt)
    nu = nus.repeat_interleave(65536)
    off_mu = torch.empty(n + 8, dtype=dt, device='cuda')[1:n + 1]
    off_nu = torch.empty(n + 8, dtype=dt, device='cuda')[1:n + 1]
    off_mu.copy_(mu)
    off_nu.copy_(nu)
    quick = adam_op.forward_updates(mu, nu, 0.9, 0.999, eps, 0.0, 3)
    exact = adam_op.forward_updates(off_mu, off_nu, 0.9, 0.999, eps, 0.0, 3)
    with np.errstate(all='ignore'):
        want = O.forward_updates(host(mu, tag), host(nu, tag), 0.9, 0.999, eps, 0.0, 3)
    assert_bit_equal(host(exact, tag), want, f'{tag} eps={eps}: element-wise path')
    assert_bit_equal(host(quick, tag), want, f'{tag} eps={eps}: aligned path')


