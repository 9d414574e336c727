"""Seeded random sweep: random lengths, alignments, hyper-parameters, element types and ops
through the GPU path against the oracle, plus one tensor longer than 2^32 elements to cover
64-bit indexing.  Everything bit for bit."""

from __future__ import annotations

import os

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd._C import adam_op

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def to_fmt(x, tag):
    if tag == 'bf16':
        return O.bf16_bits(np.asarray(x, dtype=np.float32))
    return np.asarray(x).astype({'f32': np.float32, 'f64': np.float64, 'f16': np.float16}[tag])


def dev(a, tag):
    a = np.ascontiguousarray(a)
    if tag == 'bf16':
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def host(t, tag):
    if tag == 'bf16':
        return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.detach().cpu().numpy()


# TOA_RANDOM_SEEDS=N widens the sweep for a soak run
@pytest.mark.parametrize('seed', range(int(os.environ.get('TOA_RANDOM_SEEDS', '6'))))
def test_random_cases(seed):
    rng = np.random.default_rng(1234 + seed)
    for case in range(40):
        tag = ['f32', 'f64', 'f16', 'bf16'][int(rng.integers(4))]
        n = int(rng.choice([rng.integers(0, 40), rng.integers(0, 3000), rng.integers(0, 200_000)]))
        off = int(rng.integers(0, 9))
        b1, b2 = float(rng.uniform(0, 0.999)), float(rng.uniform(0, 0.9999))
        eps = float(10.0 ** rng.uniform(-8, -2)) if tag in ('f32', 'f64') else float(
            10.0 ** rng.uniform(-4, -2))
        er = float(rng.choice([0.0, 10.0 ** rng.uniform(-6, -3)]))
        count = int(rng.choice([0, 1, 2, 17, 1000, 10 ** 6, 2 ** 40]))
        scale = float(10.0 ** rng.uniform(-3, 2))
        raw = {k: to_fmt(scale * rng.standard_normal(n + off + 3), tag)
               for k in ('updates', 'mu', 'dmu', 'dnu', 'dupdates')}
        raw['nu'] = to_fmt(np.abs(scale * scale * rng.standard_normal(n + off + 3)), tag)
        cut = {k: a[off:off + n].copy() for k, a in raw.items()}
        g = {k: dev(a, tag)[off:off + n] for k, a in raw.items()}
        label = f'seed {seed} case {case}: {tag} n={n} off={off} count={count}'
        with np.errstate(all='ignore'):
            e_mu = O.forward_mu(cut['updates'], cut['mu'], b1)
            e_nu = O.forward_nu(cut['updates'], cut['nu'], b2)
            e_u = O.forward_updates(e_mu, e_nu, b1, b2, eps, er, count)
            bm, bv = O.backward_updates(cut['dupdates'], e_u, e_mu, b1, b2, er, count)
        op = int(rng.integers(4))
        if op == 0:  # the three split forwards and the fused in-place step
            assert_bit_equal(host(adam_op.forward_mu(g['updates'], g['mu'], b1), tag), e_mu, label)
            assert_bit_equal(host(adam_op.forward_nu(g['updates'], g['nu'], b2), tag), e_nu, label)
            adam_op.forward_(g['updates'], g['mu'], g['nu'], b1, b2, eps, er, count)
            assert_bit_equal(host(g['updates'], tag), e_u, label)
            assert_bit_equal(host(g['nu'], tag), e_nu, label)
        elif op == 1:  # one-pass forward
            got = adam_op.forward_all(g['updates'], g['mu'], g['nu'], b1, b2, eps, er, count)
            for t, want in zip(got, (e_mu, e_nu, e_u)):
                assert_bit_equal(host(t, tag), want, label)
        elif op == 2:  # the three split backwards
            got = adam_op.backward_updates(g['dupdates'], dev(e_u, tag), dev(e_mu, tag),
                                           dev(e_nu, tag), b1, b2, er, count)
            assert_bit_equal(host(got[0], tag), bm, label)
            assert_bit_equal(host(got[1], tag), bv, label)
            got = adam_op.backward_mu(g['dmu'], g['updates'], g['mu'], b1)
            want = O.backward_mu(cut['dmu'], b1)
            assert_bit_equal(host(got[0], tag), want[0], label)
            got = adam_op.backward_nu(g['dnu'], g['updates'], g['nu'], b2)
            want = O.backward_nu(cut['dnu'], cut['updates'], b2)
            assert_bit_equal(host(got[0], tag), want[0], label)
            assert_bit_equal(host(got[1], tag), want[1], label)
        else:  # one-pass backward without outside gradients
            got = adam_op.backward_all(g['dupdates'], None, None, dev(e_u, tag), dev(e_mu, tag),
                                       g['updates'], b1, b2, er, count)
            with np.errstate(all='ignore'):
                du1, dmu = O.backward_mu(bm, b1)
                du2, dnu = O.backward_nu(bv, cut['updates'], b2)
            assert_bit_equal(host(got[1], tag), dmu, label)
            assert_bit_equal(host(got[2], tag), dnu, label)
        # nothing outside the views was touched
        for k in ('updates', 'mu', 'nu'):
            full = host(g[k]._base if g[k]._base is not None else g[k], tag)
            assert_bit_equal(full[:off], raw[k][:off], label + ' head guard')
            assert_bit_equal(full[off + n:], raw[k][off + n:], label + ' tail guard')


_TOP = {'f32': (np.uint32, 0x7f800000), 'f64': (np.uint64, 0x7ff0000000000000),
        'f16': (np.uint16, 0x7c00), 'bf16': (np.uint16, 0x7f80)}


def draw(rng, tag, n, kind, nonneg=False):
    """'bits': uniform over the finite bit patterns of the type (every exponent equally likely),
    now and then with an infinity or a NaN; 'sparse': half the elements zero; else normal."""
    if kind == 'bits':
        it, top = _TOP[tag]
        b = rng.integers(0, top + (3 if rng.random() < 0.3 else 0), size=n,
                         dtype=np.uint64).astype(it)
        if not nonneg:
            sign = rng.integers(0, 2, size=n, dtype=np.uint64) << np.uint64(8 * b.itemsize - 1)
            b |= sign.astype(it)
        return b if tag == 'bf16' else b.view({'f32': np.float32, 'f64': np.float64,
                                               'f16': np.float16}[tag])
    x = 10.0 ** rng.uniform(-4, 2) * rng.standard_normal(n)
    if kind == 'sparse':
        x[rng.random(n) < 0.5] = 0.0
    return to_fmt(np.abs(x) if nonneg else x, tag)


@pytest.mark.parametrize('seed', range(int(os.environ.get('TOA_RANDOM_SEEDS', '4'))))
def test_random_cases_of_the_optimizer_step_and_of_lists(seed):
    """The fused optimizer step (single tensors and lists, every type, with `maximize`, with and
    without the written-back update, weight decay for float32 / float64) and the in-place step
    over ragged lists with per-tensor step numbers, on normal, half-zero and bit-pattern-uniform
    operands, learning rates that are round decimal numbers among them."""
    rng = np.random.default_rng(977 + seed)
    for case in range(25):
        tag = ['f32', 'f64', 'f16', 'bf16'][int(rng.integers(4))]
        kind = str(rng.choice(['normal', 'bits', 'sparse']))
        b1 = float(rng.choice([0.0, 0.5, 0.9, rng.uniform(0, 0.999)]))
        b2 = float(rng.choice([0.0, 0.99, 0.999, rng.uniform(0, 0.9999)]))
        eps = float(rng.choice([0.0, 1e-8, 1e-3, 10.0 ** rng.uniform(-8, -1)]))
        er = float(rng.choice([0.0, 1e-8, 1e-4]))
        count = int(rng.choice([1, 2, 10, 1000, 10 ** 6]))
        lr = float(rng.choice([0.05, 0.1, 0.01, 1e-3, 3e-4, 1e-5, 10.0 ** rng.uniform(-6, 0)]))
        mx, wu = bool(rng.integers(2)), bool(rng.integers(2))
        wd, dec = 0.0, False
        if tag in ('f32', 'f64') and rng.random() < 0.5:
            wd, dec = 0.05, bool(rng.integers(2))
        which = int(rng.integers(3))
        label = (f'seed {seed} case {case}: {tag} {kind} b1={b1} b2={b2} eps={eps} er={er} '
                 f'count={count} lr={lr} maximize={mx} write_updates={wu} wd={wd} '
                 f'decoupled={dec} which={which}')
        print(label, flush=True)
        with np.errstate(all='ignore'):
            if which == 0:  # one tensor through the fused step, at a random element offset
                n = int(rng.choice([rng.integers(1, 600), rng.integers(1, 70_000),
                                    rng.integers(1, 1_500_000)]))
                off = int(rng.integers(0, 8))
                raw = [draw(rng, tag, n + off, kind, nonneg=(j == 3)) for j in range(4)]
                h = [a[off:].copy() for a in raw]
                d = [dev(a, tag)[off:] for a in raw]
                adam_op.fused_step_(d[0], d[1], d[2], d[3], b1, b2, eps, er, count, lr,
                                    maximize=mx, write_updates=wu, weight_decay=wd,
                                    decoupled=dec)
                O.fused_step(h[0], h[1], h[2], h[3], b1, b2, eps, er, count, lr, mx, wu, wd, dec)
                for j, what in enumerate(('params', 'updates', 'mu', 'nu')):
                    assert_bit_equal(host(d[j], tag), h[j], f'{label} {what}')
                continue
            num = int(rng.integers(1, 200))
            sizes = [int(x) for x in rng.choice([0, 1, 7, 255, 256, 513, 4096, 70_001], size=num)]
            if rng.random() < 0.3:
                sizes[int(rng.integers(num))] = int(rng.integers(1, 1_500_000))
            counts = [int(rng.choice([1, 2, 1000])) for _ in sizes] if rng.random() < 0.5 else count
            cl = counts if isinstance(counts, list) else [counts] * num
            hs = [[draw(rng, tag, m, kind, nonneg=(j == 3)) for j in range(4)] for m in sizes]
            ds = [[dev(a, tag) for a in h] for h in hs]
            if which == 1:  # the fused step over a ragged list
                adam_op.fused_step_multi_([d[0] for d in ds], [d[1] for d in ds],
                                          [d[2] for d in ds], [d[3] for d in ds], b1, b2, eps, er,
                                          counts, lr, maximize=mx, write_updates=wu,
                                          weight_decay=wd, decoupled=dec)
                for k, (h, d) in enumerate(zip(hs, ds)):
                    if sizes[k]:
                        O.fused_step(h[0], h[1], h[2], h[3], b1, b2, eps, er, cl[k], lr, mx, wu,
                                     wd, dec)
                        for j in range(4):
                            assert_bit_equal(host(d[j], tag), h[j], f'{label} tensor {k}/{j}')
            else:  # the in-place step over a ragged list
                adam_op.forward_multi_([d[1] for d in ds], [d[2] for d in ds],
                                       [d[3] for d in ds], b1, b2, eps, er, counts)
                for k, (h, d) in enumerate(zip(hs, ds)):
                    if sizes[k]:
                        want = O.forward_inplace(h[1].copy(), h[2].copy(), h[3].copy(), b1, b2,
                                                 eps, er, cl[k])
                        for j in range(3):
                            assert_bit_equal(host(d[j + 1], tag), want[j], f'{label} {k}/{j}')


def test_tensor_longer_than_2_to_32_elements():
    """2^32 + 777 float16 elements per array (8 GiB each): element indices and byte offsets pass
    32 bits inside one launch.  Windows at the start, across the 2^32 boundary and at the ragged
    end are checked against the oracle; the rest through the fused == split identity."""
    n = (1 << 32) + 777
    free, _ = torch.cuda.mem_get_info()
    if free < 6 * n * 2 + (4 << 30):
        pytest.skip('not enough free device memory for six 8 GiB arrays')
    g = torch.Generator(device='cuda').manual_seed(99)
    u = torch.empty(n, device='cuda', dtype=torch.float16).normal_(generator=g)
    m = torch.empty(n, device='cuda', dtype=torch.float16).normal_(0, 0.1, generator=g)
    v = torch.empty(n, device='cuda', dtype=torch.float16).normal_(0, 0.01, generator=g).abs_()
    b1, b2, eps, er, count = 0.9, 0.999, 1e-3, 1e-4, 12
    windows = [(0, 1 << 20), ((1 << 32) - (1 << 19), (1 << 32) + 777), (n - 4099, n)]
    saved = [[t[a:b].cpu().numpy() for t in (u, m, v)] for a, b in windows]
    m1 = adam_op.forward_mu(u, m, b1)
    v1 = adam_op.forward_nu(u, v, b2)
    u1 = adam_op.forward_updates(m1, v1, b1, b2, eps, er, count)
    adam_op.forward_(u, m, v, b1, b2, eps, er, count)
    assert torch.equal(u, u1) and torch.equal(m, m1) and torch.equal(v, v1)
    for (a, b), (hu, hm, hv) in zip(windows, saved):
        eu, em, ev = O.forward_inplace(hu, hm, hv, b1, b2, eps, er, count)
        assert_bit_equal(u[a:b].cpu().numpy(), eu, f'updates[{a}:{b}]')
        assert_bit_equal(m[a:b].cpu().numpy(), em, f'mu[{a}:{b}]')
        assert_bit_equal(v[a:b].cpu().numpy(), ev, f'nu[{a}:{b}]')
