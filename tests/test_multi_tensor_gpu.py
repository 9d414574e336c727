"""Multi-tensor entry points: one launch over a list of tensors must give, bit for bit, what the
per-tensor entry points (and the CPU oracle) give for each tensor on its own."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import _lib
from torchopt_amd._C import adam_op

import bench

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


def make_lists(dtype, sizes, seed):
    rng = np.random.default_rng(seed)
    out = {k: [] for k in ('updates', 'mu', 'nu', 'dmu', 'dnu', 'dupdates')}
    for n in sizes:
        out['updates'].append(rng.standard_normal(n).astype(dtype))
        out['mu'].append((0.1 * rng.standard_normal(n)).astype(dtype))
        out['nu'].append(np.abs(0.01 * rng.standard_normal(n)).astype(dtype))
        for k in ('dmu', 'dnu', 'dupdates'):
            out[k].append(rng.standard_normal(n).astype(dtype))
    return out


def to_dev(lists):
    return {k: [dev(a) for a in v] for k, v in lists.items()}


def check_lists(got, want, what):
    assert len(got) == len(want)
    for k, (g, w) in enumerate(zip(got, want)):
        assert_bit_equal(host(g).ravel(), w.ravel(), f'{what}[{k}] n={w.size}')


def run_all_multi(dtype, sizes, seed, eps_root, counts):
    """All seven ops through the multi-tensor entry points against the oracle per tensor."""
    h = make_lists(dtype, sizes, seed)
    g = to_dev(h)
    num = len(sizes)
    cl = counts if isinstance(counts, (list, tuple)) else [counts] * num

    new_mu = adam_op.forward_mu_multi(g['updates'], g['mu'], B1)
    new_nu = adam_op.forward_nu_multi(g['updates'], g['nu'], B2)
    e_mu = [O.forward_mu(u, m, B1) for u, m in zip(h['updates'], h['mu'])]
    e_nu = [O.forward_nu(u, v, B2) for u, v in zip(h['updates'], h['nu'])]
    check_lists(new_mu, e_mu, 'forward_mu_multi')
    check_lists(new_nu, e_nu, 'forward_nu_multi')

    new_u = adam_op.forward_updates_multi(new_mu, new_nu, B1, B2, EPS, eps_root, counts)
    e_u = [O.forward_updates(m, v, B1, B2, EPS, eps_root, c) for m, v, c in zip(e_mu, e_nu, cl)]
    check_lists(new_u, e_u, 'forward_updates_multi')

    du, dm = adam_op.backward_mu_multi(g['dmu'], g['updates'], g['mu'], B1)
    e = [O.backward_mu(d, B1) for d in h['dmu']]
    check_lists(du, [x[0] for x in e], 'backward_mu_multi dupdates')
    check_lists(dm, [x[1] for x in e], 'backward_mu_multi dmu')

    du, dn = adam_op.backward_nu_multi(g['dnu'], g['updates'], g['nu'], B2)
    e = [O.backward_nu(d, u, B2) for d, u in zip(h['dnu'], h['updates'])]
    check_lists(du, [x[0] for x in e], 'backward_nu_multi dupdates')
    check_lists(dn, [x[1] for x in e], 'backward_nu_multi dnu')

    dm, dn = adam_op.backward_updates_multi(g['dupdates'], new_u, new_mu, new_nu, B1, B2,
                                            eps_root, counts)
    e = [O.backward_updates(d, u, m, B1, B2, eps_root, c)
         for d, u, m, c in zip(h['dupdates'], e_u, e_mu, cl)]
    check_lists(dm, [x[0] for x in e], 'backward_updates_multi dnew_mu')
    check_lists(dn, [x[1] for x in e], 'backward_updates_multi dnew_nu')

    # in place, last: it overwrites the inputs
    r = adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, eps_root, counts)
    assert r[0] is g['updates'] and r[1] is g['mu'] and r[2] is g['nu']
    check_lists(g['updates'], e_u, 'forward_multi_ updates')
    check_lists(g['mu'], e_mu, 'forward_multi_ mu')
    check_lists(g['nu'], e_nu, 'forward_multi_ nu')


def test_maml_pytree_config1():
    """Config 1: the MAML conv-net parameter list, float32, eps_root = 1e-8, count = 5."""
    sizes = [bench.numel(s) for s in bench.maml_shapes()]
    assert len(sizes) == 10 and sum(sizes) == 32645
    run_all_multi(np.float32, sizes, 1001, 1e-8, 5)


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
def test_many_ragged_tensors_cross_table_capacity(dtype):
    """260 tensors: more than one kernel-argument table holds for any op; lengths include 0, 1,
    non-multiples of the vector width, exact tiles and a few large ones."""
    rng = np.random.default_rng(5)
    sizes = [0, 1, 2, 3, 4, 5, 255, 256, 257, 511, 512, 513, 1024, 4096, 100_003, 0, 7]
    sizes += [int(x) for x in rng.integers(0, 3000, size=260 - len(sizes))]
    sizes[100] = 300_001
    sizes[200] = 0
    run_all_multi(dtype, sizes, 77, 1e-8, 3)


def test_shared_output_allocation_is_bounded():
    """Small leaves' outputs share one allocation per call, up to 64 MiB: 200 leaves of 0.75 MiB
    (150 MiB per output list) get results equal to the per-leaf op, outputs that overlap neither
    one another nor the inputs, and no storage larger than the bound."""
    n, num = 196_608, 200  # 0.75 MiB of float32 per leaf
    gen = torch.Generator(device='cuda').manual_seed(11)
    g = [torch.randn(n, device='cuda', generator=gen) for _ in range(num)]
    mu = [0.1 * torch.randn(n, device='cuda', generator=gen) for _ in range(num)]
    nu = [0.01 * torch.rand(n, device='cuda', generator=gen) for _ in range(num)]
    new_mu, new_nu, new_u = adam_op.forward_all_multi(g, mu, nu, B1, B2, EPS, 1e-8, 3)
    outs = new_mu + new_nu + new_u
    assert max(t.untyped_storage().nbytes() for t in outs) <= 64 << 20
    assert min(t.untyped_storage().nbytes() for t in outs) == 4 * n  # the rest: one each
    assert all(t.data_ptr() % 256 == 0 for t in outs)
    spans = sorted((t.data_ptr(), t.data_ptr() + 4 * n) for t in outs + g + mu + nu)
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    for k in (0, 27, 28, 29, 199):  # both sides of where the shared allocation ends
        m1, v1, u1 = adam_op.forward_all(g[k], mu[k], nu[k], B1, B2, EPS, 1e-8, 3)
        assert torch.equal(new_mu[k], m1) and torch.equal(new_nu[k], v1)
        assert torch.equal(new_u[k], u1)


def test_per_tensor_counts():
    """The API lets every leaf carry its own step count; tensors are grouped per count."""
    sizes = [1000, 17, 5000, 256, 3, 70_000, 999, 1]
    counts = [1, 5, 1, 1000, 5, 2, 1000, 7]
    run_all_multi(np.float32, sizes, 9, 0.0, counts)
    # zero-dim device tensors as counts, as the transformation passes them
    tcounts = [torch.tensor(c, device='cuda') for c in counts]
    h = make_lists(np.float64, sizes, 10)
    g = to_dev(h)
    adam_op.forward_multi_(g['updates'], g['mu'], g['nu'], B1, B2, EPS, 0.0, tcounts)
    for k, c in enumerate(counts):
        u, m, v = O.forward_inplace(h['updates'][k], h['mu'][k], h['nu'][k], B1, B2, EPS, 0.0, c)
        assert_bit_equal(host(g['updates'][k]), u, f'tensor {k}')
        assert_bit_equal(host(g['nu'][k]), v, f'tensor {k}')


def test_multi_with_misaligned_members():
    """Some list members are views that start off a 16-byte boundary."""
    sizes = [1000, 4099, 64, 30_001]
    h = make_lists(np.float32, [n + 3 for n in sizes], 21)
    g = to_dev(h)
    offs = [0, 1, 3, 2]
    gv = {k: [t[o:o + n] for t, o, n in zip(g[k], offs, sizes)] for k in ('updates', 'mu', 'nu')}
    hv = {k: [a[o:o + n].copy() for a, o, n in zip(h[k], offs, sizes)]
          for k in ('updates', 'mu', 'nu')}
    adam_op.forward_multi_(gv['updates'], gv['mu'], gv['nu'], B1, B2, EPS, 0.0, 4)
    for k, n in enumerate(sizes):
        u, m, v = O.forward_inplace(hv['updates'][k], hv['mu'][k], hv['nu'][k], B1, B2, EPS, 0.0, 4)
        assert_bit_equal(host(gv['updates'][k]), u, f'updates[{k}]')
        assert_bit_equal(host(gv['mu'][k]), m, f'mu[{k}]')
        assert_bit_equal(host(gv['nu'][k]), v, f'nu[{k}]')
        # guards either side of the view
        full = host(g['mu'][k])
        assert_bit_equal(full[:offs[k]], h['mu'][k][:offs[k]], 'head guard')
        assert_bit_equal(full[offs[k] + n:], h['mu'][k][offs[k] + n:], 'tail guard')


def test_empty_lists_and_all_empty_members():
    assert adam_op.forward_multi_([], [], [], B1, B2, EPS, 0.0, 1) == ([], [], [])
    assert adam_op.forward_mu_multi([], [], B1) == []
    e = [torch.empty(0, device='cuda'), torch.empty(0, device='cuda')]
    adam_op.forward_multi_(e, [t.clone() for t in e], [t.clone() for t in e], B1, B2, EPS, 0.0, 1)
    assert [t.shape for t in adam_op.forward_nu_multi(e, e, B2)] == [(0,), (0,)]


def test_multi_argument_checks():
    a = [torch.ones(4, device='cuda'), torch.ones(5, device='cuda')]
    with pytest.raises(RuntimeError, match='length'):
        adam_op.forward_multi_(a, a[:1], a, B1, B2, EPS, 0.0, 1)
    with pytest.raises(RuntimeError, match='size mismatch'):
        adam_op.forward_multi_(a, [a[1], a[0]], a, B1, B2, EPS, 0.0, 1)
    with pytest.raises(RuntimeError, match='scalar type'):
        adam_op.forward_multi_(a, [t.double() for t in a], a, B1, B2, EPS, 0.0, 1)
    with pytest.raises(RuntimeError, match='Not implemented'):
        adam_op.forward_multi_([t.cpu() for t in a], a, a, B1, B2, EPS, 0.0, 1)
    with pytest.raises(RuntimeError, match='counts'):
        adam_op.forward_multi_(a, [t.clone() for t in a], [t.clone() for t in a], B1, B2, EPS,
                               0.0, [1])


def test_c_abi_multi_direct():
    """The raw entry point on host arrays of device pointers, with and without a counts array."""
    lib = _lib.load()
    sizes = [300, 0, 4097, 12]
    h = make_lists(np.float32, sizes, 31)
    g = to_dev(h)
    num = len(sizes)
    arr = lambda ts: (ctypes.c_void_p * num)(*[t.data_ptr() for t in ts])  # noqa: E731
    ns = (ctypes.c_size_t * num)(*sizes)
    counts = (ctypes.c_uint64 * num)(2, 9, 2, 6)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.toa_adam_forward_inplace_multi(_lib.TOA_F32, num, arr(g['updates']), arr(g['mu']),
                                            arr(g['nu']), ns, B1, B2, EPS, 1e-8, counts, 0, stream)
    assert rc == 0
    for k, c in enumerate([2, 9, 2, 6]):
        u, m, v = O.forward_inplace(h['updates'][k], h['mu'][k], h['nu'][k], B1, B2, EPS, 1e-8, c)
        assert_bit_equal(host(g['updates'][k]), u, f'tensor {k}')
        assert_bit_equal(host(g['mu'][k]), m, f'tensor {k}')
    # argument errors come back as codes, before anything is launched
    assert lib.toa_adam_forward_inplace_multi(9, num, arr(g['updates']), arr(g['mu']),
                                              arr(g['nu']), ns, B1, B2, EPS, 0.0, None, 1,
                                              stream) == -1
    bad = (ctypes.c_void_p * num)(g['mu'][0].data_ptr(), None, None, g['mu'][3].data_ptr())
    assert lib.toa_adam_forward_inplace_multi(_lib.TOA_F32, num, arr(g['updates']), bad,
                                              arr(g['nu']), ns, B1, B2, EPS, 0.0, None, 1,
                                              stream) == -2
    assert lib.toa_adam_forward_inplace_multi(_lib.TOA_F32, num, arr(g['updates']), None,
                                              arr(g['nu']), ns, B1, B2, EPS, 0.0, None, 1,
                                              stream) == -2
    torch.cuda.synchronize()
