"""The five benchmark configurations at their real sizes, checked against the CPU oracle on the
same seeded inputs, plus the size-independent properties of the path.

Inputs follow the benchmark's distributions (updates ~ N(0,1), mu ~ 0.1 N(0,1),
nu ~ |0.01 N(0,1)|) and seeds (1000 * config + tensor index); they are drawn once, on the GPU
for the large configurations, copied to the host, and the same arrays feed the oracle and the
kernels.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import AdamOp
from torchopt_amd._C import adam_op

import bench

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def host(t):
    return t.detach().cpu().numpy()


def gpu_equal(t: torch.Tensor, want: np.ndarray, what: str):
    """Bit comparison done on the GPU (the arrays are up to 1 GiB); falls back to the detailed
    host comparison only to report a mismatch."""
    w = torch.from_numpy(want).cuda()
    it = torch.int32 if t.dtype == torch.float32 else torch.int64
    same = (t.view(it) == w.view(it)) | (torch.isnan(t) & torch.isnan(w))
    if not bool(same.all()):
        assert_bit_equal(host(t), want, what)


def draw(n, dtype, seed):
    g = torch.Generator(device='cuda')
    g.manual_seed(seed)
    u = torch.randn(n, device='cuda', dtype=dtype, generator=g)
    m = torch.randn(n, device='cuda', dtype=dtype, generator=g).mul_(0.1)
    v = torch.randn(n, device='cuda', dtype=dtype, generator=g).mul_(0.01).abs_()
    return u, m, v


def test_config0_flat_1m_fp32():
    n, count = 1 << 20, 10
    u, m, v = draw(n, torch.float32, 0)
    hu, hm, hv = host(u), host(m), host(v)
    O.forward_inplace(hu, hm, hv, B1, B2, EPS, 0.0, count)
    adam_op.forward_(u, m, v, B1, B2, EPS, 0.0, count)
    gpu_equal(u, hu, 'updates'), gpu_equal(m, hm, 'mu'), gpu_equal(v, hv, 'nu')


def test_config1_differentiable_path_through_autograd():
    """MAML-style pytree, float32: forward mu/nu/updates via the autograd Functions, then the
    backward chain with seeded output cotangents; every tensor against the oracle."""
    shapes = bench.maml_shapes()
    eps_root, count = 1e-8, 5
    op = AdamOp(B1, B2, EPS, eps_root=eps_root, inplace=False)
    cnt = torch.zeros(1, dtype=torch.int64, device='cuda').squeeze_() + count
    for k, shape in enumerate(shapes):
        rng = np.random.default_rng(1000 + k)
        n = bench.numel(shape)
        hg = rng.standard_normal(n).astype(np.float32)
        hm = (0.1 * rng.standard_normal(n)).astype(np.float32)
        hv = np.abs(0.01 * rng.standard_normal(n)).astype(np.float32)
        d_u, d_m, d_v = (rng.standard_normal(n).astype(np.float32) for _ in range(3))

        def leaf(a):
            return torch.from_numpy(a).cuda().reshape(shape).requires_grad_(True)

        g, m, v = leaf(hg), leaf(hm), leaf(hv)
        new_mu, new_nu, new_u = op(m, v, g, cnt)
        assert new_u.shape == tuple(shape) and new_u.requires_grad
        e_mu, e_nu = O.forward_mu(hg, hm, B1), O.forward_nu(hg, hv, B2)
        e_u = O.forward_updates(e_mu, e_nu, B1, B2, EPS, eps_root, count)
        assert_bit_equal(host(new_mu).ravel(), e_mu, f'leaf {k} new_mu')
        assert_bit_equal(host(new_nu).ravel(), e_nu, f'leaf {k} new_nu')
        assert_bit_equal(host(new_u).ravel(), e_u, f'leaf {k} new_updates')

        def ct(a):
            return torch.from_numpy(a).cuda().reshape(shape)

        torch.autograd.backward([new_u, new_mu, new_nu], [ct(d_u), ct(d_m), ct(d_v)])
        # the chain the engine runs: updates -> (mu, nu) -> (g, m, v); sums are commutative
        bm, bv = O.backward_updates(d_u, e_u, e_mu, B1, B2, eps_root, count)
        tot_m, tot_v = d_m + bm, d_v + bv
        gu1, gm = O.backward_mu(tot_m, B1)
        gu2, gv = O.backward_nu(tot_v, hg, B2)
        assert_bit_equal(host(m.grad).ravel(), gm, f'leaf {k} d mu')
        assert_bit_equal(host(v.grad).ravel(), gv, f'leaf {k} d nu')
        assert_bit_equal(host(g.grad).ravel(), gu1 + gu2, f'leaf {k} d updates')


def test_config2_flat_256m_fp32_against_oracle():
    """The headline workload at full size: 3 x 1 GiB in place, count = 1000."""
    n, count = 1 << 28, 1000
    u, m, v = draw(n, torch.float32, 2000)
    hu, hm, hv = host(u), host(m), host(v)
    O.forward_inplace(hu, hm, hv, B1, B2, EPS, 0.0, count)
    adam_op.forward_(u, m, v, B1, B2, EPS, 0.0, count)
    gpu_equal(u, hu, 'updates'), gpu_equal(m, hm, 'mu'), gpu_equal(v, hv, 'nu')
    del hu, hm, hv
    # a second step on the evolved state (what the benchmark times) stays finite
    adam_op.forward_(u, m, v, B1, B2, EPS, 0.0, count)
    assert bool(torch.isfinite(u).all()) and bool(torch.isfinite(v).all())


def test_config2_size_fused_equals_split_chain():
    """At full size, without the oracle: the fused step is bit-identical to the split chain."""
    n, count = 1 << 28, 1000
    u, m, v = draw(n, torch.float32, 2001)
    m1 = adam_op.forward_mu(u, m, B1)
    v1 = adam_op.forward_nu(u, v, B2)
    u1 = adam_op.forward_updates(m1, v1, B1, B2, EPS, 0.0, count)
    adam_op.forward_(u, m, v, B1, B2, EPS, 0.0, count)
    assert torch.equal(u, u1) and torch.equal(m, m1) and torch.equal(v, v1)


def test_config3_fp64_forward_and_full_backward():
    n, count, eps_root = 1 << 26, 3, 1e-8
    u, m, v = draw(n, torch.float64, 3000)
    g = torch.Generator(device='cuda')
    g.manual_seed(3001)
    d_m, d_v, d_u = (torch.randn(n, device='cuda', dtype=torch.float64, generator=g)
                     for _ in range(3))
    hu, hm, hv = host(u), host(m), host(v)
    hg = hu.copy()
    O.forward_inplace(hu, hm, hv, B1, B2, EPS, eps_root, count)
    grads = u.clone()
    adam_op.forward_(u, m, v, B1, B2, EPS, eps_root, count)
    gpu_equal(u, hu, 'updates'), gpu_equal(m, hm, 'mu'), gpu_equal(v, hv, 'nu')
    # backward inputs: updates = forward output, new_mu/new_nu = forward state
    a, b = adam_op.backward_updates(d_u, u, m, v, B1, B2, eps_root, count)
    ea, eb = O.backward_updates(host(d_u), hu, hm, B1, B2, eps_root, count)
    gpu_equal(a, ea, 'dnew_mu'), gpu_equal(b, eb, 'dnew_nu')
    del a, b, ea, eb
    a, b = adam_op.backward_nu(d_v, grads, v, B2)
    ea, eb = O.backward_nu(host(d_v), hg, B2)
    gpu_equal(a, ea, 'backward_nu dupdates'), gpu_equal(b, eb, 'backward_nu dnu')
    del a, b, ea, eb
    a, b = adam_op.backward_mu(d_m, grads, m, B1)
    ea, eb = O.backward_mu(host(d_m), B1)
    gpu_equal(a, ea, 'backward_mu dupdates'), gpu_equal(b, eb, 'backward_mu dmu')


def test_config4_gpt2_medium_multi_tensor():
    """290 tensors, 354 821 120 float32 elements, one multi-tensor call; against the oracle per
    tensor, and against the per-tensor entry point."""
    shapes = bench.gpt2_medium_shapes()
    sizes = [bench.numel(s) for s in shapes]
    assert len(sizes) == 290 and sum(sizes) == 354_821_120
    us, ms, vs = [], [], []
    for k, (shape, n) in enumerate(zip(shapes, sizes)):
        u, m, v = draw(n, torch.float32, 4000 + k)
        us.append(u.reshape(shape)), ms.append(m.reshape(shape)), vs.append(v.reshape(shape))
    hus, hms, hvs = [host(t).ravel() for t in us], [host(t).ravel() for t in ms], \
        [host(t).ravel() for t in vs]
    # per-tensor route on clones of a few members, for the bitwise cross-check
    probe = [0, 1, 9, 288, 289]
    singles = {}
    for k in probe:
        cu, cm, cv = us[k].clone(), ms[k].clone(), vs[k].clone()
        adam_op.forward_(cu, cm, cv, B1, B2, EPS, 0.0, 1)
        singles[k] = (cu, cm, cv)
    adam_op.forward_multi_(us, ms, vs, B1, B2, EPS, 0.0, 1)
    for k in probe:
        assert torch.equal(us[k], singles[k][0]) and torch.equal(ms[k], singles[k][1]) and \
            torch.equal(vs[k], singles[k][2])
    for k in range(len(sizes)):
        O.forward_inplace(hus[k], hms[k], hvs[k], B1, B2, EPS, 0.0, 1)
        gpu_equal(us[k].reshape(-1), hus[k], f'updates[{k}]')
        gpu_equal(ms[k].reshape(-1), hms[k], f'mu[{k}]')
        gpu_equal(vs[k].reshape(-1), hvs[k], f'nu[{k}]')
