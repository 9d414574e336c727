"""Write the golden vectors under tests/golden/ from the reference's own compiled CPU op.

Runs only where /root/reference exists: `make -C oracle ref` compiles the reference's
src/extension.cpp, src/adam_op/adam_op.cpp and src/adam_op/adam_op_impl_cpu.cpp where they
lie into oracle/_ref/_C*.so, and this script calls that module's seven functions on CPU
tensors.  Inputs AND expected outputs are stored (plain .npz arrays, no pickles), so the
fixtures are self-contained data.

    python tests/golden/make_golden.py

Cases
  rand_<k>   seeded inputs with the benchmark distributions (updates ~ N(0,1),
             mu ~ 0.1 N(0,1), nu ~ |0.01 N(0,1)|) for hyper-parameter set k; n = 2051 for the
             first two sets (> 2000, so the reference's OpenMP branch runs with two threads;
             not a multiple of 4) and n = 259 for the rest;
  edge_<k>   a grid of special values: +-0, denormals, the smallest/largest normals, +-inf,
             NaN, powers of two, and values that cancel in b1*mu + (1-b1)*g.
One file per dtype: adam_op_f32.npz, adam_op_f64.npz; keys are "<case>/<array>".
"""

from __future__ import annotations

import itertools
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import adam_oracle  # noqa: E402

HYPER = [
    # b1, b2, eps, eps_root, count
    (0.9, 0.999, 1e-8, 0.0, 1),
    (0.9, 0.999, 1e-8, 0.0, 10),
    (0.9, 0.999, 1e-8, 1e-8, 5),
    (0.9, 0.999, 1e-8, 1e-8, 3),
    (0.9, 0.999, 1e-8, 0.0, 1000),
    (0.5, 0.75, 1e-3, 1e-4, 2),
    (0.0, 0.0, 0.0, 0.0, 7),
    (0.95, 0.9999, 1e-6, 1e-12, 123456),
]


def rand_inputs(dtype, n, seed):
    rng = np.random.default_rng(seed)
    return {
        'updates': rng.standard_normal(n).astype(dtype),
        'mu': (0.1 * rng.standard_normal(n)).astype(dtype),
        'nu': np.abs(0.01 * rng.standard_normal(n)).astype(dtype),
        'dmu': rng.standard_normal(n).astype(dtype),
        'dnu': rng.standard_normal(n).astype(dtype),
        'dupdates': rng.standard_normal(n).astype(dtype),
    }


def edge_inputs(dtype):
    fi = np.finfo(dtype)
    specials = np.array(
        [0.0, -0.0, fi.smallest_subnormal, -fi.smallest_subnormal, fi.tiny / 2, fi.tiny,
         -fi.tiny, 1e-30 if dtype == np.float32 else 1e-300, fi.eps, 0.1, -0.1, 1.0, -1.0, 3.0,
         1024.0, 1e10, -1e10, fi.max / 4, fi.max, -fi.max, np.inf, -np.inf, np.nan],
        dtype=dtype)
    # every (updates, mu) pair of specials, nu cycling through the non-negative ones
    g, m = map(np.ravel, np.meshgrid(specials, specials, indexing='ij'))
    nonneg = specials[~(np.signbit(specials))]
    v = np.resize(nonneg, g.shape)
    rng = np.random.default_rng(7)
    # cancellation: b1*mu ~ -(1-b1)*g
    gc = rng.standard_normal(64).astype(dtype)
    mc = (-(dtype(1) - dtype(0.9)) * gc / dtype(0.9)).astype(dtype)
    vc = np.abs(rng.standard_normal(64)).astype(dtype)
    g = np.concatenate([g, gc])
    m = np.concatenate([m, mc])
    v = np.concatenate([v, vc])
    n = g.size
    return {
        'updates': g, 'mu': m, 'nu': v,
        'dmu': np.resize(specials, n), 'dnu': np.resize(specials[::-1], n),
        'dupdates': np.concatenate([np.resize(specials[3:], n - 64),
                                    rng.standard_normal(64).astype(dtype)]),
    }


def run_reference(ref, inp, hyper):
    b1, b2, eps, eps_root, count = hyper
    t = {k: torch.from_numpy(v.copy()) for k, v in inp.items()}
    op = ref.adam_op
    out = {}
    out['new_mu'] = op.forward_mu(t['updates'], t['mu'], b1).numpy()
    out['new_nu'] = op.forward_nu(t['updates'], t['nu'], b2).numpy()
    out['new_updates'] = op.forward_updates(
        torch.from_numpy(out['new_mu']), torch.from_numpy(out['new_nu']),
        b1, b2, eps, eps_root, count).numpy()
    iu, im, iv = t['updates'].clone(), t['mu'].clone(), t['nu'].clone()
    r = op.forward_(iu, im, iv, b1, b2, eps, eps_root, count)
    assert r[0] is iu and r[1] is im and r[2] is iv
    out['inplace_updates'], out['inplace_mu'], out['inplace_nu'] = (x.numpy() for x in r)
    du, dm = op.backward_mu(t['dmu'], t['updates'], t['mu'], b1)
    out['bmu_dupdates'], out['bmu_dmu'] = du.numpy(), dm.numpy()
    du, dn = op.backward_nu(t['dnu'], t['updates'], t['nu'], b2)
    out['bnu_dupdates'], out['bnu_dnu'] = du.numpy(), dn.numpy()
    # backward_updates takes the forward output and the new moments
    dm, dn = op.backward_updates(
        t['dupdates'], torch.from_numpy(out['new_updates']), torch.from_numpy(out['new_mu']),
        torch.from_numpy(out['new_nu']), b1, b2, eps_root, count)
    out['bup_dnew_mu'], out['bup_dnew_nu'] = dm.numpy(), dn.numpy()
    return out


def main():
    ref = adam_oracle.load_reference()
    if ref is None:
        raise SystemExit('oracle/_ref/_C*.so not built: run `make -C oracle ref` first')
    for dtype, tag in ((np.float32, 'f32'), (np.float64, 'f64')):
        cases = {}
        for k, hyper in enumerate(HYPER):
            cases[f'rand_{k}'] = (rand_inputs(dtype, 2051 if k < 2 else 259, 100 + k), hyper)
        for k, hyper in enumerate(HYPER[1:4]):
            cases[f'edge_{k}'] = (edge_inputs(dtype), hyper)
        blob = {}
        for name, (inp, hyper) in cases.items():
            with np.errstate(all='ignore'):
                out = run_reference(ref, inp, hyper)
            blob[f'{name}/hyper'] = np.array(hyper, dtype=np.float64)
            for key, arr in itertools.chain(inp.items(), out.items()):
                blob[f'{name}/{key}'] = arr
        path = os.path.join(HERE, f'adam_op_{tag}.npz')
        np.savez_compressed(path, **blob)
        print(path, os.path.getsize(path), 'bytes,', len(cases), 'cases')


if __name__ == '__main__':
    main()
