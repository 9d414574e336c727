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
One file per dtype: adam_op_f32.npz, adam_op_f64.npz, adam_op_f16.npz, adam_op_bf16.npz; keys are
"<case>/<array>".  The reference CPU op serves at::Half and at::BFloat16 as well
(include/common.h:26-31); float16 arrays are stored as NumPy float16, bfloat16 arrays as uint16 bit
patterns (NumPy has no bfloat16).
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


class Fmt:
    """How one element type is held in NumPy and handed to torch."""

    def __init__(self, tag):
        self.tag = tag
        self.np_dtype = {'f32': np.float32, 'f64': np.float64, 'f16': np.float16,
                         'bf16': np.uint16}[tag]
        self.torch_dtype = {'f32': torch.float32, 'f64': torch.float64, 'f16': torch.float16,
                            'bf16': torch.bfloat16}[tag]

    def from_f64(self, a):
        """Round float64 values into the format (bfloat16 through float32, as torch does)."""
        if self.tag == 'bf16':
            with np.errstate(all='ignore'):
                return adam_oracle.bf16_bits(np.asarray(a, dtype=np.float64).astype(np.float32))
        with np.errstate(all='ignore'):
            return np.asarray(a, dtype=np.float64).astype(self.np_dtype)

    def to_torch(self, a):
        if self.tag == 'bf16':
            return torch.from_numpy(a.copy().view(np.int16)).view(torch.bfloat16)
        return torch.from_numpy(a.copy())

    def to_numpy(self, t):
        if self.tag == 'bf16':
            return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()
        return t.numpy().copy()

    def specials(self):
        if self.tag == 'bf16':  # bfloat16: 8 exponent bits like float32, 7 explicit mantissa bits
            sub, tiny, eps, big = 2.0 ** -133, 2.0 ** -126, 2.0 ** -7, (2 - 2.0 ** -7) * 2.0 ** 127
        else:
            fi = np.finfo(self.np_dtype)
            sub, tiny, eps, big = (float(fi.smallest_subnormal), float(fi.tiny), float(fi.eps),
                                   float(fi.max))
        small = {'f32': 1e-30, 'f64': 1e-300, 'f16': 1e-6, 'bf16': 1e-30}[self.tag]
        large = 1e10 if self.tag != 'f16' else 1e3
        return np.array([0.0, -0.0, sub, -sub, tiny / 2, tiny, -tiny, small, eps, 0.1, -0.1, 1.0,
                         -1.0, 3.0, 1024.0, large, -large, big / 4, big, -big, np.inf, -np.inf,
                         np.nan], dtype=np.float64)


def rand_inputs(fmt, n, seed):
    rng = np.random.default_rng(seed)
    return {
        'updates': fmt.from_f64(rng.standard_normal(n)),
        'mu': fmt.from_f64(0.1 * rng.standard_normal(n)),
        'nu': fmt.from_f64(np.abs(0.01 * rng.standard_normal(n))),
        'dmu': fmt.from_f64(rng.standard_normal(n)),
        'dnu': fmt.from_f64(rng.standard_normal(n)),
        'dupdates': fmt.from_f64(rng.standard_normal(n)),
    }


def edge_inputs(fmt):
    specials = fmt.specials()
    # every (updates, mu) pair of specials, nu cycling through the non-negative ones
    g, m = map(np.ravel, np.meshgrid(specials, specials, indexing='ij'))
    nonneg = specials[~(np.signbit(specials))]
    v = np.resize(nonneg, g.shape)
    rng = np.random.default_rng(7)
    # cancellation: b1*mu ~ -(1-b1)*g
    gc = rng.standard_normal(64)
    mc = -(1 - 0.9) * gc / 0.9
    vc = np.abs(rng.standard_normal(64))
    g = np.concatenate([g, gc])
    m = np.concatenate([m, mc])
    v = np.concatenate([v, vc])
    n = g.size
    return {
        'updates': fmt.from_f64(g), 'mu': fmt.from_f64(m), 'nu': fmt.from_f64(v),
        'dmu': fmt.from_f64(np.resize(specials, n)),
        'dnu': fmt.from_f64(np.resize(specials[::-1], n)),
        'dupdates': fmt.from_f64(np.concatenate([np.resize(specials[3:], n - 64),
                                                 rng.standard_normal(64)])),
    }


def run_reference(ref, fmt, inp, hyper):
    b1, b2, eps, eps_root, count = hyper
    t = {k: fmt.to_torch(v) for k, v in inp.items()}
    op = ref.adam_op
    out = {}
    new_mu = op.forward_mu(t['updates'], t['mu'], b1)
    new_nu = op.forward_nu(t['updates'], t['nu'], b2)
    new_updates = op.forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count)
    out['new_mu'], out['new_nu'], out['new_updates'] = (fmt.to_numpy(x) for x in
                                                        (new_mu, new_nu, new_updates))
    iu, im, iv = t['updates'].clone(), t['mu'].clone(), t['nu'].clone()
    r = op.forward_(iu, im, iv, b1, b2, eps, eps_root, count)
    assert r[0] is iu and r[1] is im and r[2] is iv
    out['inplace_updates'], out['inplace_mu'], out['inplace_nu'] = (fmt.to_numpy(x) for x in r)
    du, dm = op.backward_mu(t['dmu'], t['updates'], t['mu'], b1)
    out['bmu_dupdates'], out['bmu_dmu'] = fmt.to_numpy(du), fmt.to_numpy(dm)
    du, dn = op.backward_nu(t['dnu'], t['updates'], t['nu'], b2)
    out['bnu_dupdates'], out['bnu_dnu'] = fmt.to_numpy(du), fmt.to_numpy(dn)
    # backward_updates takes the forward output and the new moments
    dm, dn = op.backward_updates(t['dupdates'], new_updates, new_mu, new_nu, b1, b2, eps_root,
                                 count)
    out['bup_dnew_mu'], out['bup_dnew_nu'] = fmt.to_numpy(dm), fmt.to_numpy(dn)
    return out


def main():
    ref = adam_oracle.load_reference()
    if ref is None:
        raise SystemExit('oracle/_ref/_C*.so not built: run `make -C oracle ref` first')
    for tag in ('f32', 'f64', 'f16', 'bf16'):
        fmt = Fmt(tag)
        cases = {}
        for k, hyper in enumerate(HYPER):
            if tag in ('f16', 'bf16') and hyper[2] == 1e-8:
                # 1e-8 is zero in half precision; give the 16-bit formats an eps they can hold
                hyper = (hyper[0], hyper[1], 1e-3, hyper[3] and 1e-4, hyper[4])
            cases[f'rand_{k}'] = (rand_inputs(fmt, 2051 if k < 2 else 259, 100 + k), hyper)
        for k, hyper in enumerate(HYPER[1:4]):
            cases[f'edge_{k}'] = (edge_inputs(fmt), hyper)
        blob = {}
        for name, (inp, hyper) in cases.items():
            out = run_reference(ref, fmt, inp, hyper)
            blob[f'{name}/hyper'] = np.array(hyper, dtype=np.float64)
            for key, arr in itertools.chain(inp.items(), out.items()):
                blob[f'{name}/{key}'] = arr
        path = os.path.join(HERE, f'adam_op_{tag}.npz')
        np.savez_compressed(path, **blob)
        print(path, os.path.getsize(path), 'bytes,', len(cases), 'cases')


if __name__ == '__main__':
    main()
