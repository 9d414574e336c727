"""Shared test plumbing.

Markers
  gpu   needs a real MI355X; everything unmarked runs on CPU only.
  perf  speed gates (tests/test_perf_gates.py): need an MI355X too, but are kept out of `-m gpu`
        so that the GPU suite is a pure correctness signal; skipped where there is no GPU.

Only the test suite, the smoke check and the benchmark's CPU-baseline leg may import
`oracle`; the product package `torchopt_amd` never does.
"""

from __future__ import annotations

import os
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

GOLDEN_DIR = os.path.join(REPO, 'tests', 'golden')


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: test needs a real AMD GPU (MI355X)')
    config.addinivalue_line('markers', 'perf: speed gate (needs an MI355X); never selected by -m gpu, '
                                       'skipped where there is no GPU')


def load_golden(tag: str):
    """{case: {array name: ndarray}} from tests/golden/adam_op_<tag>.npz."""
    cases = {}
    with np.load(os.path.join(GOLDEN_DIR, f'adam_op_{tag}.npz'), allow_pickle=False) as z:
        for key in z.files:
            case, name = key.split('/')
            cases.setdefault(case, {})[name] = z[key]
    return cases


def hyper_of(case):
    b1, b2, eps, eps_root, count = case['hyper'].tolist()
    return b1, b2, eps, eps_root, int(count)


def bits(a: np.ndarray) -> np.ndarray:
    """Bit patterns, with every NaN collapsed to one pattern (NaN payloads and signs are not
    part of the contract: x86 and the GPU propagate different ones).  uint16 arrays are
    bfloat16 bit patterns."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:  # bfloat16: NaN = exponent all ones, mantissa non-zero
        u = a.copy()
        u[(a & 0x7fff) > 0x7f80] = 0xffff
        return u
    u = a.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize]).copy()
    u[np.isnan(a)] = np.iinfo(u.dtype).max
    return u


def assert_bit_equal(got: np.ndarray, want: np.ndarray, what: str = ''):
    assert got.dtype == want.dtype and got.shape == want.shape, what
    gb, wb = bits(got), bits(want)
    if not np.array_equal(gb, wb):
        bad = np.flatnonzero(gb != wb)
        i = bad[0]
        raise AssertionError(
            f'{what}: {bad.size}/{got.size} elements differ; first at {i}: '
            f'got {got.ravel()[i]!r} ({gb.ravel()[i]:#x}) want {want.ravel()[i]!r} '
            f'({wb.ravel()[i]:#x})')


def ulp_distance(got: np.ndarray, want: np.ndarray) -> np.ndarray:
    """Distance in units in the last place between same-dtype arrays (NaN == NaN -> 0,
    NaN vs number -> huge)."""
    it = np.int32 if got.dtype == np.float32 else np.int64
    big = np.iinfo(it).max

    def ordered(x):
        i = np.ascontiguousarray(x).view(it).astype(np.int64 if it is np.int32 else it)
        # map sign-magnitude to a monotone integer line
        return np.where(i < 0, np.iinfo(it).min - i, i)

    d = np.abs(ordered(got).astype(np.float64) - ordered(want).astype(np.float64))
    gn, wn = np.isnan(got), np.isnan(want)
    d[gn & wn] = 0
    d[gn ^ wn] = big
    return d


@pytest.fixture(scope='session')
def golden_f32():
    return load_golden('f32')


@pytest.fixture(scope='session')
def golden_f64():
    return load_golden('f64')
