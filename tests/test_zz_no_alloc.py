"""toa_adam_forward_inplace_multi_noalloc -- the entry point that allocates nothing: its plan
records live in a device array built into the library -- against toa_adam_forward_inplace_multi
on the same inputs, bit for bit, through the C ABI: two calls in a row, the second with a smaller
list (the array keeps the first call's records beyond the second's), then a list beyond the
stated limit, which must be refused before anything is launched."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import _lib

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8
TOA_ELIMIT = -4


def make(sizes, seed):
    rng = np.random.default_rng(seed)
    return [[rng.standard_normal(n).astype(np.float32),
             (0.1 * rng.standard_normal(n)).astype(np.float32),
             np.abs(0.01 * rng.standard_normal(n)).astype(np.float32)] for n in sizes]


def call(fn, leaves, sizes, counts, count_all):
    """One call of `fn` (either entry point) on fresh device copies; returns them as NumPy."""
    lib = _lib.load()
    dev = [[torch.from_numpy(a).cuda() for a in leaf] for leaf in leaves]
    num = len(sizes)
    col = lambda j: (ctypes.c_void_p * num)(*[leaf[j].data_ptr() for leaf in dev])
    cts = None if counts is None else (ctypes.c_uint64 * num)(*counts)
    rc = fn(_lib.TOA_F32, num, col(0), col(1), col(2), (ctypes.c_size_t * num)(*sizes), B1, B2, EPS,
            1e-8, cts, count_all, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.toa_adam_error_string(rc)
    torch.cuda.synchronize()
    return [[t.cpu().numpy() for t in leaf] for leaf in dev]


def test_two_calls_in_a_row_the_second_smaller_then_one_beyond_the_limit():
    assert torch.cuda.is_available(), 'this test needs a GPU; there is no fallback path'
    lib = _lib.load()
    rng = np.random.default_rng(77)
    first = [int(x) for x in rng.integers(0, 4000, size=300)]
    first[5], first[17], first[250] = 0, 300_001, 256 * 600
    second = [int(x) for x in rng.integers(1, 2500, size=110)]
    second[3] = 70_001
    for label, sizes, counts, count_all, seed in (
            ('first call: 300 tensors', first, None, 7, 1),
            ('second call: 110 tensors, one step count each of three', second,
             [(1, 5, 1000)[k % 3] for k in range(len(second))], 0, 2)):
        leaves = make(sizes, seed)
        print(f'toa_adam_forward_inplace_multi_noalloc f32, {label}', flush=True)
        got = call(lib.toa_adam_forward_inplace_multi_noalloc, leaves, sizes, counts, count_all)
        want = call(lib.toa_adam_forward_inplace_multi, leaves, sizes, counts, count_all)
        for k, (g, w) in enumerate(zip(got, want)):
            for a, b, name in zip(g, w, ('updates', 'mu', 'nu')):
                assert_bit_equal(a, b, f'{label}: {name}[{k}] n={sizes[k]}')
        # and the existing entry point is itself the oracle's equal on a few members
        for k in (0, 3, len(sizes) - 1):
            c = count_all if counts is None else counts[k]
            e = O.forward_inplace(*[a.copy() for a in leaves[k]], B1, B2, EPS, 1e-8, c)
            for a, b, name in zip(got[k], e, ('updates', 'mu', 'nu')):
                assert_bit_equal(a, b, f'{label}: {name}[{k}] against the oracle')

    # 4097 non-empty tensors: refused, nothing launched, nothing written
    num = 4097
    flat = torch.ones(3 * num, device='cuda')
    before = flat.clone()
    ptrs = lambda off: (ctypes.c_void_p * num)(*[flat.data_ptr() + 4 * (3 * k + off) for k in range(num)])
    print('toa_adam_forward_inplace_multi_noalloc f32, 4097 tensors (over the limit)', flush=True)
    rc = lib.toa_adam_forward_inplace_multi_noalloc(
        _lib.TOA_F32, num, ptrs(0), ptrs(1), ptrs(2), (ctypes.c_size_t * num)(*([1] * num)), B1, B2,
        EPS, 0.0, None, 1, torch.cuda.current_stream().cuda_stream)
    assert rc == TOA_ELIMIT
    assert b'4096' in lib.toa_adam_error_string(rc)
    torch.cuda.synchronize()
    assert torch.equal(flat, before)
    # exactly at the limit: served (empty members do not count)
    num = 4096 + 2
    sizes = [1] * 4096 + [0, 0]
    flat = torch.full((3 * num,), 0.5, device='cuda')
    want = flat.clone()
    ptrs = lambda t, off: (ctypes.c_void_p * num)(*[t.data_ptr() + 4 * (3 * k + off) for k in range(num)])
    args = ((ctypes.c_size_t * num)(*sizes), B1, B2, EPS, 0.0, None, 1,
            torch.cuda.current_stream().cuda_stream)
    print('toa_adam_forward_inplace_multi_noalloc f32, 4096 one-element tensors', flush=True)
    assert lib.toa_adam_forward_inplace_multi_noalloc(_lib.TOA_F32, num, ptrs(flat, 0), ptrs(flat, 1),
                                                      ptrs(flat, 2), *args) == 0
    assert lib.toa_adam_forward_inplace_multi(_lib.TOA_F32, num, ptrs(want, 0), ptrs(want, 1),
                                              ptrs(want, 2), *args) == 0
    torch.cuda.synchronize()
    assert torch.equal(flat.view(torch.int32), want.view(torch.int32))
