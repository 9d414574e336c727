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


def _lists(sizes, seed):
    """Device lists (updates, mu, nu) for `sizes`, the host copies, and the ctypes arguments."""
    leaves = make(sizes, seed)
    dev = [[torch.from_numpy(a).cuda() for a in leaf] for leaf in leaves]
    num = len(sizes)
    cols = [(ctypes.c_void_p * num)(*[leaf[j].data_ptr() for leaf in dev]) for j in range(3)]
    return leaves, dev, cols, (ctypes.c_size_t * num)(*sizes)


def test_no_device_memory_is_allocated_and_a_long_list_uses_the_finer_index():
    """After a first call (which looks up the array's address) the free device memory reads the
    same before and after calls with lists of every length up to the limit -- among them lists
    of more than 1664 tensors, whose finer tile index lives in the same array."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    prepared = []
    for num, seed in ((40, 3), (1700, 4), (4096, 5)):
        rng = np.random.default_rng(seed)
        sizes = [int(x) for x in rng.integers(1, 900, size=num)]
        sizes[num // 2] = 200_003  # one large tensor beside thousands of small ones
        prepared.append((sizes, *_lists(sizes, seed), *_lists(sizes, seed)))
    # warm-up: symbol lookup, the allocating entry point's plan cache
    for sizes, _, dev_a, cols_a, ns_a, _, dev_b, cols_b, ns_b in prepared[:1]:
        assert lib.toa_adam_forward_inplace_multi_noalloc(
            _lib.TOA_F32, len(sizes), *cols_a, ns_a, B1, B2, EPS, 0.0, None, 1, stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for sizes, _, dev_a, cols_a, ns_a, _, dev_b, cols_b, ns_b in prepared:
        print(f'toa_adam_forward_inplace_multi_noalloc f32, {len(sizes)} tensors, free memory',
              flush=True)
        for count in (2, 3):
            assert lib.toa_adam_forward_inplace_multi_noalloc(
                _lib.TOA_F32, len(sizes), *cols_a, ns_a, B1, B2, EPS, 0.0, None, count,
                stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    # same steps through the allocating entry point (on the first list: one step more, the
    # warm-up's), bit for bit
    for k, (sizes, _, dev_a, cols_a, ns_a, _, dev_b, cols_b, ns_b) in enumerate(prepared):
        for count in ((1, 2, 3) if k == 0 else (2, 3)):
            assert lib.toa_adam_forward_inplace_multi(
                _lib.TOA_F32, len(sizes), *cols_b, ns_b, B1, B2, EPS, 0.0, None, count,
                stream) == 0
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(dev_a, dev_b)):
            for x, y, name in zip(a, b, ('updates', 'mu', 'nu')):
                assert torch.equal(x.view(torch.int32), y.view(torch.int32)), \
                    f'{len(sizes)} tensors: {name}[{i}] n={sizes[i]}'


def test_captured_in_a_graph_and_replayed_on_fresh_gradients():
    """The use the entry point is for: one call captured into a HIP graph (after a call outside
    capture, so the array's address is known), replayed twice with new gradients copied into the
    captured arrays, against the allocating entry point run eagerly on copies."""
    lib = _lib.load()
    rng = np.random.default_rng(11)
    sizes = [int(x) for x in rng.integers(1, 3000, size=200)]
    sizes[7] = 150_001
    leaves, dev, cols, ns = _lists(sizes, 11)
    _, ref, ref_cols, ref_ns = _lists(sizes, 11)
    num = len(sizes)
    side = torch.cuda.Stream()
    # outside capture first: on scratch copies, so the captured state starts pristine
    _, scratch, scratch_cols, scratch_ns = _lists(sizes, 12)
    assert lib.toa_adam_forward_inplace_multi_noalloc(
        _lib.TOA_F32, num, *scratch_cols, scratch_ns, B1, B2, EPS, 1e-8, None, 4,
        torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    print('toa_adam_forward_inplace_multi_noalloc f32, 200 tensors, under stream capture',
          flush=True)
    with torch.cuda.graph(graph, stream=side):
        rc = lib.toa_adam_forward_inplace_multi_noalloc(
            _lib.TOA_F32, num, *cols, ns, B1, B2, EPS, 1e-8, None, 4,
            torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.toa_adam_error_string(rc)
    torch.cuda.synchronize()
    # capture launches nothing: the state is untouched
    for leaf, d in zip(leaves, dev):
        assert np.array_equal(d[1].cpu().numpy(), leaf[1])

    for replay in range(2):
        fresh = [torch.from_numpy(rng.standard_normal(n).astype(np.float32)).cuda() for n in sizes]
        for d, r, g in zip(dev, ref, fresh):
            d[0].copy_(g)
            r[0].copy_(g)
        # other work of the library between replays rewrites nothing the graph depends on but
        # the array itself, which every replay rewrites first
        assert lib.toa_adam_forward_inplace_multi_noalloc(
            _lib.TOA_F32, num, *scratch_cols, scratch_ns, B1, B2, EPS, 1e-8, None, 9,
            torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        print(f'replay {replay + 1} of the captured graph', flush=True)
        graph.replay()
        assert lib.toa_adam_forward_inplace_multi(
            _lib.TOA_F32, num, *ref_cols, ref_ns, B1, B2, EPS, 1e-8, None, 4,
            torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(dev, ref)):
            for x, y, name in zip(a, b, ('updates', 'mu', 'nu')):
                assert torch.equal(x.view(torch.int32), y.view(torch.int32)), \
                    f'replay {replay + 1}: {name}[{i}] n={sizes[i]}'
