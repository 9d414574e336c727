#!/usr/bin/env python3
"""Benchmark of the fused Adam operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config {0,...,7}]

A "step" is one pass of the hot path over one batch of synthetic state that is already
resident in HBM: for the default workload (config 2) one fused in-place `forward_` over three
float32 arrays of 268 435 456 elements (1 GiB each), launched through the C ABI of
libtoa_adam.so on PyTorch's current stream.  W untimed steps, then exactly K timed steps
bracketed by `torch.cuda.synchronize()`; one JSON line on stdout.

Beside the headline `value` (elements per second) the line carries
  roofline      achieved HBM bandwidth of the kernel: algorithmic bytes per launch (24 B per
                float32 element for forward_) over the average launch duration, measured with
                events on the launch stream across the timed region, against 8 TB/s;
  cpu_baseline  the reference's CPU op (or this repo's bit-identical C port of it) timed on the
                host's cores on a bounded sample of the same workload, and with it the parity of
                the GPU's result with the CPU's on that sample (differing elements, max ulp).

`--ceiling` measures, instead of the operator, what this machine's HBM delivers to streaming
kernels of the same launch shape that do next to no arithmetic (bench_probe.hip: R arrays read,
W arrays written, at every residency level), and prints those ceilings as one JSON line: the
context for `roofline.frac`.

Everything on one GPU: `--gpus N` with N > 1 is refused.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBS = 8000.0  # MI355X published peak HBM3E bandwidth

# Algorithmic bytes per element: every operand array is read or written exactly once.
BYTES_PER_ELEM = {  # op -> number of arrays streamed (multiply by the element size)
    'forward_': 6, 'forward_mu': 3, 'forward_nu': 3, 'forward_updates': 3,
    'backward_mu': 3, 'backward_nu': 4, 'backward_updates': 5,
}

# HBM bytes per step as counted by rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE in separate runs,
# each scaled by what the same counter reads for a plain 1 GiB copy: x1.99996 and x1.0); the
# commands and raw readings are in profiles/*pmc_traffic*.md.  Not measured live: a counter run
# serialises the kernels, so it cannot share a process with the timed region.
MEASURED_TRAFFIC_BYTES = {2: 6442431962, 4: 8516628944}

B1, B2, EPS = 0.9, 0.999, 1e-8


# ----------------------------------------------------------------------------- workloads


def maml_shapes():
    """Config 1: MAML-style conv net, 10 tensors, 32 645 elements."""
    return ([(32, 3, 3, 3)] + [(32, 32, 3, 3)] * 3 + [(32,)] * 4 + [(5, 800), (5,)])


def gpt2_medium_shapes():
    """Config 4: GPT-2-medium parameter list (24 layers, d=1024), embeddings last."""
    shapes = []
    for _ in range(24):
        shapes += [(3072, 1024), (3072,), (1024, 1024), (1024,), (4096, 1024), (4096,),
                   (1024, 4096), (1024,), (1024,), (1024,), (1024,), (1024,)]
    shapes += [(50257, 1024), (1024, 1024)]
    return shapes


def alg_small(array_bytes):
    """True when one operand array (and so the whole working set of three) sits in cache."""
    return array_bytes <= (32 << 20)


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


CONFIGS = {
    0: dict(name='config0: fused forward_ in place, 1 048 576 float32 elements, count=10',
            dtype='f32', n=1 << 20, eps_root=0.0, count=10),
    1: dict(name='config1: forward mu/nu/updates + backward updates/nu/mu over the MAML pytree '
                 '(10 float32 tensors, 32 645 elements), one multi-tensor pass per direction',
            dtype='f32', shapes=maml_shapes(), eps_root=1e-8, count=5, differentiable=True),
    2: dict(name='config2: fused forward_ in place, 268 435 456 float32 elements '
                 '(1 GiB per state array), count=1000',
            dtype='f32', n=1 << 28, eps_root=0.0, count=1000),
    3: dict(name='config3: fused forward_ in place, 67 108 864 float64 elements, count=3; beside '
                 'it the backward ops on the same shapes',
            dtype='f64', n=1 << 26, eps_root=1e-8, count=3, backward=True),
    4: dict(name='config4: multi-tensor forward_ in place over the GPT-2-medium parameter list '
                 '(float32), count=1',
            dtype='f32', shapes=gpt2_medium_shapes(), eps_root=0.0, count=1),
    5: dict(name='config5: classic optimizer step (Adam + scale(-lr) + apply) in one pass over the '
                 'GPT-2-medium parameter list (float32), count=1; beside it the three-pass chain',
            dtype='f32', shapes=gpt2_medium_shapes(), eps_root=0.0, count=1, fused_step=True),
    6: dict(name='config6: fused forward_ in place, 268 435 456 float16 elements (arithmetic of '
                 'the reference CPU op on at::Half: every operation rounded to 16 bits), '
                 'eps=1e-3, count=1000, a fresh gradient array every step',
            dtype='f16', n=1 << 28, eps=1e-3, eps_root=0.0, count=1000, fresh_gradients=True),
    7: dict(name='config7: fused forward_ in place, 268 435 456 bfloat16 elements (arithmetic of '
                 'the reference CPU op on at::BFloat16), eps=1e-3, count=1000, a fresh gradient array '
                 'every step',
            dtype='bf16', n=1 << 28, eps=1e-3, eps_root=0.0, count=1000, fresh_gradients=True),
}
ESIZE = {'f32': 4, 'f64': 8, 'f16': 2, 'bf16': 2}


# ----------------------------------------------------------------------------- GPU side


def make_state(torch, n, dtype, seed):
    """updates ~ N(0,1), mu ~ 0.1 N(0,1), nu ~ |0.01 N(0,1)|, generated on the GPU."""
    g = torch.Generator(device='cuda')
    g.manual_seed(seed)
    wide = torch.float32 if dtype in (torch.float16, torch.bfloat16) else dtype
    u = torch.randn(n, device='cuda', dtype=wide, generator=g).to(dtype)
    mu = torch.randn(n, device='cuda', dtype=wide, generator=g).mul_(0.1).to(dtype)
    nu = torch.randn(n, device='cuda', dtype=wide, generator=g).mul_(0.01).abs_().to(dtype)
    return u, mu, nu


def python_level_differentiable_step(torch, shapes, eps_root, count, wall_ms):
    """What a meta-learning loop pays per inner step, from Python through autograd: the Adam
    transformation's differentiable `update` over the tree plus the backward through it, next to
    the same mathematics written as per-leaf PyTorch tensor expressions (the route a build
    without the fused operator takes)."""
    from torchopt_amd.transform import scale_by_accelerated_adam

    grads = tuple(torch.randn(s, device='cuda', requires_grad=True) for s in shapes)
    transform = scale_by_accelerated_adam(B1, B2, EPS, eps_root, moment_requires_grad=True)
    state = transform.init(grads)
    c1, c2 = 1 / (1 - B1 ** count), 1 / (1 - B2 ** count)

    def fused():
        updates, _ = transform.update(grads, state, inplace=False)
        torch.autograd.grad(sum((u * u).sum() for u in updates), grads)

    def per_leaf_expressions():
        updates = []
        for g, m, v in zip(grads, state.mu, state.nu):
            m1 = m * B1 + g * (1 - B1)
            v1 = v * B2 + g * g * (1 - B2)
            updates.append((m1 * c1) / (torch.sqrt(v1 * c2 + eps_root) + EPS))
        torch.autograd.grad(sum((u * u).sum() for u in updates), grads)

    def loss_alone():  # the part of both that is not Adam
        torch.autograd.grad(sum((g * g).sum() for g in grads), grads)

    base = wall_ms(loss_alone)
    return {'python_update_plus_backward_ms': round(wall_ms(fused) - base, 5),
            'python_per_leaf_tensor_expressions_ms': round(wall_ms(per_leaf_expressions) - base, 5)}


def time_backward_ops(torch, lib, code, dtype, n, esize, eps_root, count, stream, reps=20):
    """backward_mu, backward_nu, backward_updates and the one-pass backward_all on flat arrays of
    n elements: ms per launch and achieved GB/s (algorithmic bytes: 3, 4, 5 and 9 arrays)."""
    g = torch.Generator(device='cuda')
    g.manual_seed(77)
    arrays = [torch.randn(n, device='cuda', dtype=dtype, generator=g) for _ in range(9)]
    arrays[2].mul_(0.1)
    p = [a.data_ptr() for a in arrays]
    s = stream.cuda_stream
    # slots: 0 updates / dupdates, 1 new_updates, 2 new_mu, 3 dmu, 4 dnu, 5..8 outputs
    ops = {
        'backward_mu': (3, lambda: lib.toa_adam_backward_mu(code, p[3], n, B1, p[5], p[6], s)),
        'backward_nu': (4, lambda: lib.toa_adam_backward_nu(code, p[4], p[0], n, B2, p[5], p[6],
                                                            s)),
        'backward_updates': (5, lambda: lib.toa_adam_backward_updates(
            code, p[0], p[1], p[2], n, B1, B2, eps_root, count, p[5], p[6], s)),
        'backward_all': (9, lambda: lib.toa_adam_backward_all(
            code, p[0], p[1], p[2], p[8], p[3], p[4], n, B1, B2, eps_root, count, p[5], p[6],
            p[7], s)),
    }
    out = {}
    for name, (streams, fn) in ops.items():
        for _ in range(5):
            rc = fn()
            if rc:
                raise RuntimeError(f'{name}: {lib.toa_adam_error_string(rc).decode()}')
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out[name] = {'ms': round(ms, 5), 'GB/s': round(streams * esize * n / ms / 1e6, 1)}
    return out


def run_gpu(cfg_id, steps, warmup):
    import torch

    from torchopt_amd import _lib

    if not torch.cuda.is_available():
        raise SystemExit('bench.py needs a GPU: the fused Adam op has no CPU path')
    lib = _lib.load()
    cfg = CONFIGS[cfg_id]
    dtype = {'f32': torch.float32, 'f64': torch.float64, 'f16': torch.float16,
             'bf16': torch.bfloat16}[cfg['dtype']]
    code = {'f32': _lib.TOA_F32, 'f64': _lib.TOA_F64, 'f16': _lib.TOA_F16,
            'bf16': _lib.TOA_BF16}[cfg['dtype']]
    esize = ESIZE[cfg['dtype']]
    eps = cfg.get('eps', EPS)
    stream = torch.cuda.current_stream()
    sptr = stream.cuda_stream
    eps_root, count = cfg['eps_root'], cfg['count']

    bytes_per_elem = BYTES_PER_ELEM['forward_'] * esize
    if cfg.get('differentiable'):
        import ctypes

        sizes = [numel(s) for s in cfg['shapes']]
        total, num = sum(sizes), len(sizes)
        g = torch.Generator(device='cuda')
        g.manual_seed(1000 * cfg_id)

        def fresh():
            return [torch.randn(n, device='cuda', dtype=dtype, generator=g) for n in sizes]

        def arr(ts):
            return (ctypes.c_void_p * num)(*[t.data_ptr() for t in ts])

        ups, mus, nus = fresh(), [t.mul_(0.1) for t in fresh()], [t.mul_(0.01).abs_() for t in fresh()]
        d_u, d_m, d_v = fresh(), fresh(), fresh()
        outs = [fresh() for _ in range(9)]  # new_mu, new_nu, new_u, 2 x 3 backward outputs
        keep = (ups, mus, nus, d_u, d_m, d_v, outs)  # noqa: F841  (owns the device memory)
        a_up, a_mu, a_nu, a_du, a_dm, a_dv = (arr(x) for x in (ups, mus, nus, d_u, d_m, d_v))
        o = [arr(x) for x in outs]
        ns = (ctypes.c_size_t * num)(*sizes)

        def check(rc):
            if rc:
                raise RuntimeError(lib.toa_adam_error_string(rc).decode())

        def six_launch_step():
            check(lib.toa_adam_forward_mu_multi(code, num, a_up, a_mu, ns, B1, o[0], sptr))
            check(lib.toa_adam_forward_nu_multi(code, num, a_up, a_nu, ns, B2, o[1], sptr))
            check(lib.toa_adam_forward_updates_multi(code, num, o[0], o[1], ns, B1, B2, EPS,
                                                     eps_root, None, count, o[2], sptr))
            check(lib.toa_adam_backward_updates_multi(code, num, a_du, o[2], o[0], ns, B1, B2,
                                                      eps_root, None, count, o[3], o[4], sptr))
            check(lib.toa_adam_backward_nu_multi(code, num, a_dv, a_up, ns, B2, o[5], o[6], sptr))
            check(lib.toa_adam_backward_mu_multi(code, num, a_dm, ns, B1, o[7], o[8], sptr))

        def step():  # the whole differentiable step: one pass forward, one pass backward
            check(lib.toa_adam_forward_all_multi(code, num, a_up, a_mu, a_nu, ns, B1, B2, EPS,
                                                 eps_root, None, count, o[0], o[1], o[2], sptr))
            check(lib.toa_adam_backward_all_multi(code, num, a_du, o[2], o[0], a_up, a_dm, a_dv,
                                                  ns, B1, B2, eps_root, None, count, o[3], o[4],
                                                  o[5], sptr))

        ptrs = [[t.data_ptr() for t in x] for x in (ups, mus, nus, d_u, d_m, d_v, *outs)]

        def per_tensor_step():  # what the reference's per-leaf loop launches: 6 kernels per leaf
            for k, n in enumerate(sizes):
                p = [x[k] for x in ptrs]
                lib.toa_adam_forward_mu(code, p[0], p[1], n, B1, p[6], sptr)
                lib.toa_adam_forward_nu(code, p[0], p[2], n, B2, p[7], sptr)
                lib.toa_adam_forward_updates(code, p[6], p[7], n, B1, B2, EPS, eps_root, count,
                                             p[8], sptr)
                lib.toa_adam_backward_updates(code, p[3], p[8], p[6], n, B1, B2, eps_root, count,
                                              p[9], p[10], sptr)
                lib.toa_adam_backward_nu(code, p[5], p[0], n, B2, p[11], p[12], sptr)
                lib.toa_adam_backward_mu(code, p[4], n, B1, p[13], p[14], sptr)

        def wall_ms(fn):
            for _ in range(warmup):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / steps

        per_leaf_ms = wall_ms(per_tensor_step)
        six_ms = wall_ms(six_launch_step)
        # the one-pass pair streams 24 + 36 bytes per float32 element (3R+3W, 6R+3W); the
        # separate ops stream 84
        bytes_per_elem = (6 + 9) * esize
        extra = {'tensors': num, 'launches_per_step': 2,
                 'six_list_launches_ms_per_step': round(six_ms, 5),
                 'per_leaf_loop_ms_per_step': round(per_leaf_ms, 5),
                 'per_leaf_loop_launches_per_step': 6 * num,
                 **python_level_differentiable_step(torch, cfg['shapes'], eps_root, count,
                                                    wall_ms)}
    elif 'shapes' in cfg:
        import ctypes

        sizes = [numel(s) for s in cfg['shapes']]
        total = sum(sizes)
        # Allocation order as the Adam transformation produces it: the gradients of the whole
        # tree, then mu for every leaf, then nu for every leaf (init_fn maps zeros_like over
        # the tree once per moment, /root/reference/torchopt/transform/scale_by_adam.py:401-414),
        # so the three arrays of one leaf lie far apart.
        gens = []
        for k in range(len(sizes)):
            g = torch.Generator(device='cuda')
            g.manual_seed(1000 * cfg_id + k)
            gens.append(g)
        us = [torch.randn(n, device='cuda', dtype=dtype, generator=g) for n, g in zip(sizes, gens)]
        ms = [torch.randn(n, device='cuda', dtype=dtype, generator=g).mul_(0.1)
              for n, g in zip(sizes, gens)]
        vs = [torch.randn(n, device='cuda', dtype=dtype, generator=g).mul_(0.01).abs_()
              for n, g in zip(sizes, gens)]
        tensors = list(zip(us, ms, vs))
        num = len(sizes)
        pu = (ctypes.c_void_p * num)(*[t[0].data_ptr() for t in tensors])
        pm = (ctypes.c_void_p * num)(*[t[1].data_ptr() for t in tensors])
        pv = (ctypes.c_void_p * num)(*[t[2].data_ptr() for t in tensors])
        ns = (ctypes.c_size_t * num)(*sizes)

        def step():
            rc = lib.toa_adam_forward_inplace_multi(code, num, pu, pm, pv, ns, B1, B2, EPS,
                                                    eps_root, None, count, sptr)
            if rc:
                raise RuntimeError(lib.toa_adam_error_string(rc).decode())
        extra = {'tensors': num}
        if cfg.get('fused_step'):
            ps = [torch.randn(n, device='cuda', dtype=dtype, generator=g)
                  for n, g in zip(sizes, gens)]
            pp = (ctypes.c_void_p * num)(*[t.data_ptr() for t in ps])
            lr = 1e-3

            def chain_step():  # the reference's three passes, per-leaf PyTorch kernels for two
                step()
                torch._foreach_mul_(us, -lr)
                torch._foreach_add_(ps, us)

            for _ in range(3):
                chain_step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                chain_step()
            torch.cuda.synchronize()
            chain_ms = (time.perf_counter() - t0) * 1e3 / steps

            def step():  # noqa: F811
                rc = lib.toa_adam_fused_step_multi(code, num, pp, pu, pm, pv, ns, B1, B2, EPS,
                                                   eps_root, None, count, lr, 0.0, 0, 0, 0, sptr)
                if rc:
                    raise RuntimeError(lib.toa_adam_error_string(rc).decode())
            bytes_per_elem = 7 * esize  # reads g, mu, nu, p; writes mu, nu, p
            extra.update(three_pass_chain_ms_per_step=round(chain_ms, 5),
                         three_pass_chain_bytes_per_element=11 * esize)
    else:
        total = cfg['n']
        u, mu, nu = make_state(torch, total, dtype, 1000 * cfg_id)
        pu, pm, pv = u.data_ptr(), mu.data_ptr(), nu.data_ptr()

        extra = {}
        if cfg.get('fresh_gradients'):
            # A training loop hands the step a new gradient every time; re-applying the step to
            # its own output instead drives every element towards one fixed point, which no real
            # run does and which the 16-bit kernels' data-dependent quick route would be timed
            # on.  So each step gets its own freshly drawn gradient array (as many as the step
            # count, at most 64 of them in rotation).
            g = torch.Generator(device='cuda')
            g.manual_seed(1000 * cfg_id + 1)
            fresh = [torch.randn(total, device='cuda', generator=g).to(dtype)
                     for _ in range(min(steps + warmup, 64))]
            ptrs, turn = [t.data_ptr() for t in fresh], [0]
            extra['gradient_arrays'] = len(fresh)

            def step():
                k = turn[0]
                turn[0] = (k + 1) % len(ptrs)
                rc = lib.toa_adam_forward_inplace(code, ptrs[k], pm, pv, total, B1, B2, eps,
                                                  eps_root, count, sptr)
                if rc:
                    raise RuntimeError(lib.toa_adam_error_string(rc).decode())
        else:
            def step():
                rc = lib.toa_adam_forward_inplace(code, pu, pm, pv, total, B1, B2, eps, eps_root,
                                                  count, sptr)
                if rc:
                    raise RuntimeError(lib.toa_adam_error_string(rc).decode())
        if cfg.get('backward'):
            extra['backward_ops'] = time_backward_ops(torch, lib, code, dtype, total, esize,
                                                      eps_root, count, stream)
        if alg_small(total * esize):
            # The timed loop below re-runs on state that stays in the 256 MB Infinity Cache; a
            # real optimizer step finds its state in HBM.  Time single launches after sweeping
            # 512 MB through the caches as well.
            sweep = torch.empty(512 << 20, dtype=torch.uint8, device='cuda')
            cold = []
            for _ in range(10):
                sweep.fill_(1)
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                step()
                b.record(stream)
                torch.cuda.synchronize()
                cold.append(a.elapsed_time(b))
            del sweep
            extra['cold_cache_ms_per_launch'] = round(sorted(cold)[len(cold) // 2], 5)

    for _ in range(warmup):
        step()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(steps):
        step()
    ev1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    # per-step spread, from a second short pass with one pair of events per step (outside the
    # timed region; event overhead makes it meaningless for microsecond steps)
    spread = {}
    if (t1 - t0) * 1e3 / steps > 0.05:
        pairs = []
        for _ in range(min(steps, 20)):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            step()
            b.record(stream)
            pairs.append((a, b))
        torch.cuda.synchronize()
        each = sorted(a.elapsed_time(b) for a, b in pairs)
        spread = {'step_ms_min': round(each[0], 5), 'step_ms_median': round(each[len(each) // 2], 5)}

    wall_ms = (t1 - t0) * 1e3 / steps
    kern_ms = ev0.elapsed_time(ev1) / steps  # stream time per launch (launches are back to back)
    alg_bytes = bytes_per_elem * total
    achieved = alg_bytes / (kern_ms * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC_BYTES.get(cfg_id)
    return {
        'elements': total,
        'ms_per_step': wall_ms,
        'value': total / (wall_ms * 1e-3),
        'roofline': {
            'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
            'frac': round(achieved / HBM_PEAK_GBS, 4), 'traffic': traffic,
            'kernel_ms': round(kern_ms, 5), 'algorithmic_bytes_per_launch': alg_bytes,
            'bytes_per_element': bytes_per_elem, **spread,
        },
        'extra': extra,
        'device': torch.cuda.get_device_name(0),
    }


# ----------------------------------------------------------------------------- HBM ceilings

PROBE_SRC = os.path.join(REPO, 'bench_probe.hip')
PROBE_LIB = os.path.join(REPO, 'bench_probe.so')
RESIDENCY_LEVELS = (32, 25, 21, 18, 16, 14, 12, 11, 10, 9, 8)  # floor(128 / LDS granules)


def build_probe():
    """hipcc -> bench_probe.so (cross-compiles without a GPU)."""
    import subprocess

    subprocess.run(['hipcc', '-O3', '-std=c++17', '--offload-arch=gfx950', '-fPIC', '-shared',
                    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
                    '-fvisibility=hidden', '-o', PROBE_LIB, PROBE_SRC], check=True,
                   stderr=subprocess.DEVNULL)
    return PROBE_LIB


def lds_for_waves(waves):
    """Dynamic LDS per single-wave workgroup that caps a gfx950 CU (128 granules of 1280 B) at
    `waves` resident workgroups."""
    return 0 if waves >= 32 else (128 // (waves + 1) + 1) * 1280


def run_ceiling(array_bytes=1 << 30, reps=20):
    import ctypes

    import torch

    if not os.path.exists(PROBE_LIB):
        build_probe()
    probe = ctypes.CDLL(PROBE_LIB)
    probe.bench_probe_stream.restype = ctypes.c_int
    probe.bench_probe_stream.argtypes = [ctypes.c_int, ctypes.c_int,
                                         ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t,
                                         ctypes.c_uint, ctypes.c_void_p]
    stream = torch.cuda.current_stream()
    arrays = [torch.rand(array_bytes // 4, device='cuda') for _ in range(7)]
    torch.cuda.synchronize()
    out = {}
    shapes = [(r, w, False) for r, w in ((1, 0), (3, 0), (0, 1), (0, 3), (1, 1), (2, 1), (3, 3),
                                         (4, 3))]
    shapes += [(3, 3, True), (4, 3, True)]  # written back over the arrays just read, as forward_
    for reads, writes, in_place in shapes:
        order = list(range(reads)) + (list(range(reads - writes, reads)) if in_place
                                      else list(range(reads, reads + writes)))
        ptrs = (ctypes.c_void_p * (reads + writes))(*[arrays[k].data_ptr() for k in order])
        best = (0.0, None)
        for waves in RESIDENCY_LEVELS:
            def launch():
                rc = probe.bench_probe_stream(reads, writes, ptrs, array_bytes,
                                              lds_for_waves(waves), stream.cuda_stream)
                if rc:
                    raise RuntimeError(f'bench_probe_stream({reads}, {writes}) returned {rc}')
            for _ in range(4):
                launch()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record(stream)
            for _ in range(reps):
                launch()
            ev1.record(stream)
            torch.cuda.synchronize()
            gbs = (reads + writes) * array_bytes / (ev0.elapsed_time(ev1) / reps * 1e-3) / 1e9
            if gbs > best[0]:
                best = (gbs, waves)
        out[f'{reads}R{writes}W' + (' in place' if in_place else '')] = {'GB/s': round(best[0], 1), 'frac_of_peak': round(
            best[0] / HBM_PEAK_GBS, 4), 'waves_per_cu': best[1]}
    return {'metric': 'hbm_streaming_ceiling', 'unit': 'GB/s', 'peak': HBM_PEAK_GBS,
            'array_bytes': array_bytes, 'launches_timed': reps,
            'device': torch.cuda.get_device_name(0), 'ceilings': out}


# ----------------------------------------------------------------------------- CPU baseline


def run_cpu_baseline(cfg_id, budget_s=12.0):
    """Time the reference CPU op (oracle/_ref, where built) or the C port on a bounded sample.

    Only this leg touches `oracle/`; it is the reported baseline, never the measured product.
    """
    import numpy as np

    from oracle import adam_oracle

    cfg = CONFIGS[cfg_id]
    tag = cfg['dtype']
    np_dtype = {'f32': np.float32, 'f64': np.float64, 'f16': np.float16, 'bf16': np.float32}[tag]
    eps = cfg.get('eps', EPS)
    full = cfg['n'] if 'n' in cfg else sum(numel(s) for s in cfg['shapes'])
    n = min(full, 1 << 26)

    # the box's CPU share, not every core the machine shows
    share = int(os.environ.get('OMP_NUM_THREADS', '16') or 16)
    try:
        avail = sorted(os.sched_getaffinity(0))
        cores = max(1, min(share, len(avail)))
        os.sched_setaffinity(0, set(avail[:cores]))
    except (AttributeError, OSError):
        cores = max(1, min(share, os.cpu_count() or 1))

    rng = np.random.default_rng(1000 * cfg_id)
    block = 1 << 20
    reps = (n + block - 1) // block
    u = np.tile(rng.standard_normal(block).astype(np_dtype), reps)[:n].copy()
    mu = np.tile((0.1 * rng.standard_normal(block)).astype(np_dtype), reps)[:n].copy()
    nu = np.tile(np.abs(0.01 * rng.standard_normal(block)).astype(np_dtype), reps)[:n].copy()
    if tag == 'bf16':  # bfloat16 travels as uint16 bit patterns on the NumPy side
        u, mu, nu = (adam_oracle.bf16_bits(a) for a in (u, mu, nu))

    def as_torch(a):
        t = torch.from_numpy(a.view(np.int16) if tag == 'bf16' else a)
        return t.view(torch.bfloat16) if tag == 'bf16' else t

    ref = None
    try:
        ref = adam_oracle.load_reference()
    except Exception as exc:  # noqa: BLE001
        print(f'[bench] compiled reference not usable ({exc}); timing the C port',
              file=sys.stderr)
    import torch

    from torchopt_amd import _lib

    if ref is not None:
        tu, tm, tv = as_torch(u), as_torch(mu), as_torch(nu)  # share memory with u, mu, nu

        def one():
            ref.adam_op.forward_(tu, tm, tv, B1, B2, eps, cfg['eps_root'], cfg['count'])
        kind = 'reference'
    else:
        def one():
            adam_oracle.forward_inplace(u, mu, nu, B1, B2, eps, cfg['eps_root'], cfg['count'])
        kind = 'port'

    # Parity on this sample: the GPU's first application from the seeded state against the
    # CPU's (which doubles as the CPU warm-up: threads, page faults).
    dev = [as_torch(a).cuda() for a in (u, mu, nu)]
    code = {'f32': _lib.TOA_F32, 'f64': _lib.TOA_F64, 'f16': _lib.TOA_F16,
            'bf16': _lib.TOA_BF16}[tag]
    rc = _lib.load().toa_adam_forward_inplace(
        code, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(), n, B1, B2, eps,
        cfg['eps_root'], cfg['count'], torch.cuda.current_stream().cuda_stream)
    if rc:
        raise RuntimeError(f'toa_adam_forward_inplace returned {rc}')
    one()
    itype = {2: np.int16, 4: np.int32, 8: np.int64}[ESIZE[tag]]
    worst, differing = 0, 0
    for got, want in zip(dev, (u, mu, nu)):
        got = got.view(torch.int16) if tag == 'bf16' else got
        a = got.cpu().numpy().view(itype).astype(np.int64)
        b = want.view(itype).astype(np.int64)
        lo = np.iinfo(itype).min
        a, b = np.where(a < 0, lo - a, a), np.where(b < 0, lo - b, b)  # monotone integer line
        d = np.abs(a - b)
        worst, differing = max(worst, int(d.max())), differing + int(np.count_nonzero(d))
    del dev
    parity = {'elements_checked': 3 * n, 'differing': differing, 'max_ulp': worst}

    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 25):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    esize = ESIZE[tag]
    return {
        'value': n / med, 'unit': 'elements/s', 'cores': cores, 'kind': kind,
        'sample': f'{n} of {full} elements ({cfg["dtype"]}), forward_ in place, '
                  f'median of {len(times)} passes after 1 warm-up',
        'gb_per_s': round(BYTES_PER_ELEM['forward_'] * esize * n / med / 1e9, 2),
        'parity_gpu_vs_cpu': parity,
    }


# ----------------------------------------------------------------------------- main


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split('\n')[0])
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--config', type=int, default=2, choices=sorted(CONFIGS))
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--pmc-calibration', action='store_true',
                    help='after the timed region also run 5 plain device copies of 1 GiB, so a '
                         'rocprofv3 --pmc run holds a kernel of known traffic to scale '
                         'FETCH_SIZE / WRITE_SIZE by')
    ap.add_argument('--ceiling', action='store_true',
                    help='measure the streaming ceilings of this machine (probe kernels with '
                         'the operator\'s launch shape) instead of the operator')
    args = ap.parse_args(argv)

    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this build measures one GPU only (the op needs no exchange between '
              'GPUs; each would run the same kernel on its shard). Run with --gpus 1.',
              file=sys.stderr)
        return 2

    if args.ceiling:
        print(json.dumps(run_ceiling()), flush=True)
        return 0

    gpu = run_gpu(args.config, args.steps, args.warmup)
    cfg = CONFIGS[args.config]
    if args.pmc_calibration:
        import torch

        src = torch.ones(1 << 28, device='cuda')
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    line = {
        'metric': ('adam_forward_backward_elements_per_s' if cfg.get('differentiable')
                   else 'adam_fused_step_elements_per_s' if cfg.get('fused_step')
                   else 'adam_forward_inplace_elements_per_s'),
        'value': gpu['value'],
        'unit': 'elements/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': gpu['ms_per_step'],
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': cfg['dtype'],
        'data': 'synthetic',
        'config': {'workload': cfg['name'], 'elements': gpu['elements'], 'b1': B1, 'b2': B2,
                   'eps': cfg.get('eps', EPS), 'eps_root': cfg['eps_root'], 'count': cfg['count'],
                   'device': gpu['device'], **gpu['extra']},
        'roofline': gpu['roofline'],
    }
    if not args.no_cpu_baseline:
        line['cpu_baseline'] = run_cpu_baseline(args.config)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == '__main__':
    sys.exit(main())
