#!/usr/bin/env python3
"""Benchmark of the fused Adam operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config {0,...,9}]
                    [--state {init,separate,plain}] [--operator-preheat N]

A "step" is one pass of the hot path over one batch of synthetic state that is already
resident in HBM: for the default workload (config 2) one fused in-place `forward_` over three
float32 arrays of 268 435 456 elements (1 GiB each), launched through the C ABI of
libtoa_adam.so on PyTorch's current stream.  W untimed steps, then exactly K timed steps
bracketed by `torch.cuda.synchronize()`; one JSON line on stdout.  The gradient array is a
PyTorch allocation; the two moments are allocated as the package's own init allocates state
(`--state init`: torchopt_amd.state_zeros_like_tree; `separate` and `plain` are there to show what
that placement is worth).  Before the W warm-up steps the bandwidth-bound configurations run the
operator 60-100 times on scratch state, past its start-up transient (`--operator-preheat 0`
switches that off); the line records both.

Beside the headline `value` (elements per second) the line carries
  roofline      achieved HBM bandwidth of the kernel: algorithmic bytes per launch (24 B per
                float32 element for forward_) over the average launch duration, measured with
                events on the launch stream across the timed region, against 8 TB/s;
  cpu_baseline  the reference's CPU op (or this repo's bit-identical C port of it) timed on the
                host's cores on a bounded sample of the same workload, and with it the parity of
                the GPU's result with the CPU's on that sample (differing elements, max ulp).

Everything on one GPU: `--gpus N` with N > 1 is refused.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

# Thread placement of the CPU baseline leg (read by the OpenMP runtime when it starts, so set
# before anything loads it); values already in the environment win and are what the line reports.
os.environ.setdefault('OMP_PROC_BIND', 'close')
os.environ.setdefault('OMP_PLACES', 'cores')

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
# each scaled by what the same counter reads for a plain 1 GiB copy); the commands and raw
# readings are in the profile named beside each figure.  RECORDED there, not measured live: a
# counter run serialises the kernels, so it cannot share a process with the timed region.  The
# figures belong to the kernels as they were when the profile was taken; re-record them whenever
# adam_kernels.hpp or the launch shape changes.
RECORDED_TRAFFIC = {
    2: (6442409480, 'profiles/forward_inplace_f32_config2_pmc_traffic.md'),
    4: (8516253697, 'profiles/forward_inplace_multi_f32_config4_kernel_trace_and_traffic.md'),
    5: (9935440703, 'profiles/fused_step_multi_f32_config5_kernel_trace_and_traffic.md'),
}

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
            dtype='f32', n=1 << 28, eps_root=0.0, count=1000, operator_preheat=60),
    3: dict(name='config3: fused forward_ in place, 67 108 864 float64 elements, count=3; beside '
                 'it the backward ops on the same shapes',
            dtype='f64', n=1 << 26, eps_root=1e-8, count=3, backward=True, operator_preheat=60),
    4: dict(name='config4: multi-tensor forward_ in place over the GPT-2-medium parameter list '
                 '(float32), count=1',
            dtype='f32', shapes=gpt2_medium_shapes(), eps_root=0.0, count=1, operator_preheat=60),
    5: dict(name='config5: classic optimizer step (Adam + scale(-lr) + apply) in one pass over the '
                 'GPT-2-medium parameter list (float32), count=1; beside it the three-pass chain',
            dtype='f32', shapes=gpt2_medium_shapes(), eps_root=0.0, count=1, fused_step=True,
            operator_preheat=60),
    6: dict(name='config6: fused forward_ in place, 268 435 456 float16 elements (arithmetic of '
                 'the reference CPU op on at::Half: every operation rounded to 16 bits), '
                 'eps=1e-3, count=1000, a fresh N(0,1) gradient array every step',
            dtype='f16', n=1 << 28, eps=1e-3, eps_root=0.0, count=1000, fresh_gradients=True,
            operator_preheat=100),
    7: dict(name='config7: fused forward_ in place, 268 435 456 bfloat16 elements (arithmetic of '
                 'the reference CPU op on at::BFloat16), eps=1e-3, count=1000, a fresh N(0,1) '
                 'gradient array every step',
            dtype='bf16', n=1 << 28, eps=1e-3, eps_root=0.0, count=1000, fresh_gradients=True,
            operator_preheat=100),
    8: dict(name='config8: multi-tensor forward_ in place over 64 float32 leaves of 4096 x 1024 '
                 '(16 MiB each, the GPT-2-medium fc weight), the gradient, mu and nu lists each '
                 'contiguous, so the three arrays of every leaf lie exactly 1 GiB = 64 x 16 MiB '
                 'apart and meet in the same DRAM banks; count=1',
            dtype='f32', shapes=[(4096, 1024)] * 64, eps_root=0.0, count=1,
            lists_contiguous=True, operator_preheat=60),
    9: dict(name='config9: classic optimizer step (Adam + scale(-lr) + apply) in one pass over the '
                 'GPT-2-medium parameter list in bfloat16 (parameters, gradients and both moments), '
                 'eps=1e-3, count=1; beside it the three-pass chain',
            dtype='bf16', shapes=gpt2_medium_shapes(), eps=1e-3, eps_root=0.0, count=1,
            fused_step=True, operator_preheat=100),
}
ESIZE = {'f32': 4, 'f64': 8, 'f16': 2, 'bf16': 2}


# ----------------------------------------------------------------------------- GPU side


_HOST = {}  # (config, tensor index) -> the seeded host arrays, shared by the GPU and CPU legs


def host_state(cfg_id, index, n, tag, extra=0):
    """The seeded host arrays of one tensor, as torch CPU tensors: updates ~ N(0,1),
    mu = 0.1 N(0,1), nu = |0.01 N(0,1)| and `extra` more N(0,1) arrays, drawn in that order from
    torch's CPU generator with seed 1000 * config + tensor index.  float64 for 'f64', float32
    otherwise; the 16-bit types are rounded from the float32 draws."""
    import torch

    key = (cfg_id, index, n, tag, extra)
    if key not in _HOST:
        g = torch.Generator(device='cpu')
        g.manual_seed(1000 * cfg_id + index)
        wide = torch.float64 if tag == 'f64' else torch.float32
        arrays = [torch.randn(n, generator=g, dtype=wide),
                  torch.randn(n, generator=g, dtype=wide).mul_(0.1),
                  torch.randn(n, generator=g, dtype=wide).mul_(0.01).abs_()]
        arrays += [torch.randn(n, generator=g, dtype=wide) for _ in range(extra)]
        narrow = {'f16': torch.float16, 'bf16': torch.bfloat16}.get(tag)
        if narrow is not None:
            arrays = [a.to(narrow) for a in arrays]
        _HOST[key] = arrays
    return _HOST[key]


def preheat(torch, launches=120):
    """GPU clocks ramp for the first ~15 ms of sustained load in a cold process (the state was
    just generated on the host and uploaded, so the GPU has been idle): stream through scratch
    arrays -- never the benchmark's own state, and with PyTorch's own kernels, so that a kernel
    trace of the run holds the operator's kernels for the benchmark's steps only -- for ~40 ms
    before the warm-up steps."""
    a = torch.rand(1 << 27, device='cuda')
    b = torch.rand(1 << 27, device='cuda')
    for _ in range(launches):
        a.add_(b)
    torch.cuda.synchronize()
    return launches


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

    from torchopt_amd import MultiAdamOp

    base = wall_ms(loss_alone)
    out = {'python_update_plus_backward_ms': round(wall_ms(fused) - base, 5),
           'python_update_alone_ms': round(wall_ms(
               lambda: transform.update(grads, state, inplace=False)), 5),
           'python_loss_and_its_backward_alone_ms': round(base, 5)}
    # the same tree-level autograd node written in Python (the route `torch.compile` traces)
    MultiAdamOp.use_native_node = False
    try:
        out['python_update_plus_backward_ms_with_the_node_in_python'] = round(
            wall_ms(fused) - base, 5)
    finally:
        MultiAdamOp.use_native_node = True
    out['python_per_leaf_tensor_expressions_ms'] = round(wall_ms(per_leaf_expressions) - base, 5)
    return out


def time_backward_ops(torch, lib, cfg_id, code, dtype, tag, n, esize, eps_root, count, stream,
                      reps=20):
    """backward_mu, backward_nu, backward_updates and the one-pass backward_all on flat arrays of
    n elements: ms per launch and achieved GB/s (algorithmic bytes: 3, 4, 5 and 9 arrays).  The
    inputs are what a differentiable step produces from the configuration's seeded state
    (updates, new_mu, new_updates) and three seeded N(0,1) arrays as incoming gradients."""
    g, mu, nu, d_mu, d_nu, d_u = (a.cuda() for a in host_state(cfg_id, 0, n, tag, extra=3))
    new_mu, new_nu, new_u = (torch.empty_like(g) for _ in range(3))
    s = stream.cuda_stream
    rc = lib.toa_adam_forward_all(code, g.data_ptr(), mu.data_ptr(), nu.data_ptr(), n, B1, B2, EPS,
                                  eps_root, count, new_mu.data_ptr(), new_nu.data_ptr(),
                                  new_u.data_ptr(), s)
    if rc:
        raise RuntimeError(f'forward_all: {lib.toa_adam_error_string(rc).decode()}')
    del mu, nu, new_nu
    out = [torch.empty_like(g) for _ in range(3)]
    o = [t.data_ptr() for t in out]
    ops = {
        'backward_mu': (3, lambda: lib.toa_adam_backward_mu(code, d_mu.data_ptr(), n, B1, o[0],
                                                            o[1], s)),
        'backward_nu': (4, lambda: lib.toa_adam_backward_nu(code, d_nu.data_ptr(), g.data_ptr(), n,
                                                            B2, o[0], o[1], s)),
        'backward_updates': (5, lambda: lib.toa_adam_backward_updates(
            code, d_u.data_ptr(), new_u.data_ptr(), new_mu.data_ptr(), n, B1, B2, eps_root, count,
            o[0], o[1], s)),
        'backward_all': (9, lambda: lib.toa_adam_backward_all(
            code, d_u.data_ptr(), new_u.data_ptr(), new_mu.data_ptr(), g.data_ptr(),
            d_mu.data_ptr(), d_nu.data_ptr(), n, B1, B2, eps_root, count, o[0], o[1], o[2], s)),
    }
    res = {}
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
        res[name] = {'ms': round(ms, 5), 'GB/s': round(streams * esize * n / ms / 1e6, 1)}
    return res


def timed_region(torch, step, stream, warmup, steps, before_warmup=None, before_timed=None):
    """`warmup` untimed steps, then exactly `steps` steps between two device synchronisations:
    (wall-clock ms per step, stream ms per step from events around the same steps).  The two
    hooks run on the host just before the warm-up steps and, after the first synchronisation,
    just before the clock starts (they may enqueue work on OTHER streams)."""
    if before_warmup is not None:
        before_warmup()
    for _ in range(warmup):
        step()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    if before_timed is not None:
        before_timed()
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(steps):
        step()
    ev1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, ev0.elapsed_time(ev1) / steps


def sysfs_gpu_state():
    """What the driver says about the first GPU right now: the current shader and memory clock
    levels (the starred lines of pp_dpm_sclk / pp_dpm_mclk) and the socket power.  Read while
    work is queued on the GPU, these describe the state the timings were taken in.  Empty where
    the files are not readable."""
    import glob

    out = {}
    for dev in sorted(glob.glob('/sys/class/drm/card*/device')):
        if not os.path.exists(os.path.join(dev, 'pp_dpm_sclk')):
            continue
        for key, name in (('sclk', 'pp_dpm_sclk'), ('mclk', 'pp_dpm_mclk')):
            try:
                with open(os.path.join(dev, name)) as f:
                    for line in f:
                        if line.rstrip().endswith('*'):
                            out[f'{key}_MHz'] = int(''.join(c for c in line.split(':')[1]
                                                            if c.isdigit()))
            except (OSError, ValueError, IndexError):
                pass
        for path in glob.glob(os.path.join(dev, 'hwmon', '*', 'power1_input')):
            try:
                with open(path) as f:
                    out['power_W'] = round(int(f.read()) / 1e6, 1)
            except (OSError, ValueError):
                pass
        break
    return out


class ClockProbe:
    """Shader-clock evidence beside a timing: the library's one-lane spin kernel
    (toa_adam_clock_probe) reports shader-clock ticks and constant-rate (100 MHz) ticks for a
    fixed spin; their ratio is the shader clock the wave ran at."""

    SPINS = 20000  # ~60 us at 2.4 GHz: long against the counters' granularity, short in a stream

    def __init__(self, torch, lib, slots=16):  # noqa: D107
        self.torch, self.lib = torch, lib
        self.buf = torch.zeros(slots, 3, dtype=torch.int64, device='cuda')
        self.names = []

    def sample(self, name, stream, spins=None):
        k = len(self.names)
        if k >= self.buf.shape[0]:
            return
        rc = self.lib.toa_adam_clock_probe(self.buf[k].data_ptr(), spins or self.SPINS,
                                           stream.cuda_stream)
        if rc:
            raise RuntimeError(self.lib.toa_adam_error_string(rc).decode())
        self.names.append((name, spins or self.SPINS))

    def chain(self, name, stream, count, spins):
        """`count` probes one after the other on `stream`: a time series of the shader clock."""
        for k in range(count):
            self.sample(f'{name}[{k}]', stream, spins)

    def read(self):
        host = self.buf.cpu().tolist()
        out = {}
        for (name, spins), (core, wall, _) in zip(self.names, host):
            out[name] = {'spins': spins, 'shader_clock_ticks': core, 'constant_100MHz_ticks': wall,
                         'shader_MHz': round(100.0 * core / wall, 1) if wall else None}
        return out

    def series(self, name):
        """(MHz of every probe of chain `name`, mean milliseconds a probe took)."""
        got = [v for k, v in self.read().items() if k.startswith(name + '[') and v['shader_MHz']]
        if not got:
            return [], None
        return ([round(v['shader_MHz']) for v in got],
                round(sum(v['constant_100MHz_ticks'] for v in got) / len(got) / 1e5, 3))


def in_situ(torch, step, stream, alg_bytes, iterations=50, busy_ms=5.0):
    """The operator where an optimizer runs it: ONE launch per iteration, after `busy_ms` of
    unrelated GPU work (a chain of matrix products on scratch tensors, as a backward pass would
    leave the caches, clocks and queues), events around the operator's launch alone."""
    a = torch.randn(4096, 4096, device='cuda')
    b = torch.randn(4096, 4096, device='cuda') / 64.0  # keeps the chain's values bounded
    for _ in range(3):
        torch.matmul(a, b)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(4):
        torch.matmul(a, b)
    e1.record(stream)
    torch.cuda.synchronize()
    one_ms = e0.elapsed_time(e1) / 4
    chain = max(1, int(busy_ms / one_ms + 0.999))
    pairs = []
    for _ in range(iterations + 5):
        x = a
        for _ in range(chain):
            x = torch.matmul(x, b)
        p, q = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        p.record(stream)
        step()
        q.record(stream)
        pairs.append((p, q))
    torch.cuda.synchronize()
    each = sorted(p.elapsed_time(q) for p, q in pairs[5:])
    med = each[len(each) // 2]
    return {'iterations': len(each), 'other_work_ms_per_iteration': round(chain * one_ms, 3),
            'other_work': f'{chain} float32 matrix products of 4096 x 4096 on scratch tensors',
            'operator_ms_median': round(med, 5), 'operator_ms_min': round(each[0], 5),
            'operator_ms_max': round(each[-1], 5),
            'GB/s_median': round(alg_bytes / med / 1e6, 1),
            'frac_median': round(alg_bytes / med / 1e6 / HBM_PEAK_GBS, 4),
            'frac_min_time': round(alg_bytes / each[0] / 1e6 / HBM_PEAK_GBS, 4)}


def run_gpu(cfg_id, steps, warmup, operator_preheat=None, state='init'):
    import torch

    from torchopt_amd import _lib
    from torchopt_amd.placement import state_zeros_like_tree

    def moments(host_mu, host_nu, like):
        """The two moment arrays on the GPU: allocated the way the package's own init allocates
        the state of a one-leaf tree (--state init: one block, the first moment 8 KiB past a
        multiple of 16 KiB, the second at one, a whole even number of MiB plus those 8 KiB apart
        modulo 16 MiB), each in a block of its own at its phase (--state separate), or wherever
        torch's allocator puts them (--state plain)."""
        if state == 'plain':
            return host_mu.cuda(), host_nu.cuda()
        if state == 'separate':
            from torchopt_amd.placement import state_empty_like
            return (state_empty_like(like, moment=0).copy_(host_mu),
                    state_empty_like(like, moment=1).copy_(host_nu))
        (mu,), (nu,) = state_zeros_like_tree([like])
        return mu.copy_(host_mu), nu.copy_(host_nu)

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
        host = [host_state(cfg_id, k, n, cfg['dtype'], extra=3) for k, n in enumerate(sizes)]

        def arr(ts):
            return (ctypes.c_void_p * num)(*[t.data_ptr() for t in ts])

        ups, mus, nus, d_m, d_v, d_u = ([h[j].cuda() for h in host] for j in range(6))
        # new_mu, new_nu, new_u, 2 x 3 backward outputs
        outs = [[torch.empty(n, device='cuda', dtype=dtype) for n in sizes] for _ in range(9)]
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
        extra_arrays = 1 if cfg.get('fused_step') else 0
        host = [host_state(cfg_id, k, n, cfg['dtype'], extra=extra_arrays)
                for k, n in enumerate(sizes)]
        num = len(sizes)
        ns = (ctypes.c_size_t * num)(*sizes)
        extra = {'tensors': num}

        def carve(gap_elems):
            """The three lists carved from one allocation, each list contiguous, the lists
            `gap_elems` elements further apart than their own length."""
            arena = torch.empty(3 * total + 2 * gap_elems, device='cuda', dtype=dtype)
            lists = []
            for j in range(3):
                at, views = j * (total + gap_elems), []
                for h, n in zip(host, sizes):
                    views.append(arena[at:at + n])
                    views[-1].copy_(h[j])
                    at += n
                lists.append(views)
            return lists

        def list_step(us_, ms_, vs_):
            a, b, c = ((ctypes.c_void_p * num)(*[t.data_ptr() for t in ts])
                       for ts in (us_, ms_, vs_))

            def one():
                rc = lib.toa_adam_forward_inplace_multi(code, num, a, b, c, ns, B1, B2, eps,
                                                        eps_root, None, count, sptr)
                if rc:
                    raise RuntimeError(lib.toa_adam_error_string(rc).decode())
            return one

        if cfg.get('lists_contiguous'):
            # beside the timed layout: the same lists 3 MiB further apart, where no leaf's arrays
            # meet in the same banks -- what the colliding placement costs
            apart = carve((3 << 20) // esize)
            other = list_step(*apart)
            for _ in range(60):  # past the operator's start-up transient (see the preheat below)
                other()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for _ in range(20):
                other()
            b.record(stream)
            torch.cuda.synchronize()
            apart_ms = a.elapsed_time(b) / 20
            extra['lists_3_mib_further_apart'] = {
                'ms_per_step': round(apart_ms, 5),
                'GB/s': round(bytes_per_elem * total / apart_ms / 1e6, 1)}
            del apart, other
            us, ms, vs = carve(0)
        else:
            us = [h[0].cuda() for h in host]
            if state == 'plain':
                ms = [h[1].cuda() for h in host]
                vs = [h[2].cuda() for h in host]
            elif state == 'separate':
                from torchopt_amd.placement import state_empty_like

                ms = [state_empty_like(u, moment=0).copy_(h[1]) for h, u in zip(host, us)]
                vs = [state_empty_like(u, moment=1).copy_(h[2]) for h, u in zip(host, us)]
            else:  # as the package's init allocates the moments of a tree
                ms, vs = state_zeros_like_tree(us)
                for h, m, v in zip(host, ms, vs):
                    m.copy_(h[1])
                    v.copy_(h[2])
            extra['state_allocation'] = state
        step = list_step(us, ms, vs)
        pu, pm, pv = ((ctypes.c_void_p * num)(*[t.data_ptr() for t in ts]) for ts in (us, ms, vs))
        if cfg.get('fused_step'):
            ps = [h[3].cuda() for h in host]
            pp = (ctypes.c_void_p * num)(*[t.data_ptr() for t in ps])
            lr = 1e-3

            # The reference's three passes, PyTorch's list kernels for two of them.  forward_
            # leaves the scaled update where the gradient was, so every chain step starts from the
            # pristine gradients again (restored outside the clock: a training loop brings new
            # gradients every step, and re-feeding a step its own output drives the data to
            # values no run holds).
            pristine = [u.clone() for u in us]
            pairs = []
            for k in range(steps + 3):
                torch._foreach_copy_(us, pristine)
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                step()
                torch._foreach_mul_(us, -lr)
                torch._foreach_add_(ps, us)
                b.record(stream)
                if k >= 3:
                    pairs.append((a, b))
            torch.cuda.synchronize()
            chain_ms = sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)
            torch._foreach_copy_(us, pristine)
            del pristine, pairs

            def step():  # noqa: F811
                rc = lib.toa_adam_fused_step_multi(code, num, pp, pu, pm, pv, ns, B1, B2, eps,
                                                   eps_root, None, count, lr, 0.0, 0, 0, 0, sptr)
                if rc:
                    raise RuntimeError(lib.toa_adam_error_string(rc).decode())
            bytes_per_elem = 7 * esize  # reads g, mu, nu, p; writes mu, nu, p
            extra.update(three_pass_chain_ms_per_step=round(chain_ms, 5),
                         three_pass_chain_bytes_per_element=11 * esize)
    else:
        total = cfg['n']
        h_u, h_mu, h_nu = host_state(cfg_id, 0, total, cfg['dtype'])
        u = h_u.cuda()
        mu, nu = moments(h_mu, h_nu, u)
        pu, pm, pv = u.data_ptr(), mu.data_ptr(), nu.data_ptr()

        extra = {'state_allocation': state,
                 'address_mod_16KiB': {'updates': pu % 16384, 'mu': pm % 16384, 'nu': pv % 16384}}
        if cfg.get('fresh_gradients'):
            # A training loop hands the step a new gradient every time.  The step overwrites its
            # gradient array with the update, so an array used twice feeds the operator its own
            # output: over a few dozen steps that drifts the data away from anything a real run
            # holds, and the 16-bit kernels' data-dependent quick route with it (measured: the same
            # loop slows by up to 20 % after 150 steps over eight arrays in rotation, and holds
            # its speed when every step reads a fresh array).  So every step of this run --
            # warm-up, timed region and the per-step spread pass -- gets an array of its own,
            # drawn N(0, 1) before the clock starts; only a run longer than kMaxGradientArrays
            # steps wraps around.
            kMaxGradientArrays = 160  # 80 GiB of 16-bit gradients at most
            g = torch.Generator(device='cuda')
            g.manual_seed(1000 * cfg_id + 1)
            fresh = [torch.randn(total, device='cuda', generator=g).to(dtype)
                     for _ in range(min(steps + warmup + min(steps, 20), kMaxGradientArrays))]
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
            extra['backward_ops'] = time_backward_ops(torch, lib, cfg_id, code, dtype,
                                                      cfg['dtype'], total, esize, eps_root, count,
                                                      stream)
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

    extra['preheat_launches_on_scratch_arrays'] = preheat(torch)
    alg_bytes = bytes_per_elem * total
    beside = {}  # measurements taken beside the headline, in this process

    def leg(wall_ms, kern_ms, **more):
        return {'ms_per_step_wall': round(wall_ms, 5), 'kernel_ms': round(kern_ms, 5),
                'frac': round(alg_bytes / kern_ms / 1e6 / HBM_PEAK_GBS, 4),
                'frac_by_wall_clock': round(alg_bytes / wall_ms / 1e6 / HBM_PEAK_GBS, 4), **more}

    # The first launches of the operator in a process are not its steady state, whatever ran
    # before: launches 1-2 run at the steady rate, launches 4-8 up to 4 % slower (float32 in place:
    # 0.948, 0.953, 0.960 ... 0.985 ms), and the time settles back over the next 15 (float32) to
    # 45 (16-bit types) launches -- the clocks boost and settle under this kernel's own mix of
    # arithmetic and traffic (the clock probes below show the shader clock on either side of the
    # timed region).  Isolated steps on the initial and on a late state take the same time, so it
    # is not the data.  The bandwidth-bound configurations therefore run the operator before the
    # warm-up steps, and the line says how often and on what:
    #   * float32 / float64 single tensors: on the timed arrays themselves, as the first steps of
    #     a training run would (the library also settles its choice of load order for this call
    #     site during its first 30 launches); what the same W + K steps read WITHOUT any of that
    #     is measured first and reported as `cold_start`;
    #   * the 16-bit single tensors and the lists: on scratch state of the same shape (the 16-bit
    #     step's speed depends on its data, which a step fed its own output drifts away from);
    #   * a fused step, which only reads its gradients, on its own lists.
    # --operator-preheat 0 switches it off.
    op_launches = cfg.get('operator_preheat', 0) if operator_preheat is None else operator_preheat
    single_wide = ('shapes' not in cfg and not cfg.get('fresh_gradients')
                   and not alg_small(total * esize))
    if single_wide:
        # beside these first launches a chain of clock probes runs on a second stream (one wave,
        # ~0.5 ms a probe): the shader clock through the operator's start-up transient
        series = ClockProbe(torch, lib, slots=128)
        side = torch.cuda.Stream()
        per_probe_spins = 30000
        est_ms = bytes_per_elem * total / 6.8e9  # one step at 6.8 TB/s
        was = lib.toa_adam_set_tuning(0)
        cold = timed_region(
            torch, step, stream, warmup, steps,
            # (the chains end before the steps they accompany do: the region's synchronisation
            # must wait for the steps, not for the probes)
            before_warmup=lambda: series.chain('warmup', side, min(40, int(1.4 * est_ms * warmup)),
                                               per_probe_spins),
            before_timed=lambda: series.chain('timed', side, min(80, int(1.4 * est_ms * steps)),
                                              per_probe_spins))
        lib.toa_adam_set_tuning(was)
        torch.cuda.synchronize()
        mhz_w, ms_w = series.series('warmup')
        mhz_t, ms_t = series.series('timed')
        beside['cold_start'] = leg(*cold, note=(
            f'{warmup} + {steps} steps straight after upload and the PyTorch-kernel preheat: no '
            'launch of the operator before them, load-order tuning off (order 0 throughout)'),
            shader_MHz_beside_the_warmup_steps=mhz_w, shader_MHz_beside_the_timed_steps=mhz_t,
            ms_per_clock_probe=ms_t or ms_w)
        del series, side
    if op_launches and single_wide:
        for _ in range(op_launches):
            step()
        torch.cuda.synchronize()
        extra['preheat_operator_launches_on_the_timed_arrays'] = op_launches
        extra['load_order_kept_for_this_call_site'] = lib.toa_adam_tuned_load_order(
            code, pu, pm, pv, total)
    elif op_launches and cfg.get('fused_step'):
        for _ in range(op_launches):
            step()
        torch.cuda.synchronize()
        extra['preheat_operator_launches'] = op_launches
    elif op_launches and 'shapes' in cfg and not cfg.get('differentiable'):
        scratch = [[torch.randn(n, device='cuda').mul_(scale).abs_().to(dtype) for n in sizes]
                   for scale in (1.0, 0.1, 0.01)]
        scratch_step = list_step(*scratch)
        for _ in range(op_launches):
            scratch_step()
        torch.cuda.synchronize()
        del scratch, scratch_step
        extra['preheat_operator_launches_on_scratch_state'] = op_launches
    elif op_launches and 'shapes' not in cfg:
        sg = [torch.randn(total, device='cuda').to(dtype) for _ in range(4)]
        sm = (torch.randn(total, device='cuda') * 0.1).to(dtype)
        sv = (torch.randn(total, device='cuda') * 0.01).abs_().to(dtype)
        for k in range(op_launches):
            rc = lib.toa_adam_forward_inplace(code, sg[k % 4].data_ptr(), sm.data_ptr(),
                                              sv.data_ptr(), total, B1, B2, eps, eps_root, count,
                                              sptr)
            if rc:
                raise RuntimeError(lib.toa_adam_error_string(rc).decode())
        torch.cuda.synchronize()
        del sg, sm, sv
        extra['preheat_operator_launches_on_scratch_state'] = op_launches

    # ---- the headline: W warm-up steps, a clock probe, exactly K timed steps, a clock probe
    bandwidth_bound = not alg_small(total * esize) and not cfg.get('differentiable')
    probes = ClockProbe(torch, lib)
    for _ in range(warmup):
        step()
    if bandwidth_bound:
        probes.sample('before_the_timed_region', stream)
    wall_ms, kern_ms = timed_region(torch, step, stream, 0, steps)
    if bandwidth_bound:
        probes.sample('after_the_timed_region', stream)
        torch.cuda.synchronize()

    # per-step spread, from a second short pass with one pair of events per step (outside the
    # timed region; event overhead makes it meaningless for microsecond steps).  While those steps
    # are queued the driver's view of the GPU is read, and a long clock probe runs beside them on
    # a second stream: the clock state INSIDE a region of the same work.
    spread = {}
    if wall_ms > 0.05:
        reps = min(steps, 20)
        beside_probes = None
        if bandwidth_bound:
            beside_probes = ClockProbe(torch, lib, slots=64)
            side = torch.cuda.Stream()
            beside_probes.chain('beside', side, min(60, int(2 * reps * kern_ms) + 2), 30000)
        pairs = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            step()
            b.record(stream)
            pairs.append((a, b))
        busy_state = sysfs_gpu_state() if bandwidth_bound else {}
        torch.cuda.synchronize()
        each = sorted(a.elapsed_time(b) for a, b in pairs)
        spread = {'step_ms_min': round(each[0], 5), 'step_ms_median': round(each[len(each) // 2], 5),
                  'step_ms_max': round(each[-1], 5)}
        if bandwidth_bound:
            mhz, probe_ms = beside_probes.series('beside')
            beside['clock'] = {
                'probes': probes.read(),
                'shader_MHz_beside_the_per_step_pass': mhz, 'ms_per_clock_probe': probe_ms,
                'probe': 'toa_adam_clock_probe: one lane, a fixed spin of dependent integer '
                         'multiply-adds; shader-clock ticks against ticks of the constant 100 MHz '
                         'counter.  before / after: on the timed stream, either side of the timed '
                         'region (the GPU otherwise idle: the boost clock); beside: a chain of '
                         'probes on a second stream while 20 further steps of the same work run '
                         '(those that start after the steps have ended read the boost clock again)',
                'driver_while_steps_are_queued': busy_state}

    # ---- the same W + K steps with the moments where the ALLOCATOR puts them (what a caller
    # gets whose state comes from zeros_like, as through the reference's own init)
    if single_wide and state != 'plain':
        p_mu, p_nu = h_mu.cuda(), h_nu.cuda()

        def plain_step():
            rc = lib.toa_adam_forward_inplace(code, pu, p_mu.data_ptr(), p_nu.data_ptr(), total,
                                              B1, B2, eps, eps_root, count, sptr)
            if rc:
                raise RuntimeError(lib.toa_adam_error_string(rc).decode())
        for _ in range(op_launches):
            plain_step()
        torch.cuda.synchronize()
        beside['state_where_the_allocator_puts_it'] = leg(
            *timed_region(torch, plain_step, stream, warmup, steps),
            address_mod_16KiB={'updates': pu % 16384, 'mu': p_mu.data_ptr() % 16384,
                               'nu': p_nu.data_ptr() % 16384},
            load_order_kept=lib.toa_adam_tuned_load_order(code, pu, p_mu.data_ptr(),
                                                          p_nu.data_ptr(), total),
            note=f'{op_launches} launches on these arrays first, then {warmup} + {steps} steps')
        del p_mu, p_nu

    # ---- one launch per iteration between other kernels
    if bandwidth_bound:
        beside['one_launch_per_iteration_between_other_work'] = in_situ(torch, step, stream,
                                                                        alg_bytes)

    achieved = alg_bytes / (kern_ms * 1e-3) / 1e9
    traffic, traffic_source = RECORDED_TRAFFIC.get(cfg_id, (None, None))
    return {
        'elements': total,
        'ms_per_step': wall_ms,
        'value': total / (wall_ms * 1e-3),
        'roofline': {
            'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
            'frac': round(achieved / HBM_PEAK_GBS, 4), 'traffic': traffic,
            'traffic_source': (f'recorded in {traffic_source} (rocprofv3 --pmc), not measured in '
                               'this run' if traffic_source else None),
            'kernel_ms': round(kern_ms, 5), 'algorithmic_bytes_per_launch': alg_bytes,
            'bytes_per_element': bytes_per_elem,
            'frac_by_wall_clock': round(alg_bytes / wall_ms / 1e6 / HBM_PEAK_GBS, 4), **spread,
        },
        'extra': extra,
        'beside': beside,
        'device': torch.cuda.get_device_name(0),
    }


# ----------------------------------------------------------------------------- CPU baseline


def host_cores():
    """The CPUs this process may run on, cut to the box's CPU share (OMP_NUM_THREADS, 16 where it
    is unset) -- not every core the machine shows.  The reference's op asks the OpenMP runtime
    for the number of processors, which is the size of the affinity mask the runtime saw when it
    loaded, so `main()` calls this before anything imports torch."""
    global _HOST_CORES
    if _HOST_CORES is None:  # once: an OpenMP runtime with OMP_PROC_BIND set pins this thread later
        share = int(os.environ.get('OMP_NUM_THREADS', '16') or 16)
        try:
            avail = sorted(os.sched_getaffinity(0))
            if len(avail) > share:
                os.sched_setaffinity(0, set(avail[:share]))
                avail = avail[:share]
            _HOST_CORES = max(1, len(avail))
        except (AttributeError, OSError):
            _HOST_CORES = max(1, min(share, os.cpu_count() or 1))
    return _HOST_CORES


_HOST_CORES = None


CPU_SAMPLE_ELEMS = 1 << 28  # most elements the CPU leg works on: all of config 2 (3 x 1 GiB)


def cpu_model():
    try:
        with open('/proc/cpuinfo') as f:
            for line in f:
                if line.startswith('model name'):
                    return line.split(':', 1)[1].strip()
    except OSError:
        pass
    return 'unknown'


class CpuOps:
    """The seven CPU ops on torch CPU tensors: the reference's own compiled CPU op where
    oracle/_ref holds it (kind 'reference'), this repository's C restatement of it otherwise
    (kind 'port').  Only this leg of the benchmark touches `oracle/`."""

    def __init__(self):
        from oracle import adam_oracle

        self.port = adam_oracle
        self.ref = None
        try:
            self.ref = adam_oracle.load_reference()
        except Exception as exc:  # noqa: BLE001
            print(f'[bench] compiled reference not usable ({exc}); timing the C port',
                  file=sys.stderr)
        self.kind = 'reference' if self.ref is not None else 'port'

    def _np(self, t):
        import torch

        if t.dtype == torch.bfloat16:  # bfloat16 travels as uint16 bit patterns on the NumPy side
            import numpy as np

            return t.view(torch.int16).numpy().view(np.uint16)
        return t.numpy()

    def _t(self, a, like):
        import numpy as np
        import torch

        if like.dtype == torch.bfloat16:
            return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
        return torch.from_numpy(a)

    def forward_(self, u, m, v, eps, eps_root, count):
        if self.ref is not None:
            self.ref.adam_op.forward_(u, m, v, B1, B2, eps, eps_root, count)
        else:
            self.port.forward_inplace(self._np(u), self._np(m), self._np(v), B1, B2, eps, eps_root,
                                      count)

    def forward_mu(self, u, m):
        if self.ref is not None:
            return self.ref.adam_op.forward_mu(u, m, B1)
        return self._t(self.port.forward_mu(self._np(u), self._np(m), B1), u)

    def forward_nu(self, u, v):
        if self.ref is not None:
            return self.ref.adam_op.forward_nu(u, v, B2)
        return self._t(self.port.forward_nu(self._np(u), self._np(v), B2), u)

    def forward_updates(self, m, v, eps, eps_root, count):
        if self.ref is not None:
            return self.ref.adam_op.forward_updates(m, v, B1, B2, eps, eps_root, count)
        return self._t(self.port.forward_updates(self._np(m), self._np(v), B1, B2, eps, eps_root,
                                                 count), m)

    def backward_mu(self, d, u, m):
        if self.ref is not None:
            return self.ref.adam_op.backward_mu(d, u, m, B1)
        return [self._t(a, d) for a in self.port.backward_mu(self._np(d), B1)]

    def backward_nu(self, d, u, v):
        if self.ref is not None:
            return self.ref.adam_op.backward_nu(d, u, v, B2)
        return [self._t(a, d) for a in self.port.backward_nu(self._np(d), self._np(u), B2)]

    def backward_updates(self, d, u, m, v, eps_root, count):
        if self.ref is not None:
            return self.ref.adam_op.backward_updates(d, u, m, v, B1, B2, eps_root, count)
        return [self._t(a, d) for a in self.port.backward_updates(
            self._np(d), self._np(u), self._np(m), B1, B2, eps_root, count)]


def ulp_report(pairs, chunk=1 << 24):
    """(GPU tensor, CPU tensor) pairs -> elements checked, elements that differ, largest distance
    in units in the last place (NaNs of any payload count as equal).  Works through the arrays
    in pieces, so whole configurations can be compared without holding 64-bit copies of them."""
    import numpy as np
    import torch

    checked = differing = worst = 0
    for got, want in pairs:
        got = got.detach().cpu().contiguous().view(-1)
        want = want.contiguous().view(-1)
        size = got.element_size()
        bits = {2: torch.int16, 4: torch.int32, 8: torch.int64}[size]
        lo = int(np.iinfo({2: np.int16, 4: np.int32, 8: np.int64}[size]).min)
        for at in range(0, got.numel(), chunk):
            g, w = got[at:at + chunk], want[at:at + chunk]
            if torch.equal(g.view(bits), w.view(bits)):  # the usual case: the same bits
                checked += g.numel()
                continue
            nan = torch.isnan(g.float() if size == 2 else g) & torch.isnan(
                w.float() if size == 2 else w)
            a = g.view(bits).numpy().astype(np.int64)
            b = w.view(bits).numpy().astype(np.int64)
            a, b = np.where(a < 0, lo - a, a), np.where(b < 0, lo - b, b)  # monotone integer line
            d = np.abs(a - b)
            d[nan.numpy()] = 0
            checked += d.size
            differing += int(np.count_nonzero(d))
            worst = max(worst, int(d.max(initial=0)))
    return {'elements_checked': checked, 'differing': differing, 'max_ulp': worst}


def run_cpu_baseline(cfg_id, budget_s=12.0):
    """The CPU ops the configuration names, timed on the host's cores on a bounded sample of the
    same seeded inputs the GPU leg uses (untiled: every element its own draw), and the parity of
    the GPU's results with the CPU's on that sample.

    Only this leg touches `oracle/`; it is the reported baseline, never the measured product.
    """
    import ctypes

    import torch

    from torchopt_amd import _lib

    cfg = CONFIGS[cfg_id]
    tag = cfg['dtype']
    eps = cfg.get('eps', EPS)
    eps_root, count = cfg['eps_root'], cfg['count']
    esize = ESIZE[tag]
    lib = _lib.load()
    code = {'f32': _lib.TOA_F32, 'f64': _lib.TOA_F64, 'f16': _lib.TOA_F16,
            'bf16': _lib.TOA_BF16}[tag]
    sptr = torch.cuda.current_stream().cuda_stream

    cores = host_cores()
    torch.set_num_threads(cores)
    cpu = CpuOps()

    def check(rc):
        if rc:
            raise RuntimeError(lib.toa_adam_error_string(rc).decode())

    # ---- the leaves of the sample: seeded host arrays, cloned (the GPU leg owns the originals)
    if 'shapes' in cfg:
        sizes = [numel(x) for x in cfg['shapes']]
        extra = 3 if cfg.get('differentiable') else (1 if cfg.get('fused_step') else 0)
        leaves, taken = [], 0
        for k, n in enumerate(sizes):
            if taken + n > CPU_SAMPLE_ELEMS and leaves:
                break
            leaves.append([a.clone() for a in host_state(cfg_id, k, n, tag, extra=extra)])
            taken += n
        full = sum(sizes)
        what = (f'the first {len(leaves)} of {len(sizes)} tensors ({taken} of {full} elements)'
                if taken < full else
                f'all: the whole configuration, {len(sizes)} tensors, {full} elements')
    else:
        full = cfg['n']
        n = min(full, CPU_SAMPLE_ELEMS)
        extra = 3 if cfg.get('backward') else 0
        leaves = [[a[:n].clone() for a in host_state(cfg_id, 0, full, tag, extra=extra)]]
        taken = n
        what = (f'the first {n} of {full} elements' if n < full
                else f'all: the whole configuration, {full} elements')
    dev = [[a.cuda() for a in leaf] for leaf in leaves]
    num = len(leaves)

    def col(j):
        return (ctypes.c_void_p * num)(*[leaf[j].data_ptr() for leaf in dev])

    ns = (ctypes.c_size_t * num)(*[leaf[0].numel() for leaf in leaves])

    # ---- one pass of the configuration's ops on the CPU; the first pass doubles as warm-up
    # (threads, page faults) and as the reference for the parity check
    if cfg.get('differentiable'):
        ops = 'forward_mu, forward_nu, forward_updates, backward_updates, backward_nu, backward_mu, leaf by leaf'
        bytes_per_elem = 21 * esize  # 3 + 3 + 3 arrays forward, 5 + 4 + 3 backward

        def one():
            outs = []
            for g, m, v, d_m, d_v, d_u in leaves:
                new_m, new_v = cpu.forward_mu(g, m), cpu.forward_nu(g, v)
                new_u = cpu.forward_updates(new_m, new_v, eps, eps_root, count)
                bm, bv = cpu.backward_updates(d_u, new_u, new_m, new_v, eps_root, count)
                outs.append((new_m, new_v, new_u, bm, bv, *cpu.backward_nu(d_v, g, v),
                             *cpu.backward_mu(d_m, g, m)))
            return outs

        want = one()
        o = [[torch.empty_like(leaf[0]) for leaf in dev] for _ in range(9)]
        oc = [(ctypes.c_void_p * num)(*[t.data_ptr() for t in x]) for x in o]
        check(lib.toa_adam_forward_mu_multi(code, num, col(0), col(1), ns, B1, oc[0], sptr))
        check(lib.toa_adam_forward_nu_multi(code, num, col(0), col(2), ns, B2, oc[1], sptr))
        check(lib.toa_adam_forward_updates_multi(code, num, oc[0], oc[1], ns, B1, B2, eps, eps_root,
                                                 None, count, oc[2], sptr))
        check(lib.toa_adam_backward_updates_multi(code, num, col(5), oc[2], oc[0], ns, B1, B2,
                                                  eps_root, None, count, oc[3], oc[4], sptr))
        check(lib.toa_adam_backward_nu_multi(code, num, col(4), col(0), ns, B2, oc[5], oc[6], sptr))
        check(lib.toa_adam_backward_mu_multi(code, num, col(3), ns, B1, oc[7], oc[8], sptr))
        pairs = [(o[j][k], want[k][j]) for k in range(num) for j in range(9)]
    elif cfg.get('backward'):
        ops = 'forward_ in place, then backward_mu, backward_nu, backward_updates'
        bytes_per_elem = (6 + 3 + 4 + 5) * esize
        g0, m0, v0, d_m, d_v, d_u = leaves[0]
        gw, mw, vw = g0.clone(), m0.clone(), v0.clone()  # forward_ overwrites these, pass after pass

        def one():
            cpu.forward_(gw, mw, vw, eps, eps_root, count)  # gw: the update, mw / vw: new moments
            return (gw, mw, vw, *cpu.backward_mu(d_m, g0, m0), *cpu.backward_nu(d_v, g0, v0),
                    *cpu.backward_updates(d_u, gw, mw, vw, eps_root, count))

        want = [t.clone() for t in one()]
        dg, dm, dv = (t.clone() for t in dev[0][:3])
        o = [torch.empty_like(dg) for _ in range(6)]
        p = [t.data_ptr() for t in o]
        check(lib.toa_adam_forward_inplace(code, dg.data_ptr(), dm.data_ptr(), dv.data_ptr(), taken,
                                           B1, B2, eps, eps_root, count, sptr))
        check(lib.toa_adam_backward_mu(code, dev[0][3].data_ptr(), taken, B1, p[0], p[1], sptr))
        check(lib.toa_adam_backward_nu(code, dev[0][4].data_ptr(), dev[0][0].data_ptr(), taken, B2,
                                       p[2], p[3], sptr))
        check(lib.toa_adam_backward_updates(code, dev[0][5].data_ptr(), dg.data_ptr(),
                                            dm.data_ptr(), taken, B1, B2, eps_root, count, p[4],
                                            p[5], sptr))
        pairs = list(zip((dg, dm, dv, *o), want))
    elif cfg.get('fused_step'):
        ops = 'forward_ in place, updates.mul_(-lr), params.add_(updates), leaf by leaf'
        bytes_per_elem = 11 * esize
        lr = 1e-3

        def one():
            for g, m, v, p in leaves:
                cpu.forward_(g, m, v, eps, eps_root, count)
                g.mul_(-lr)
                p.add_(g)

        one()
        check(lib.toa_adam_fused_step_multi(code, num, col(3), col(0), col(1), col(2), ns, B1, B2,
                                            eps, eps_root, None, count, lr, 0.0, 0, 0, 1, sptr))
        pairs = [(dev[k][j], leaves[k][j]) for k in range(num) for j in range(4)]
    else:
        ops = 'forward_ in place' + (', leaf by leaf' if num > 1 else '')
        bytes_per_elem = 6 * esize

        def one():
            for g, m, v in leaves:
                cpu.forward_(g, m, v, eps, eps_root, count)

        one()
        check(lib.toa_adam_forward_inplace_multi(code, num, col(0), col(1), col(2), ns, B1, B2,
                                                 eps, eps_root, None, count, sptr))
        pairs = [(dev[k][j], leaves[k][j]) for k in range(num) for j in range(3)]
    torch.cuda.synchronize()
    parity = ulp_report(pairs)
    del dev, pairs

    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 25):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {
        'value': taken / med, 'unit': 'elements/s', 'cores': cores, 'kind': cpu.kind,
        'sample': f'{what} ({tag}); {ops}; median of {len(times)} passes after 1 warm-up pass; '
                  'untiled seeded inputs, the ones the GPU leg uses',
        'gb_per_s': round(bytes_per_elem * taken / med / 1e9, 2),
        'bytes_per_element': bytes_per_elem,
        'cpu_model': cpu_model(),
        'threads_policy': 'min(n / 1000, cores) per op, as the reference sets it',
        'omp': {k: os.environ.get(k, 'unset') for k in ('OMP_NUM_THREADS', 'OMP_PROC_BIND',
                                                      'OMP_PLACES')},
        'note': 'host CPUs differ between GPU boxes (5e9 to 1e10 elements/s seen for config 2): '
                'compare only within one line',
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
    ap.add_argument('--state', choices=('init', 'separate', 'plain'), default='init',
                    help="how mu and nu are allocated: 'init' = as the package's init does "
                         '(torchopt_amd.state_zeros_like_tree: the moments of a tree in one block, '
                         'the two moments of a large leaf 8 KiB apart modulo 16 KiB), '
                         "'separate' = every moment in a block of its own at its phase "
                         "(state_zeros_like), 'plain' = torch's allocator alone")
    ap.add_argument('--operator-preheat', type=int, default=None,
                    help='launches of the operator on scratch state before the warm-up steps '
                         '(default: 100 for the 16-bit configurations, 60 for the other '
                         'bandwidth-bound ones, 0 for configs 0 and 1)')
    ap.add_argument('--pmc-calibration', action='store_true',
                    help='after the timed region also run 5 plain device copies of 1 GiB, so a '
                         'rocprofv3 --pmc run holds a kernel of known traffic to scale '
                         'FETCH_SIZE / WRITE_SIZE by')
    args = ap.parse_args(argv)

    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this build measures one GPU only (the op needs no exchange between '
              'GPUs; each would run the same kernel on its shard). Run with --gpus 1.',
              file=sys.stderr)
        return 2

    host_cores()  # before torch (and with it the OpenMP runtime) loads

    gpu = run_gpu(args.config, args.steps, args.warmup, args.operator_preheat, args.state)
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
        'data': 'synthetic (seeded CPU generator, seed = 1000 * config + tensor index, uploaded once)',
        'config': {'workload': cfg['name'], 'elements': gpu['elements'], 'b1': B1, 'b2': B2,
                   'eps': cfg.get('eps', EPS), 'eps_root': cfg['eps_root'], 'count': cfg['count'],
                   'device': gpu['device'], **gpu['extra']},
        'roofline': gpu['roofline'],
        'beside_the_headline': gpu['beside'],
    }
    if not args.no_cpu_baseline:
        line['cpu_baseline'] = run_cpu_baseline(args.config)
    _HOST.clear()
    print(json.dumps(line), flush=True)
    return 0


if __name__ == '__main__':
    sys.exit(main())
