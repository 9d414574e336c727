"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
public header declares, the ctypes table agrees with the header, argument errors come back as
codes before any device work, and the Python surface refuses what it cannot serve instead of
computing it somewhere else."""

from __future__ import annotations

import ctypes
import warnings
import os
import re

import pytest
import torch

from conftest import REPO
from torchopt_amd import AdamOp, _lib, accelerated_op_available
from torchopt_amd._C import adam_op

HEADER = os.path.join(REPO, 'include', 'toa_adam.h')


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    decls = re.findall(r'TOA_API\s+(?:const\s+char\s*\*|int|unsigned|size_t)\s*(\w+)\s*\(([^;]*?)\)\s*;', text,
                       flags=re.S)
    return {name: [a.strip() for a in args.split(',')] if args.strip() != 'void' else []
            for name, args in decls}


def test_header_declares_the_expected_surface():
    names = set(declared_functions())
    singles = {'forward_inplace', 'forward_mu', 'forward_nu', 'forward_updates', 'backward_mu',
               'backward_nu', 'backward_updates'}
    want = {f'toa_adam_{s}' for s in singles} | {f'toa_adam_{s}_multi' for s in singles}
    want |= {'toa_adam_abi_version', 'toa_adam_error_string', 'toa_adam_set_waves_per_cu',
             'toa_adam_fused_step', 'toa_adam_fused_step_multi', 'toa_adam_set_max_grid',
             'toa_adam_set_schedule', 'toa_adam_clock_probe', 'toa_adam_set_load_order', 'toa_adam_set_tuning', 'toa_adam_tuned_load_order',
             'toa_adam_set_plan_mode', 'toa_adam_release_plans',
             'toa_adam_state_slack', 'toa_adam_state_shift',
             'toa_adam_forward_inplace_multi_noalloc', 'toa_adam_bias_rows',
             'toa_adam_bias_rows_needed', 'toa_adam_count_advance',
             'toa_adam_forward_inplace_devcount', 'toa_adam_forward_inplace_multi_devcount',
             'toa_adam_fused_step_devcount', 'toa_adam_fused_step_multi_devcount',
             'toa_adam_forward_all', 'toa_adam_forward_all_multi', 'toa_adam_backward_all',
             'toa_adam_backward_all_multi'}
    assert names == want


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f'{name} declared in include/toa_adam.h but not exported'


def test_ctypes_table_matches_header_arity():
    decl = declared_functions()
    for name, argtypes in _lib.SIGNATURES.items():
        assert name in decl
        assert len(argtypes) == len(decl[name]), (name, len(argtypes), decl[name])
    assert set(_lib.SIGNATURES) | {'toa_adam_abi_version', 'toa_adam_error_string'} == set(decl)


def test_abi_version_and_error_strings():
    lib = _lib.load()
    assert lib.toa_adam_abi_version() == _lib.ABI_VERSION
    assert lib.toa_adam_error_string(0) == b'success'
    for code in (-1, -2, -3):
        assert b'toa_adam' in lib.toa_adam_error_string(code)
    with pytest.raises(RuntimeError, match='unsupported dtype'):
        _lib.check(-1, 'x')
    # the fused optimizer step serves the 16-bit types without weight decay only (n = 0: no launch)
    for code in (_lib.TOA_F16, _lib.TOA_BF16):
        assert lib.toa_adam_fused_step(code, None, None, None, None, 0, 0.9, 0.999, 1e-8, 0.0, 1,
                                       1e-3, 0.0, 0, 0, 0, None) == 0
        for decoupled in (0, 1):
            assert lib.toa_adam_fused_step(code, None, None, None, None, 0, 0.9, 0.999, 1e-8, 0.0,
                                           1, 1e-3, 0.01, decoupled, 0, 0, None) == -1
    assert b'weight decay' in lib.toa_adam_error_string(-1)


def test_argument_errors_need_no_device():
    """Bad dtype and empty inputs return before any HIP call."""
    lib = _lib.load()
    assert lib.toa_adam_forward_inplace(5, None, None, None, 0, 0.9, 0.999, 1e-8, 0.0, 1, None) == -1
    assert lib.toa_adam_forward_inplace(0, None, None, None, 0, 0.9, 0.999, 1e-8, 0.0, 1, None) == 0
    assert lib.toa_adam_forward_inplace(0, None, None, None, 8, 0.9, 0.999, 1e-8, 0.0, 1, None) == -2
    assert lib.toa_adam_backward_updates(1, None, None, None, 0, 0.9, 0.999, 0.0, 1, None, None,
                                         None) == 0
    assert lib.toa_adam_forward_inplace_multi(0, 0, None, None, None, None, 0.9, 0.999, 1e-8, 0.0,
                                              None, 1, None) == 0
    assert lib.toa_adam_forward_inplace_multi(9, 2, None, None, None, None, 0.9, 0.999, 1e-8, 0.0,
                                              None, 1, None) == -1
    assert lib.toa_adam_forward_inplace_multi(0, 2, None, None, None, None, 0.9, 0.999, 1e-8, 0.0,
                                              None, 1, None) == -2


def test_waves_knob_round_trip():
    lib = _lib.load()
    first = lib.toa_adam_set_waves_per_cu(16)
    assert lib.toa_adam_set_waves_per_cu(99) == 16  # out of range restores the per-op defaults
    assert lib.toa_adam_set_waves_per_cu(first) == 0


def test_max_grid_knob_round_trip():
    lib = _lib.load()
    default = lib.toa_adam_set_max_grid(64)
    assert default == 1 << 25
    assert lib.toa_adam_set_max_grid(0) == 64  # 0 restores the default
    assert lib.toa_adam_set_max_grid(default) == default


def test_python_surface_names_and_keywords():
    """The seven functions and their keyword names as the reference registers them
    (/root/reference/src/adam_op/adam_op.cpp:157-214), read off the extension's docstrings."""
    want = {
        'forward_': ['updates', 'mu', 'nu', 'b1', 'b2', 'eps', 'eps_root', 'count'],
        'forward_mu': ['updates', 'mu', 'b1'],
        'forward_nu': ['updates', 'nu', 'b2'],
        'forward_updates': ['new_mu', 'new_nu', 'b1', 'b2', 'eps', 'eps_root', 'count'],
        'backward_mu': ['dmu', 'updates', 'mu', 'b1'],
        'backward_nu': ['dnu', 'updates', 'nu', 'b1'],
        'backward_updates': ['dupdates', 'updates', 'new_mu', 'new_nu', 'b1', 'b2', 'eps_root',
                             'count'],
    }
    for name, params in want.items():
        sig = getattr(adam_op, name).__doc__.splitlines()[0]
        assert re.findall(r'(\w+): ', sig) == params, sig
    assert 'count: typing.SupportsInt' in adam_op.forward_.__doc__  # size_t (include/common.h:24)
    # a real extension module with the reference's structure: _C with one submodule
    import torchopt_amd._C
    import torchopt_amd._C.adam_op as sub

    assert sub is adam_op and torchopt_amd._C.__file__.endswith('.so')


def test_cpu_and_meta_tensors_are_refused_not_computed():
    """No CPU path hides behind the op: other devices raise the reference's own error."""
    a = torch.ones(4)
    for fn, args in [
        (adam_op.forward_, (a, a.clone(), a.clone(), 0.9, 0.999, 1e-8, 0.0, 1)),
        (adam_op.forward_mu, (a, a, 0.9)),
        (adam_op.forward_nu, (a, a, 0.999)),
        (adam_op.forward_updates, (a, a, 0.9, 0.999, 1e-8, 0.0, 1)),
        (adam_op.backward_mu, (a, a, a, 0.9)),
        (adam_op.backward_nu, (a, a, a, 0.999)),
        (adam_op.backward_updates, (a, a, a, a, 0.9, 0.999, 0.0, 1)),
        (adam_op.forward_multi_, ([a], [a.clone()], [a.clone()], 0.9, 0.999, 1e-8, 0.0, 1)),
    ]:
        with pytest.raises(RuntimeError, match='Not implemented'):
            fn(*args)
    m = torch.ones(4, device='meta')
    with pytest.raises(RuntimeError, match='Not implemented'):
        adam_op.forward_mu(m, m, 0.9)
    assert torch.equal(a, torch.ones(4))  # untouched


def test_availability_probe_semantics():
    """tests/test_accelerated_op.py:36-40 of the reference: `meta` is never available; here the
    CPU is not served either, and `cuda` follows the machine."""
    assert not accelerated_op_available('meta')
    assert not accelerated_op_available(torch.device('meta'))
    assert not accelerated_op_available('cpu')
    assert not accelerated_op_available(['cpu', 'meta'])
    if not torch.cuda.is_available():
        assert not accelerated_op_available()
        assert not accelerated_op_available('cuda')
        assert not accelerated_op_available('cuda:0')
        assert not accelerated_op_available(0)
        assert not accelerated_op_available(['cuda', 'cpu'])


def test_adam_op_passes_none_updates_through():
    """accelerated_op/adam_op.py:148-149 of the reference."""
    mu, nu = torch.ones(3), torch.ones(3)
    for inplace in (True, False):
        r = AdamOp(inplace=inplace)(mu, nu, None, 1)
        assert r[0] is mu and r[1] is nu and r[2] is None


def test_adam_op_defaults_and_function_classes():
    op = AdamOp()
    assert (op.b1, op.b2, op.eps, op.eps_root, op.inplace) == (0.9, 0.999, 1e-8, 0.0, True)
    with pytest.raises(TypeError):
        AdamOp(0.9, 0.999, 1e-8, 0.0)  # eps_root and inplace are keyword-only
    for cls in (AdamOp.MuOp, AdamOp.NuOp, AdamOp.UpdatesOp):
        assert issubclass(cls, torch.autograd.Function)


def test_fused_adam_argument_validation():
    from torchopt_amd import FusedAdam

    p = [torch.ones(3)]
    for kwargs in (dict(lr=-1.0), dict(eps=-1.0), dict(betas=(1.0, 0.9)), dict(betas=(0.9, 1.0)),
                   dict(weight_decay=-0.01)):
        with pytest.raises(ValueError):
            FusedAdam(p, **kwargs)
    with pytest.raises(TypeError):
        FusedAdam([1.0])
    import torchopt_amd

    # the reference's class names and its `use_accelerated_op` keyword carry over
    assert torchopt_amd.Adam is FusedAdam and torchopt_amd.AdamW is torchopt_amd.FusedAdamW
    assert torchopt_amd.AdamW(p, use_accelerated_op=True).weight_decay == 1e-2
    opt = FusedAdam(p, use_accelerated_op=True)
    assert opt.state_dict() == (None,)
    opt.zero_grad()  # no grads yet: nothing to do
    assert opt.step() is None  # no grads: nothing is launched, counts stay at zero
    assert [int(c) for c in opt.state_dict()[0].count] == [0]
    p[0].grad = torch.ones(3)
    with pytest.raises(RuntimeError, match='Not implemented'):  # CPU parameters are refused
        opt.step()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setattr(_lib, 'LIB_PATH', str(tmp_path / 'libtoa_adam.so'))
    with pytest.raises(ImportError, match='no fallback'):
        _lib.load()


def test_product_never_imports_the_oracle():
    """The oracle is test infrastructure; nothing under torchopt_amd/ may reference it."""
    pkg = os.path.join(REPO, 'torchopt_amd')
    for root, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(('.py', '.hip', '.hpp', '.h')):
                text = open(os.path.join(root, f)).read()
                assert not re.search(r'^\s*(from|import)\s+oracle\b', text, flags=re.M), f
                assert 'liboracle' not in text and 'adam_oracle' not in text, f


def test_asking_for_the_non_accelerated_path_warns():
    """The reference builds another scaler for use_accelerated_op=False
    (/root/reference/torchopt/alias/adam.py:118); here the request is answered with a warning."""
    import torchopt_amd
    from torchopt_amd import alias

    with pytest.warns(UserWarning, match='use_accelerated_op=False'):
        alias.adam(use_accelerated_op=False)
    with pytest.warns(UserWarning, match='use_accelerated_op=False'):
        alias.adamw(use_accelerated_op=False)
    with pytest.warns(UserWarning, match='use_accelerated_op=False'):
        torchopt_amd.FusedAdam([torch.zeros(3, requires_grad=True)], use_accelerated_op=False)
    with warnings.catch_warnings():
        warnings.simplefilter('error')
        alias.adam(use_accelerated_op=True)


def test_availability_probe_is_loud_about_the_cpu():
    """TorchOpt answers True for 'cpu' (/root/reference/tests/test_accelerated_op.py:33-34);
    this build has no CPU kernels and says so."""
    with pytest.warns(UserWarning, match='no CPU kernels'):
        assert not accelerated_op_available('cpu')
    with pytest.warns(UserWarning, match='no CPU kernels'):
        assert not accelerated_op_available(['cpu', 'cuda'])
    assert not accelerated_op_available('not-a-device')


def test_state_placement_advice():
    """toa_adam_state_shift: the bytes to skip so a first moment starts 8 KiB past a multiple of
    16 KiB and a second moment at one: the two 8 KiB apart modulo 16 KiB."""
    lib = _lib.load()
    slack = lib.toa_adam_state_slack()
    assert slack == 16 << 10
    for base in (0, 256, 8 << 10, (8 << 10) + 512, (16 << 10) - 256, (2 << 20) * 37, 0x7f12_3456_7800):
        for moment, phase in ((0, 8 << 10), (1, 0)):
            shift = lib.toa_adam_state_shift(base, moment)
            assert 0 <= shift < slack and shift % 256 == base % 256 == 0
            assert (base + shift) % slack == phase
    # CPU tensors, small tensors and non-contiguous ones are plain zeros_like / empty_like
    import torch

    from torchopt_amd.placement import state_empty_like, state_zeros_like

    t = torch.ones(3, 5, dtype=torch.float64).t()
    z = state_zeros_like(t, requires_grad=True)
    assert z.shape == t.shape and z.stride() == t.stride() and z.requires_grad and not z.any()
    assert state_empty_like(torch.ones(7)).storage_offset() == 0
    from torchopt_amd.placement import state_zeros_like_tree

    mu, nu = state_zeros_like_tree([torch.ones(1 << 19), None, t], requires_grad=True)
    assert mu[1] is None and nu[1] is None and mu[0].storage_offset() == 0 and nu[2].stride() == t.stride()
    assert all(x.requires_grad and not x.any() for x in (mu[0], nu[0], mu[2], nu[2]))


def test_recorded_traffic_figures_are_the_ones_in_the_profile_summaries():
    """bench.py quotes counter traffic recorded by rocprofv3 runs; each figure must be the one its
    named summary under profiles/ states."""
    import bench

    for cfg, (traffic, source) in bench.RECORDED_TRAFFIC.items():
        text = open(os.path.join(REPO, source)).read()
        spaced = f'{traffic:,}'.replace(',', ' ')
        assert spaced in text or str(traffic) in text, (cfg, traffic, source)
