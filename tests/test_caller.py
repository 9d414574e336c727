"""`scale_by_accelerated_adam` host logic that needs no GPU: argument validation, empty and
None-only trees (the cases /root/reference/tests/test_alias.py:35-79 pushes through the
accelerated path), state construction, count bookkeeping."""

from __future__ import annotations

import collections

import pytest
import torch

from torchopt_amd.base import GradientTransformation
from torchopt_amd.transform import ScaleByAdamState, scale_by_accelerated_adam
from torchopt_amd.transform.scale_by_adam import INT64_MAX, _host_value, _inc_counts, _remember


def test_returns_an_init_update_pair():
    t = scale_by_accelerated_adam()
    assert isinstance(t, GradientTransformation) and isinstance(t, tuple) and len(t) == 2
    init, update = t
    assert callable(init) and callable(update)
    assert callable(scale_by_accelerated_adam.flat) and callable(scale_by_accelerated_adam.impl)


@pytest.mark.parametrize('kwargs', [dict(eps=-1e-8), dict(eps=float('nan')), dict(b1=1.0),
                                    dict(b1=-0.1), dict(b2=1.0), dict(b2=1.5)])
def test_hyper_parameter_validation(kwargs):
    with pytest.raises(ValueError):
        scale_by_accelerated_adam(**kwargs)
    with pytest.raises(ValueError):
        scale_by_accelerated_adam.flat(**kwargs)


@pytest.mark.parametrize('tree', [{}, (), [], (None,), {'a': (), 'b': {'c': []}, 'd': None}],
                         ids=['dict', 'tuple', 'list', 'none-leaf', 'nested'])
@pytest.mark.parametrize('inplace', [True, False])
def test_empty_trees_pass_through(tree, inplace):
    t = scale_by_accelerated_adam()
    state = t.init(tree)
    assert state == ScaleByAdamState(mu=tree, nu=tree, count=tree)
    updates, new_state = t.update(tree, state, params=tree, inplace=inplace)
    assert updates == tree and new_state == state
    assert type(updates) is type(tree)


def test_flat_variant_keeps_sequence_types():
    t = scale_by_accelerated_adam.flat()
    for seq in ([], (), [None, None], (None,)):
        state = t.init(seq)
        assert type(state.mu) is type(seq) and type(state.count) is type(seq)
        updates, new_state = t.update(seq, state, inplace=True)
        assert updates == seq and type(updates) is type(seq)
        assert type(new_state.nu) is type(seq)


def test_init_builds_zero_moments_and_zero_dim_counts():
    Point = collections.namedtuple('Point', 'w b')
    params = {'layer': Point(torch.randn(3, 4, dtype=torch.float64), torch.randn(4)), 'skip': None}
    state = scale_by_accelerated_adam(moment_requires_grad=True).init(params)
    assert isinstance(state.mu['layer'], Point) and state.mu['skip'] is None
    for m, p in ((state.mu['layer'].w, params['layer'].w), (state.nu['layer'].b, params['layer'].b)):
        assert m.shape == p.shape and m.dtype == p.dtype and m.requires_grad
        assert not m.any()
    c = state.count['layer'].w
    assert c.dim() == 0 and c.dtype == torch.int64 and int(c) == 0
    # every leaf has its counter; leaves of one device may share the tensor while in step
    assert int(state.count['layer'].b) == 0 and state.count['skip'] is None


def test_count_increment_skips_missing_gradients_and_saturates():
    counts = [_remember(torch.tensor(0), 0), _remember(torch.tensor(4), 4),
              torch.tensor(INT64_MAX), None]
    grads = [torch.ones(1), None, torch.ones(1), None]
    new, values = _inc_counts(counts, grads)
    assert values == [1, 4, INT64_MAX, None]
    assert int(new[0]) == 1 and new[1] is counts[1] and new[2] is counts[2] and new[3] is None
    assert int(counts[0]) == 0  # functional: the old state is untouched


def test_count_mirror_notices_in_place_edits():
    c = _remember(torch.tensor(7), 7)
    assert _host_value(c) == 7
    c.add_(5)  # someone rewinds or restores the state in place
    assert _host_value(c) == 12
    fresh = torch.tensor(3)  # e.g. from a loaded state dict: no mirror yet
    assert _host_value(fresh) == 3 and _host_value(fresh) == 3


def test_mismatched_state_is_reported():
    t = scale_by_accelerated_adam()
    state = t.init([None, None])
    with pytest.raises(ValueError, match='tree structures'):
        t.update([None], state)


def test_cpu_leaves_are_refused():
    """The op has no CPU path and the caller does not invent one."""
    t = scale_by_accelerated_adam()
    params = [torch.ones(3)]
    state = t.init(params)
    with pytest.raises(RuntimeError, match='Not implemented'):
        t.update([torch.ones(3)], state, inplace=True)


def test_fused_adam_refuses_weight_decay_on_16_bit_parameters():
    from torchopt_amd import FusedAdam, FusedAdamW

    p16 = torch.zeros(4, dtype=torch.bfloat16, requires_grad=True)
    p32 = torch.zeros(4, requires_grad=True)
    FusedAdam([p16, p32])  # no decay: fine
    FusedAdamW([p32], weight_decay=0.01)
    for cls in (FusedAdam, FusedAdamW):
        with pytest.raises(ValueError, match='float32 and float64 parameters only'):
            cls([p32, p16], weight_decay=0.01)
