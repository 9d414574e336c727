"""Functional Adam / AdamW on the fused operator, and the glue around it.

Counterparts of /root/reference/torchopt/alias/adam.py:116-137 and alias/adamw.py:127-151 with
``use_accelerated_op=True`` built in: the same chains of gradient transformations

    adam:   flip_sign_and_add_weight_decay -> scale_by_accelerated_adam -> scale_by_neg_lr
    adamw:  flip_sign (no decay)           -> scale_by_accelerated_adam -> add_decayed_weights
                                           -> scale_by_neg_lr

where only `scale_by_accelerated_adam` is native code; its neighbours are the reference's
one-line tensor operations (`neg`, `add(p, alpha=wd)`, `mul(step)`;
/root/reference/torchopt/alias/utils.py:75-193, transform/add_decayed_weights.py:195-258,
transform/scale.py:65-107, transform/scale_by_schedule.py:72-128), applied leaf by leaf out of
place so gradients flow, and with one fused list call per transformation in place.
`chain` (/root/reference/torchopt/base.py:154-235, combine.py:49-105) threads updates through
the transformations and keeps one state per transformation; `apply_updates`
(/root/reference/torchopt/update.py:50-81) adds updates to parameters.

Trees are plain containers (``None`` is a leaf), flattened by `torchopt_amd._tree`: flat lists,
tuples and dicts of tensors directly, anything else with ``torch.utils._pytree``.
"""

from __future__ import annotations

from itertools import repeat
from operator import is_
from typing import Any, Callable, NamedTuple

import torch

from torchopt_amd._tree import flatten, leaves_like, rebuild
from torchopt_amd.base import GradientTransformation, accelerated_only
from torchopt_amd.transform.scale_by_adam import _inc_counts, _remember, scale_by_accelerated_adam


__all__ = ['adam', 'adamw', 'apply_updates', 'chain']


class EmptyState(NamedTuple):
    """State of a transformation that keeps none."""


class ScaleByScheduleState(NamedTuple):
    """Step count per leaf, fed to the learning-rate schedule."""

    count: Any


def _map_leaves(fn: Callable, tree: Any, *rest: Any) -> Any:
    """``fn`` over corresponding leaves; a ``None`` in the first tree stays ``None``."""
    leaves, spec = flatten(tree)
    others = [leaves_like(r, spec) for r in rest]
    out = [None if x is None else fn(x, *(o[k] for o in others)) for k, x in enumerate(leaves)]
    return rebuild(out, tree, spec)


def _tensors(tree: Any, *rest: Any):
    """Parallel lists of the non-``None`` leaves of `tree` and their partners in `rest`."""
    leaves, spec = flatten(tree)
    others = [leaves_like(r, spec) for r in rest]
    if not any(map(is_, leaves, repeat(None))):
        return leaves, others
    keep = [k for k, x in enumerate(leaves) if x is not None]
    return [leaves[k] for k in keep], [[o[k] for k in keep] for o in others]


def chain(*transformations: GradientTransformation) -> GradientTransformation:
    """Apply transformations in sequence; the state is the tuple of their states."""
    inits = [t[0] for t in transformations]
    updates_fns = [t[1] for t in transformations]

    def init_fn(params):
        return tuple(fn(params) for fn in inits)

    def update_fn(updates, state, *, params=None, inplace=True):
        if len(updates_fns) != len(state):
            raise ValueError('The number of updates and states has to be the same in chain! '
                             'Make sure you have called init first!')
        new_state = []
        for s, fn in zip(state, updates_fns):
            updates, new_s = fn(updates, s, params=params, inplace=inplace)
            new_state.append(new_s)
        return updates, tuple(new_state)

    return GradientTransformation(init_fn, update_fn)


def _stateless(update: Callable) -> GradientTransformation:
    def update_fn(updates, state, *, params=None, inplace=True):
        return update(updates, params, inplace), state

    return GradientTransformation(lambda params: EmptyState(), update_fn)


def _flip_sign_and_add_weight_decay(weight_decay: float, maximize: bool) -> GradientTransformation:
    """``g (+ wd * p)`` for descent, ``-g (+ wd * p)`` for ascent (alias/utils.py:75-193)."""
    if not weight_decay >= 0.0:
        raise ValueError(f'Invalid weight_decay value: {weight_decay}')

    def update(updates, params, inplace):
        if not maximize and weight_decay == 0.0:
            return updates
        if weight_decay != 0.0 and params is None:
            raise AssertionError('Parameters are required for weight decay. '
                                 'Call `update(updates, state, params=params)` instead.')
        if inplace:
            if weight_decay != 0.0:
                gs, (ps,) = _tensors(updates, params)
            else:
                gs, ps = _tensors(updates)[0], []
            if gs and maximize:
                torch._foreach_neg_(gs)
            if gs and weight_decay != 0.0:
                torch._foreach_add_(gs, [p.detach() for p in ps], alpha=weight_decay)
            return updates
        if weight_decay == 0.0:
            return _map_leaves(lambda g: g.neg(), updates)
        if maximize:
            return _map_leaves(lambda g, p: g.neg().add_(p, alpha=weight_decay), updates, params)
        return _map_leaves(lambda g, p: g.add(p, alpha=weight_decay), updates, params)

    return _stateless(update)


def _add_decayed_weights(weight_decay: float, mask: Any = None) -> GradientTransformation:
    """``u + wd * p`` after the Adam scaling (transform/add_decayed_weights.py:195-258).  `mask`
    is a tree of booleans shaped like the parameters, or a callable that makes one from them:
    leaves marked ``False`` pass through undecayed (transform/add_decayed_weights.py:252-258 via
    the masked wrapper)."""
    if not weight_decay >= 0.0:
        raise ValueError(f'Invalid weight_decay value: {weight_decay}')

    def update(updates, params, inplace):
        if weight_decay == 0.0:
            return updates
        if params is None:
            raise AssertionError('Parameters are required for weight decay. '
                                 'Call `update(updates, state, params=params)` instead.')
        if mask is None:
            chosen = None
        else:
            chosen = leaves_like(mask(params) if callable(mask) else mask, flatten(updates)[1])
        if inplace:
            gs, (ps,) = _tensors(updates, params)
            if chosen is not None:
                keep = [k for k, x in enumerate(flatten(updates)[0]) if x is not None]
                picked = [j for j, k in enumerate(keep) if chosen[k]]
                gs, ps = [gs[j] for j in picked], [ps[j] for j in picked]
            if gs:
                torch._foreach_add_(gs, [p.detach() for p in ps], alpha=weight_decay)
            return updates
        if chosen is None:
            return _map_leaves(lambda g, p: g.add(p, alpha=weight_decay), updates, params)
        marks = iter(chosen)
        leaves, spec = flatten(updates)
        p_leaves = leaves_like(params, spec)
        out = [g if (g is None or not m) else g.add(p, alpha=weight_decay)
               for g, p, m in zip(leaves, p_leaves, marks)]
        return rebuild(out, updates, spec)

    return _stateless(update)


def _scale_by_neg_lr(lr) -> GradientTransformation:
    """``u * -lr``, or ``u * -lr(count)`` with a schedule (alias/utils.py:209-226)."""
    if not (callable(lr) or lr >= 0.0):
        raise ValueError(f'Invalid learning rate: {lr}')
    if not callable(lr):
        def update(updates, params, inplace):
            if inplace:
                gs = _tensors(updates)[0]
                if gs:
                    torch._foreach_mul_(gs, -lr)
                return updates
            return _map_leaves(lambda g: g.mul(-lr), updates)

        return _stateless(update)

    def init_fn(params):
        return ScaleByScheduleState(count=_map_leaves(
            lambda t: _remember(torch.zeros(1, dtype=torch.int64, device=t.device).squeeze_(), 0),
            params))

    def update_fn(updates, state, *, params=None, inplace=True):
        def scale(g, c):
            step = -lr(c)  # the schedule sees the count before this step, as in the reference
            return g.mul_(step) if inplace else g.mul(step)

        new_updates = _map_leaves(scale, updates, state.count)
        c_leaves, c_spec = flatten(state.count)
        new_counts, _ = _inc_counts(c_leaves, leaves_like(updates, c_spec))
        return new_updates, ScaleByScheduleState(count=rebuild(new_counts, state.count, c_spec))

    return GradientTransformation(init_fn, update_fn)


def _check(lr, b1, b2, eps, weight_decay):
    if not (callable(lr) or lr >= 0.0):
        raise ValueError(f'Invalid learning rate: {lr}')
    if not eps >= 0.0:
        raise ValueError(f'Invalid epsilon value: {eps}')
    if not 0.0 <= b1 < 1.0:
        raise ValueError(f'Invalid beta parameter at index 0: {b1}')
    if not 0.0 <= b2 < 1.0:
        raise ValueError(f'Invalid beta parameter at index 1: {b2}')
    if not weight_decay >= 0.0:
        raise ValueError(f'Invalid weight_decay value: {weight_decay}')


def adam(
    lr=1e-3,
    betas: tuple[float, float] = (0.9, 0.999),
    eps: float = 1e-8,
    weight_decay: float = 0.0,
    *,
    eps_root: float = 0.0,
    moment_requires_grad: bool = False,
    maximize: bool = False,
    use_accelerated_op: bool = True,  # False warns: only the accelerated path exists here
) -> GradientTransformation:
    """Functional Adam on the fused operator (L2 weight decay is added to the gradient)."""
    accelerated_only(use_accelerated_op, 'adam')
    b1, b2 = betas
    _check(lr, b1, b2, eps, weight_decay)
    return chain(
        _flip_sign_and_add_weight_decay(weight_decay, maximize),
        scale_by_accelerated_adam(b1, b2, eps, eps_root, moment_requires_grad),
        _scale_by_neg_lr(lr),
    )


def adamw(
    lr=1e-3,
    betas: tuple[float, float] = (0.9, 0.999),
    eps: float = 1e-8,
    weight_decay: float = 1e-2,
    *,
    eps_root: float = 0.0,
    mask: Any = None,
    moment_requires_grad: bool = False,
    maximize: bool = False,
    use_accelerated_op: bool = True,  # False warns: only the accelerated path exists here
) -> GradientTransformation:
    """Functional AdamW on the fused operator (decoupled decay is added to the scaled update;
    `mask` selects the leaves that decay)."""
    accelerated_only(use_accelerated_op, 'adamw')
    b1, b2 = betas
    _check(lr, b1, b2, eps, weight_decay)
    return chain(
        _flip_sign_and_add_weight_decay(0.0, maximize),
        scale_by_accelerated_adam(b1, b2, eps, eps_root, moment_requires_grad),
        _add_decayed_weights(weight_decay, mask),
        _scale_by_neg_lr(lr),
    )


def apply_updates(params: Any, updates: Any, *, inplace: bool = True) -> Any:
    """``params + updates`` leaf by leaf; a ``None`` update leaves its parameter as it is."""
    p_leaves, spec = flatten(params)
    u_leaves = leaves_like(updates, spec)
    if inplace:
        pairs = [(p, u) for p, u in zip(p_leaves, u_leaves) if p is not None and u is not None]
        if pairs:
            torch._foreach_add_([p.data for p, _ in pairs], [u for _, u in pairs])
        return params
    out = [p if (p is None or u is None) else p.add(u) for p, u in zip(p_leaves, u_leaves)]
    return rebuild(out, params, spec)
