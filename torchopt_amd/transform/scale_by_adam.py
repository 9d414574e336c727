"""`scale_by_accelerated_adam`: the caller of the fused Adam operator.

Counterpart of /root/reference/torchopt/transform/scale_by_adam.py:225-420 and of `inc_count`
(/root/reference/torchopt/transform/utils.py:111-126).  Same contract:

  * validates ``eps >= 0`` and ``0 <= b1, b2 < 1`` (:293-298);
  * ``init(params)`` -> ``ScaleByAdamState(mu, nu, count)`` with, per leaf, zero moments shaped
    like the parameter (``requires_grad=moment_requires_grad``) and a 0-dim int64 count on the
    leaf's device (:401-414; the leaves of one device share one count tensor for as long as they
    step together, which the reference's per-leaf tensors of equal value cannot be told from
    unless somebody writes into one in place); ``None`` parameters give ``None`` state leaves;
  * ``update(updates, state, *, params=None, inplace=True)`` increments the count of every leaf
    whose gradient is not ``None`` (saturating at INT64_MAX), applies the Adam op and returns
    ``(new_updates, ScaleByAdamState(new_mu, new_nu, count_inc))`` with the container types of
    the inputs; a ``None`` gradient leaves that leaf's mu, nu and count as they are and yields a
    ``None`` update; a ``None`` moment yields ``(None, None, None)``; empty trees pass through
    (:304-399);
  * `.flat` takes and returns flat sequences, `.impl` takes ``already_flattened``.

What is different is the mechanics.  The reference calls the op once per leaf from Python and
hands it the count as a device tensor, which costs a launch and a device-to-host read per leaf.
Here the whole tree goes to the multi-tensor entry points (one launch per op for about a
hundred leaves), the counts are advanced with one fused launch, and their values are mirrored on
the host so no step reads them back from the device.

Trees are plain Python containers (dict / list / tuple / namedtuple; ``None`` is a leaf),
flattened by `torchopt_amd._tree`: flat lists, tuples and dicts of tensors directly -- dicts
matched by name, as the reference's key-sorting pytree library has it -- and anything nested with
``torch.utils._pytree``.
"""

from __future__ import annotations

from itertools import repeat
from operator import is_
from typing import Any, NamedTuple, Sequence

import torch

from torchopt_amd import _tree
from torchopt_amd.accelerated_op import MultiAdamOp
from torchopt_amd.accelerated_op.adam_op import adam_op
from torchopt_amd.base import GradientTransformation
from torchopt_amd.placement import state_zeros_like_tree


__all__ = ['ScaleByAdamState', 'scale_by_accelerated_adam']

INT64_MAX = torch.iinfo(torch.int64).max
_MIRROR = '_toa_host_value'


class ScaleByAdamState(NamedTuple):
    """State for the Adam algorithm: first moment, second moment, step count (one per leaf)."""

    mu: Any
    nu: Any
    count: Any


# ------------------------------------------------------------------------------ count mirror


def _remember(t: torch.Tensor, value: int) -> torch.Tensor:
    """Attach the host copy of a count tensor's value, valid while the tensor is unmodified."""
    setattr(t, _MIRROR, (value, t._version))
    return t


def _host_value(t: torch.Tensor) -> int:
    """Value of a 0-dim count tensor; reads the device only if the mirror is missing or stale."""
    known = getattr(t, _MIRROR, None)
    if known is not None and known[1] == t._version:
        return known[0]
    value = int(t)
    _remember(t, value)
    return value


def _inc_counts(counts: Sequence[torch.Tensor | None], grads: Sequence[Any]):
    """``c + (c != INT64_MAX)`` for leaves with a gradient, the same tensor otherwise.
    Returns (new count leaves, host values of the new counts).

    Leaves that hold the very same count tensor (as the leaves of one `init` do, see there) are
    advanced together: one addition, one new tensor, shared again by all of them."""
    first = counts[0] if counts else None
    if (first is not None and all(c is first for c in counts)
            and all(g is not None for g in grads)):
        # the usual case, in one go: every leaf shares the count tensor `init` made and every
        # leaf has a gradient
        v = _host_value(first)
        if v == INT64_MAX:
            return list(counts), [v] * len(counts)
        fresh = _remember(first + 1, v + 1)
        return [fresh] * len(counts), [v + 1] * len(counts)
    values = [None] * len(counts)
    seen: dict[int, int] = {}      # id(count tensor) -> its host value
    bump: dict[int, torch.Tensor] = {}  # id -> tensor to advance
    for k, c in enumerate(counts):
        if c is None:
            continue
        key = id(c)
        v = seen.get(key)
        if v is None:
            v = seen[key] = _host_value(c)
        values[k] = v
        if grads[k] is not None and v != INT64_MAX:
            bump[key] = c
    if not bump:
        return list(counts), values
    olds = list(bump.values())
    by_device: dict[torch.device, list[int]] = {}
    for j, c in enumerate(olds):
        by_device.setdefault(c.device, []).append(j)
    fresh: dict[int, torch.Tensor] = {}
    for js in by_device.values():
        bumped = torch._foreach_add([olds[j] for j in js], 1)  # one fused launch per device
        for j, t in zip(js, bumped):
            key = id(olds[j])
            fresh[key] = _remember(t, seen[key] + 1)
    new = list(counts)
    for k, c in enumerate(counts):
        if c is not None and grads[k] is not None:
            t = fresh.get(id(c))
            if t is not None:
                new[k] = t
                values[k] += 1
    return new, values


# ------------------------------------------------------------------------------ the transformation


def scale_by_accelerated_adam(
    b1: float = 0.9,
    b2: float = 0.999,
    eps: float = 1e-8,
    eps_root: float = 0.0,
    moment_requires_grad: bool = False,
) -> GradientTransformation:
    """Rescale updates according to the Adam algorithm, on the fused GPU operator.

    Args:
        b1: decay rate of the first moment.
        b2: decay rate of the second raw moment.
        eps: added to the denominator outside the square root.
        eps_root: added inside the square root (keeps the backward pass finite).
        moment_requires_grad: create the moments with ``requires_grad=True``.

    Returns:
        An ``(init, update)`` pair.
    """
    return _scale_by_accelerated_adam(b1, b2, eps, eps_root, moment_requires_grad,
                                      already_flattened=False)


def _scale_by_accelerated_adam_flat(
    b1: float = 0.9,
    b2: float = 0.999,
    eps: float = 1e-8,
    eps_root: float = 0.0,
    moment_requires_grad: bool = False,
) -> GradientTransformation:
    return _scale_by_accelerated_adam(b1, b2, eps, eps_root, moment_requires_grad,
                                      already_flattened=True)


def _scale_by_accelerated_adam(
    b1: float = 0.9,
    b2: float = 0.999,
    eps: float = 1e-8,
    eps_root: float = 0.0,
    moment_requires_grad: bool = False,
    *,
    already_flattened: bool = False,
) -> GradientTransformation:
    if not eps >= 0.0:
        raise ValueError(f'Invalid epsilon value: {eps}')
    if not 0.0 <= b1 < 1.0:
        raise ValueError(f'Invalid beta parameter at index 0: {b1}')
    if not 0.0 <= b2 < 1.0:
        raise ValueError(f'Invalid beta parameter at index 1: {b2}')

    ops = {flag: MultiAdamOp(b1=b1, b2=b2, eps=eps, eps_root=eps_root, inplace=flag)
           for flag in (False, True)}

    def flatten(tree):
        if already_flattened:
            return list(tree), None
        return _tree.flatten(tree)

    rebuild = _tree.rebuild

    def init_fn(params):
        leaves, spec = flatten(params)
        count = []
        # The leaves of one device start from ONE 0-dim count tensor and keep sharing the
        # tensors `update` returns for as long as they step together (a leaf that misses a
        # gradient falls behind and goes its own way from there).  The values are what the
        # reference's per-leaf tensors hold; what is saved is a tensor object and an addition per
        # leaf per step.  Counts are never modified in place here.
        zeros: dict[torch.device, torch.Tensor] = {}
        for t in leaves:
            if t is None:
                count.append(None)
                continue
            zero = zeros.get(t.device)
            if zero is None:
                zero = zeros[t.device] = _remember(
                    torch.zeros(1, dtype=torch.int64, device=t.device).squeeze_(), 0)
            count.append(zero)
        # every mu, then every nu, as mapping zeros_like over the tree once per moment does
        # (:407-414): a leaf's two moments then lie a whole model apart in memory, which the
        # three-stream in-place step measurably prefers to neighbours (+2 % on a transformer's
        # parameter list).  Large GPU leaves get their moments from one block, every first moment
        # and then every second, each at the address phase the step streams fastest from
        # (placement.py); values and layout are zeros_like's.
        mu, nu = state_zeros_like_tree(leaves, requires_grad=moment_requires_grad)
        return ScaleByAdamState(mu=rebuild(mu, params, spec), nu=rebuild(nu, params, spec),
                                count=rebuild(count, params, spec))

    def update_fn(updates, state, *, params=None, inplace=True):  # noqa: ARG001
        if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
            # The step numbers advance on the host here (a mirror of the count tensors), and the
            # launches carry their bias corrections as arguments: a captured update would replay
            # one step number for ever.  (The reference fails here too: converting its device
            # count to size_t reads the device, which capture forbids.)
            raise RuntimeError(
                'scale_by_accelerated_adam.update() cannot be captured in a HIP graph: the step '
                'count is read on the host.  Use torchopt_amd.FusedAdam(..., capturable=True), '
                'or call the torchopt_amd._C.adam_op functions with the count you mean to freeze.')
        g_leaves, g_spec = flatten(updates)
        mu_leaves, mu_spec = flatten(state.mu)
        nu_leaves, nu_spec = flatten(state.nu)
        c_leaves, c_spec = flatten(state.count)
        if (type(g_spec) is _tree.DictSpec and type(mu_spec) is _tree.DictSpec
                and g_spec.keys != mu_spec.keys):
            # the same names in another order: line the gradients up with the state
            g_leaves = _tree.leaves_like(updates, mu_spec)
            g_spec = _tree.DictSpec(g_spec.kind, mu_spec.keys)
        n = len(g_leaves)
        if not (len(mu_leaves) == len(nu_leaves) == len(c_leaves) == n):
            raise ValueError('updates and optimizer state have different tree structures; '
                             'make sure `init` was called on matching parameters')

        new_counts, count_values = _inc_counts(c_leaves, g_leaves)

        op = ops[bool(inplace)]
        if adam_op.one_kind(g_leaves) and not any(map(is_, mu_leaves, repeat(None))):
            # the usual tree in one go: every leaf has a gradient and a state, one device, one
            # dtype (asked in C; the general sorting below costs ~0.3 us per leaf)
            first = count_values[0]
            counts = first if count_values.count(first) == n else count_values
            new_mu, new_nu, new_g = op(mu_leaves, nu_leaves, g_leaves, counts)
            return (rebuild(list(new_g), updates, g_spec),
                    ScaleByAdamState(mu=rebuild(list(new_mu), state.mu, mu_spec),
                                     nu=rebuild(list(new_nu), state.nu, nu_spec),
                                     count=rebuild(new_counts, state.count, c_spec)))

        new_mu, new_nu, new_g = list(mu_leaves), list(nu_leaves), list(g_leaves)
        groups: dict[tuple, list[int]] = {}
        for k in range(n):
            if mu_leaves[k] is None:  # no state for this leaf: nothing comes out of it
                new_mu[k] = new_nu[k] = new_g[k] = None
            elif g_leaves[k] is not None:
                g = g_leaves[k]
                groups.setdefault((g.device, g.dtype), []).append(k)
            # a None gradient keeps mu and nu and yields a None update

        for ks in groups.values():
            values = [count_values[k] for k in ks]
            counts = values[0] if len(set(values)) == 1 else values
            if len(ks) == n:  # the whole tree is one group: no re-indexing
                new_mu, new_nu, new_g = (list(x) for x in op(mu_leaves, nu_leaves, g_leaves,
                                                             counts))
                break
            out_mu, out_nu, out_g = op([mu_leaves[k] for k in ks], [nu_leaves[k] for k in ks],
                                       [g_leaves[k] for k in ks], counts)
            for k, m, v, g in zip(ks, out_mu, out_nu, out_g):
                new_mu[k], new_nu[k], new_g[k] = m, v, g

        return (rebuild(new_g, updates, g_spec),
                ScaleByAdamState(mu=rebuild(new_mu, state.mu, mu_spec),
                                 nu=rebuild(new_nu, state.nu, nu_spec),
                                 count=rebuild(new_counts, state.count, c_spec)))

    return GradientTransformation(init_fn, update_fn)


scale_by_accelerated_adam.flat = _scale_by_accelerated_adam_flat  # type: ignore[attr-defined]
scale_by_accelerated_adam.impl = _scale_by_accelerated_adam  # type: ignore[attr-defined]
