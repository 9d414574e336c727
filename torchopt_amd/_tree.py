"""Flattening of parameter trees into lists of leaves and back.

Trees are plain Python containers; ``None`` is a leaf.  The general case is
``torch.utils._pytree`` (pure Python: ~0.5 us per leaf per direction).  The two shapes that
optimizer code meets almost always are flattened here without that walk: a list or tuple of
tensors, which is its own flattening, and a dict of tensors (``dict(module.named_parameters())``),
which flattens to its values in insertion order, as ``torch.utils._pytree`` has it.

Two flat dicts with the same keys in different orders are lined up BY NAME (`leaves_like`):
the reference's pytree library sorts the keys of a dict
(/root/reference/torchopt/pytree.py, on `optree`), so order never matters there, and it must
not here.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import Any, NamedTuple

import torch
from torch.utils import _pytree as pytree


# exact leaf types a flat container may hold to count as already flattened (checked in C)
PLAIN_LEAVES = frozenset({torch.Tensor, torch.nn.Parameter, type(None)})


class DictSpec(NamedTuple):
    """How to put a flat dict back together: its type (dict or OrderedDict) and its keys."""

    kind: type
    keys: tuple


def flatten(tree: Any):
    """``(leaves, spec)``; `spec` is None for a flat list / tuple, a `DictSpec` for a flat dict,
    a ``TreeSpec`` otherwise."""
    kind = type(tree)
    if kind in (list, tuple) and PLAIN_LEAVES.issuperset(map(type, tree)):
        return list(tree), None
    if kind in (dict, OrderedDict) and PLAIN_LEAVES.issuperset(map(type, tree.values())):
        return list(tree.values()), DictSpec(kind, tuple(tree.keys()))
    return pytree.tree_flatten(tree)


def rebuild(leaves: list, like: Any, spec: Any):
    """The tree `flatten` took apart, with new leaves; `like` gives a flat sequence its type."""
    if spec is None:
        return leaves if type(like) is list else type(like)(leaves)
    if type(spec) is DictSpec:
        return spec.kind(zip(spec.keys, leaves))
    return pytree.tree_unflatten(leaves, spec)


def leaves_like(other: Any, spec: Any) -> list:
    """The leaves of `other` in the order `spec` (from `flatten` of a partner tree) lists them:
    by name when both are flat dicts, by position otherwise."""
    leaves, other_spec = flatten(other)
    if (type(spec) is DictSpec and type(other_spec) is DictSpec
            and other_spec.keys != spec.keys):
        if len(other_spec.keys) != len(spec.keys) or set(other_spec.keys) != set(spec.keys):
            raise ValueError('trees are dicts with different keys; make sure `init` was called '
                             'on matching parameters')
        return [other[k] for k in spec.keys]
    return leaves
