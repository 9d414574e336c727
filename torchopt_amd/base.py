"""The two-callable protocol every TorchOpt transformation follows
(/root/reference/torchopt/base.py:118-151).  A plain NamedTuple of (init, update): the
reference's `chain` accepts any such pair, so a transformation built here can be chained with
the reference's own."""

from __future__ import annotations

from typing import Any, Callable, NamedTuple


class GradientTransformation(NamedTuple):
    """``init(params) -> state`` and ``update(updates, state, *, params=None, inplace=True)
    -> (updates, state)``."""

    init: Callable[..., Any]
    update: Callable[..., Any]
