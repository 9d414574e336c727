"""The two-callable protocol every TorchOpt transformation follows
(/root/reference/torchopt/base.py:118-151).  A plain NamedTuple of (init, update): the
reference's `chain` accepts any such pair, so a transformation built here can be chained with
the reference's own."""

from __future__ import annotations

import warnings
from typing import Any, Callable, NamedTuple


class GradientTransformation(NamedTuple):
    """``init(params) -> state`` and ``update(updates, state, *, params=None, inplace=True)
    -> (updates, state)``."""

    init: Callable[..., Any]
    update: Callable[..., Any]


def accelerated_only(use_accelerated_op: bool, who: str) -> None:
    """The reference builds a different (pure-PyTorch) scaler when ``use_accelerated_op`` is false
    (/root/reference/torchopt/alias/adam.py:118).  This package holds the fused operator only, so
    a caller asking for the other path is told that it still gets the fused one."""
    if not use_accelerated_op:
        warnings.warn(
            f'{who}: use_accelerated_op=False was requested, but torchopt_amd implements the '
            'accelerated (fused, GPU-only) Adam operator alone; the accelerated path is used. '
            'Take the non-accelerated scaler from TorchOpt itself if that is what you need.',
            UserWarning, stacklevel=3)
