"""`FuncOptimizer`: holds the state of a functional optimizer and steps a tree of parameters.

Counterpart of /root/reference/torchopt/optim/func/base.py:33-126: ``step(loss, params)`` takes
the gradients of `loss` with ``create_graph=True``, runs the transformation (out of place unless
told otherwise) and returns the updated parameters in the container they came in.  With
``torchopt_amd.adam(...)`` as the transformation one step is two launches of the fused operator
for the whole tree.
"""

from __future__ import annotations

import torch
from torch.utils import _pytree as pytree

from torchopt_amd import alias
from torchopt_amd.base import GradientTransformation


__all__ = ['FuncOptimizer']


class FuncOptimizer:
    """Wrapper that owns the optimizer state of a `GradientTransformation`."""

    def __init__(self, impl: GradientTransformation, *, inplace: bool = False) -> None:
        if not isinstance(impl, GradientTransformation):
            raise TypeError(f'{impl} (type: {type(impl).__name__}) is not a GradientTransformation')
        self.impl = impl
        self.optim_state = None  # built from the parameters on the first step
        self.inplace = bool(inplace)

    def step(self, loss: torch.Tensor, params, inplace: bool | None = None):
        """Differentiate `loss` with respect to `params`, update, return the new parameters."""
        if self.optim_state is None:
            self.optim_state = self.impl.init(params)
        if inplace is None:
            inplace = self.inplace
        leaves, spec = pytree.tree_flatten(params)
        live = [p for p in leaves if p is not None]
        taken = iter(torch.autograd.grad(loss, live, create_graph=True, allow_unused=True))
        grads = pytree.tree_unflatten([None if p is None else next(taken) for p in leaves], spec)
        updates, self.optim_state = self.impl.update(grads, self.optim_state, params=params,
                                                     inplace=inplace)
        return alias.apply_updates(params, updates, inplace=inplace)

    def state_dict(self):
        """The state itself, not a copy: in-place changes show up in the optimizer."""
        return self.optim_state

    def load_state_dict(self, state_dict) -> None:
        self.optim_state = state_dict
