"""`MetaAdam`: the differentiable optimizer the fused operator exists for.

Counterpart of /root/reference/torchopt/optim/meta/adam.py:43-92 on
/root/reference/torchopt/optim/meta/base.py:36-114: ``step(loss)`` takes gradients with
``create_graph=True``, runs the Adam chain out of place, and replaces the module's parameters
with the (non-leaf) results, so an outer loss can be differentiated through any number of inner
steps.  On the fused operator one inner step costs two launches for the whole module.
"""

from __future__ import annotations

from typing import Sequence

import torch
from torch import nn

from torchopt_amd import alias
from torchopt_amd.base import accelerated_only


__all__ = ['MetaAdam', 'MetaAdamW']


class _MetaOptimizer:
    def __init__(self, module: nn.Module, impl) -> None:
        if not isinstance(module, nn.Module):
            raise RuntimeError(f'Unexpected class of {module}')
        self.impl = impl
        self.param_containers_groups: list[tuple[dict, ...]] = []
        self.state_groups: list = []
        self.add_param_group(module)

    def add_param_group(self, module: nn.Module) -> None:
        # references to the modules' own parameter dictionaries (base.py:98-102 via
        # /root/reference/torchopt/utils.py:278-306)
        seen, containers = set(), []
        for sub in module.modules():
            if sub not in seen and len(sub._parameters) > 0:
                containers.append(sub._parameters)
            seen.add(sub)
        self.param_containers_groups.append(tuple(containers))
        self.state_groups.append(None)

    def step(self, loss: torch.Tensor) -> None:
        """One differentiable update of every parameter from `loss`."""
        for i, (containers, state) in enumerate(zip(self.param_containers_groups,
                                                    self.state_groups)):
            keys = [(c, k) for c in containers for k in c]
            flat_params = tuple(c[k] for c, k in keys)
            if state is None:
                state = self.impl.init(flat_params)
            live = [p for p in flat_params if p is not None]
            grads = iter(torch.autograd.grad(loss, live, create_graph=True, allow_unused=True))
            flat_grads = tuple(None if p is None else next(grads) for p in flat_params)
            updates, new_state = self.impl.update(flat_grads, state, params=flat_params,
                                                  inplace=False)
            self.state_groups[i] = new_state
            new_params = alias.apply_updates(flat_params, updates, inplace=False)
            for (c, k), new in zip(keys, new_params):
                c[k] = new

    def state_dict(self) -> tuple:
        return tuple(self.state_groups)

    def load_state_dict(self, state_dict: Sequence) -> None:
        self.state_groups[:] = list(state_dict)


class MetaAdam(_MetaOptimizer):
    """Differentiable Adam over a module's parameters."""

    def __init__(self, module: nn.Module, lr=1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 0.0, *, eps_root: float = 0.0,
                 moment_requires_grad: bool = True, maximize: bool = False,
                 use_accelerated_op: bool = True) -> None:
        accelerated_only(use_accelerated_op, 'MetaAdam')
        super().__init__(module, alias.adam(lr, betas, eps, weight_decay, eps_root=eps_root,
                                            moment_requires_grad=moment_requires_grad,
                                            maximize=maximize))


class MetaAdamW(_MetaOptimizer):
    """Differentiable AdamW over a module's parameters."""

    def __init__(self, module: nn.Module, lr=1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2, *, eps_root: float = 0.0, mask=None,
                 moment_requires_grad: bool = False, maximize: bool = False,
                 use_accelerated_op: bool = True) -> None:
        accelerated_only(use_accelerated_op, 'MetaAdamW')
        super().__init__(module, alias.adamw(lr, betas, eps, weight_decay, eps_root=eps_root,
                                             mask=mask,
                                             moment_requires_grad=moment_requires_grad,
                                             maximize=maximize))
