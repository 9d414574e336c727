"""`FusedAdam` / `FusedAdamW`: the classic `Adam(..., use_accelerated_op=True)` and `AdamW`
optimizers with their whole step -- sign flip, weight decay, Adam scaling, multiplication by -lr
and the addition to the parameters -- in one pass over memory.

Counterparts of /root/reference/torchopt/optim/adam.py:43-92 and optim/adamw.py on top of
/root/reference/torchopt/optim/base.py:30-135.  What `step()` leaves in the parameters and in the moments is
bit-identical to the reference chain (`flip_sign_and_add_weight_decay` ->
`scale_by_accelerated_adam` [-> `add_decayed_weights`] -> `scale(-lr)` -> `apply_updates`, all in
place); the differences are mechanical:

  * one multi-tensor launch per hundred-odd parameters instead of three passes per parameter
    (28 instead of 44 bytes of HBM traffic per float32 element);
  * `p.grad` is left untouched (the reference's in-place chain overwrites it with the update);
  * the step count lives on the host; the 0-dim device tensors the state carries are brought up
    to date when the state is asked for (`state_dict()`);
  * a learning-rate schedule (a callable of the step count) is evaluated on the host with the
    integer number of steps already taken, as `scale_by_schedule` feeds it the count before the
    increment (/root/reference/torchopt/transform/scale_by_schedule.py:93-123); the reference
    hands the schedule a 0-dim device tensor, so a schedule that computes in tensor arithmetic
    there may round the rate differently in the last place.

State per parameter group is a `ScaleByAdamState(mu, nu, count)` of tuples, as the
transformation's own state, so it can be handed to `scale_by_accelerated_adam(...).update`.

`capturable=True` (the name `torch.optim.Adam` uses) keeps the step number where the reference
keeps it, in a device tensor (/root/reference/torchopt/transform/scale_by_adam.py:401-414), and
nowhere else: `step()` advances it with a one-thread kernel and the fused step reads it when it
starts, picking its bias corrections from a table the host filled once (in double with libm's
`pow`, as the reference's launchers compute them, so results stay bit-identical).  One HIP graph
captured around `step()` then serves the whole training loop: every replay is the next step.
Without it a captured `step()` would replay the step number it was captured with, so `step()`
refuses to run under capture.
"""

from __future__ import annotations

from itertools import repeat
from operator import is_
from typing import Callable, Iterable, Sequence

import torch

from torchopt_amd.accelerated_op.adam_op import adam_op
from torchopt_amd.base import accelerated_only
from torchopt_amd.placement import placed_like_tree, state_zeros_like_tree
from torchopt_amd.transform.scale_by_adam import (INT64_MAX, ScaleByAdamState, _host_value,
                                                 _remember)


__all__ = ['Adam', 'AdamW', 'FusedAdam', 'FusedAdamW']


class FusedAdam:
    """Classic Adam with the fused single-pass step (GPU tensors; float32 / float64, and float16 /
    bfloat16 without weight decay).  `weight_decay` is the L2 kind: added to the gradient before
    the moments."""

    _decoupled = False
    _mask = None  # FusedAdamW: which parameters decay

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float | Callable[[int], float] = 1e-3,
        betas: tuple[float, float] = (0.9, 0.999),
        eps: float = 1e-8,
        weight_decay: float = 0.0,
        *,
        eps_root: float = 0.0,
        maximize: bool = False,
        use_accelerated_op: bool = True,
        capturable: bool = False,
    ) -> None:
        # `use_accelerated_op` is accepted so that the reference's constructor calls carry over
        # (optim/adam.py:56-65); the fused operator is the only path here, and False warns
        accelerated_only(use_accelerated_op, type(self).__name__)
        if not callable(lr) and not lr >= 0.0:
            raise ValueError(f'Invalid learning rate: {lr}')
        if not eps >= 0.0:
            raise ValueError(f'Invalid epsilon value: {eps}')
        b1, b2 = betas
        if not 0.0 <= b1 < 1.0:
            raise ValueError(f'Invalid beta parameter at index 0: {b1}')
        if not 0.0 <= b2 < 1.0:
            raise ValueError(f'Invalid beta parameter at index 1: {b2}')
        if not weight_decay >= 0.0:
            raise ValueError(f'Invalid weight_decay value: {weight_decay}')
        self.lr, self.b1, self.b2, self.eps, self.weight_decay = lr, b1, b2, eps, weight_decay
        self.eps_root, self.maximize = eps_root, maximize
        self.capturable = bool(capturable)
        if self.capturable:
            if callable(lr):
                raise ValueError('capturable=True needs a constant learning rate: a schedule is '
                                 'evaluated on the host, which a captured graph would freeze')
            rows = adam_op.bias_rows_needed(b1, b2, 1, _MAX_BIAS_ROWS)
            if rows == 0:
                raise ValueError(
                    f'capturable=True: the bias corrections of betas={betas} take more than '
                    f'{_MAX_BIAS_ROWS} steps to settle, too many to tabulate')
            self._bias_rows_needed = rows
        self._bias_tables: dict[tuple, torch.Tensor] = {}  # (device, dtype) -> (rows, 4) table
        self.param_groups: list[tuple[torch.Tensor, ...]] = []
        self.state_groups: list[ScaleByAdamState | None] = []
        self._kinds: list[list[tuple]] = []       # (device, dtype) per parameter
        self._decays: list[list[bool]] = []       # whether weight decay applies, per parameter
        self._steps: list[list[int] | None] = []  # host-side step numbers per parameter
        self._stale: list[bool] = []              # device count tensors lag the host numbers
        self._uniform: list[bool] = []            # the group's parameters form one bucket
        self.add_param_group(params)

    def add_param_group(self, params: Iterable[torch.Tensor]) -> None:
        group = tuple(params)
        for p in group:
            if not isinstance(p, torch.Tensor):
                raise TypeError(f'expected tensors, got {type(p).__name__}')
        self.param_groups.append(group)
        self.state_groups.append(None)  # built on the first step, like the reference
        self._kinds.append([(p.device, p.dtype) for p in group])
        mask = self._mask(group) if callable(self._mask) else self._mask
        self._decays.append([True] * len(group) if mask is None else [bool(m) for m in mask])
        if len(self._decays[-1]) != len(group):
            raise ValueError('mask and parameters differ in length')
        if self.weight_decay != 0.0:
            for p, decays in zip(group, self._decays[-1]):
                if decays and p.dtype in (torch.float16, torch.bfloat16):
                    # the chain this step reproduces applies decay with Tensor.add_(p, alpha=wd),
                    # which on 16-bit CPU tensors is not one arithmetic (vectorized body and
                    # scalar tails round differently): there is no result to be identical to
                    raise ValueError(f'{type(self).__name__}: weight decay is served for float32 '
                                     f'and float64 parameters only, got {p.dtype}')
        self._steps.append(None)
        self._stale.append(False)
        # one bucket for the whole group: a single (device, dtype) and a single decay flag
        self._uniform.append(len(group) > 0 and len(set(self._kinds[-1])) == 1
                             and len(set(self._decays[-1])) == 1)

    def zero_grad(self, set_to_none: bool = False) -> None:
        for group in self.param_groups:
            for p in group:
                if set_to_none:
                    p.grad = None
                elif p.grad is not None:
                    if p.grad.grad_fn is not None:
                        p.grad.detach_()
                    else:
                        p.grad.requires_grad_(False)
                    p.grad.zero_()

    def state_dict(self) -> tuple:
        """Per group a `ScaleByAdamState` (or None before the first step)."""
        for i in range(len(self.state_groups)):
            self._sync_counts(i)
        return tuple(self.state_groups)

    def load_state_dict(self, state_dict: Sequence) -> None:
        """Takes the state of `state_dict()` back (as /root/reference/torchopt/optim/base.py:130-135
        does).  Large moments that do not lie where this package's own init would have put them
        -- state that went through `torch.save` / `torch.load`, or came from another process --
        are copied to that placement once, here, so that the steps after a restart stream as
        fast as the steps before it; values are untouched."""
        groups = []
        for s in state_dict:
            if s is not None:
                mu, nu = placed_like_tree(s.mu, s.nu)
                s = s._replace(mu=tuple(mu), nu=tuple(nu))
            groups.append(s)
        self.state_groups[:] = groups
        self._steps = [None if s is None else [_host_value(c) for c in s.count]
                       for s in self.state_groups]
        self._stale = [False] * len(self.state_groups)
        if self.capturable:
            # the leaves of one device step together from one shared count tensor
            for i, s in enumerate(self.state_groups):
                if s is None:
                    continue
                shared: dict[torch.device, torch.Tensor] = {}
                for c, v in zip(s.count, self._steps[i]):
                    if c.device not in shared:
                        shared[c.device] = torch.full((), v, dtype=torch.int64, device=c.device)
                    elif int(shared[c.device]) != v:
                        raise ValueError('capturable=True needs the parameters of a group on one '
                                         'device to share one step count')
                self.state_groups[i] = s._replace(count=tuple(shared[c.device] for c in s.count))

    def _init_state(self, i: int) -> ScaleByAdamState:
        group = self.param_groups[i]
        if self.capturable:
            # one count tensor per device, shared by that device's leaves: they step together
            shared = {}
            for p in group:
                if p.device not in shared:
                    shared[p.device] = torch.zeros(1, dtype=torch.int64, device=p.device).squeeze_()
            count = tuple(shared[p.device] for p in group)
        else:
            count = tuple(_remember(torch.zeros(1, dtype=torch.int64, device=p.device).squeeze_(),
                                    0) for p in group)
        self._steps[i] = [0] * len(group)
        self._stale[i] = False
        mu, nu = state_zeros_like_tree(group)
        return ScaleByAdamState(mu=tuple(mu), nu=tuple(nu), count=count)

    def _sync_counts(self, i: int) -> None:
        """Bring the 0-dim device count tensors of group `i` up to the host's step numbers.
        `step()` advances only the host numbers; the tensors are rebuilt (one upload per
        device) when somebody asks for the state."""
        if not self._stale[i] or self.capturable:
            return
        state, steps = self.state_groups[i], self._steps[i]
        by_device: dict[torch.device, list[int]] = {}
        for k, c in enumerate(state.count):
            by_device.setdefault(c.device, []).append(k)
        counts = list(state.count)
        for device, ks in by_device.items():
            fresh = torch.tensor([steps[k] for k in ks], dtype=torch.int64, device=device).unbind(0)
            for k, t in zip(ks, fresh):
                counts[k] = _remember(t, steps[k])
        self.state_groups[i] = state._replace(count=tuple(counts))
        self._stale[i] = False

    def _bias_table(self, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
        key = (device, dtype)
        if key not in self._bias_tables:
            host = adam_op.bias_rows(dtype, self.b1, self.b2, self.eps_root, 1,
                                     self._bias_rows_needed)
            self._bias_tables[key] = host.to(device)
        return self._bias_tables[key]

    def _step_on_device(self) -> None:
        """`step()` with the step numbers on the device: nothing here depends on their values,
        so a HIP graph captured around it replays as the following steps."""
        capturing = torch.cuda.is_current_stream_capturing()
        for i, group in enumerate(self.param_groups):
            if self.state_groups[i] is None:
                if capturing:
                    raise RuntimeError('FusedAdam: take one step (or call init_state()) before '
                                       'capturing, so that the state exists outside the graph')
                self.state_groups[i] = self._init_state(i)
            state = self.state_groups[i]
            grads = [p.grad for p in group]
            if all(g is None for g in grads):
                continue
            if any(g is None for g in grads):
                raise RuntimeError('FusedAdam(capturable=True): every parameter of a group must '
                                   'have a gradient at every step (they share one step count)')
            buckets: dict[tuple, list[int]] = {}
            for k in range(len(group)):
                buckets.setdefault((self._kinds[i][k], self._decays[i][k]), []).append(k)
            tables = {kind: self._bias_table(*kind) for kind, _ in buckets}  # before any launch
            advanced = set()
            for c in state.count:
                if id(c) not in advanced:
                    advanced.add(id(c))
                    adam_op.count_advance_(c)
            for (kind, decays), ks in buckets.items():
                whole = len(ks) == len(group)
                adam_op.fused_step_multi_devcount_(
                    list(group) if whole else [group[k] for k in ks],
                    grads if whole else [grads[k] for k in ks],
                    list(state.mu) if whole else [state.mu[k] for k in ks],
                    list(state.nu) if whole else [state.nu[k] for k in ks],
                    self.b1, self.b2, self.eps, self.eps_root, tables[kind], 1,
                    state.count[ks[0]], self.lr, maximize=self.maximize, write_updates=False,
                    weight_decay=self.weight_decay if decays else 0.0,
                    decoupled=self._decoupled)
            self._steps[i] = None  # the device holds the step numbers now

    def init_state(self) -> None:
        """Create the moments and step counts now (they are otherwise created by the first
        `step()`), e.g. before capturing `step()` in a graph."""
        for i in range(len(self.param_groups)):
            if self.state_groups[i] is None:
                self.state_groups[i] = self._init_state(i)
                if self.capturable:
                    for p in self.param_groups[i]:
                        self._bias_table(p.device, p.dtype)

    @torch.no_grad()
    def step(self, closure: Callable[[], torch.Tensor] | None = None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if self.capturable:
            self._step_on_device()
            return loss
        if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                'FusedAdam.step() under stream capture would bake the current step number (and '
                'its bias corrections) into the graph, and every replay would repeat that step. '
                'Construct the optimizer with capturable=True to keep the step number on the '
                'device, or call torchopt_amd._C.adam_op.fused_step_multi_ yourself with the '
                'count you mean to freeze.')
        scheduled = callable(self.lr)
        for i, group in enumerate(self.param_groups):
            if self.state_groups[i] is None:
                self.state_groups[i] = self._init_state(i)
            state, steps = self.state_groups[i], self._steps[i]
            grads = [p.grad for p in group]
            if (self._uniform[i] and not scheduled and steps.count(steps[0]) == len(steps)
                    and not any(map(is_, grads, repeat(None)))):
                # the usual step in one go: every parameter has a gradient, the group is one
                # bucket (one device and type, one decay flag) and has stepped together so far
                c = steps[0]
                if c != INT64_MAX:
                    c += 1
                    steps[:] = [c] * len(steps)
                self._stale[i] = True
                adam_op.fused_step_multi_(
                    list(group), grads, list(state.mu), list(state.nu), self.b1, self.b2,
                    self.eps, self.eps_root, c, self.lr, maximize=self.maximize,
                    write_updates=False,
                    weight_decay=self.weight_decay if self._decays[i][0] else 0.0,
                    decoupled=self._decoupled)
                continue
            live = [k for k, g in enumerate(grads) if g is not None]
            if not live:
                continue
            for k in live:
                if steps[k] != INT64_MAX:
                    steps[k] += 1
            self._stale[i] = True
            buckets: dict[tuple, list[int]] = {}
            for k in live:
                # a schedule makes the rate depend on the leaf's own step count
                key = (self._kinds[i][k], steps[k] if scheduled else None, self._decays[i][k])
                buckets.setdefault(key, []).append(k)
            for key, ks in buckets.items():
                vals = [steps[k] for k in ks]
                counts = vals[0] if vals.count(vals[0]) == len(vals) else vals
                lr = float(self.lr(vals[0] - 1)) if scheduled else self.lr
                whole = len(ks) == len(group)
                adam_op.fused_step_multi_(
                    list(group) if whole else [group[k] for k in ks],
                    grads if whole else [grads[k] for k in ks],
                    list(state.mu) if whole else [state.mu[k] for k in ks],
                    list(state.nu) if whole else [state.nu[k] for k in ks],
                    self.b1, self.b2, self.eps, self.eps_root, counts, lr,
                    maximize=self.maximize, write_updates=False,
                    weight_decay=self.weight_decay if key[2] else 0.0,
                    decoupled=self._decoupled)
        return loss


class FusedAdamW(FusedAdam):
    """Classic AdamW with the fused single-pass step: `weight_decay` is decoupled, added to the
    Adam-scaled update (/root/reference/torchopt/alias/adamw.py:140-151)."""

    _decoupled = True

    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2, *, eps_root: float = 0.0, mask=None,
                 maximize: bool = False, use_accelerated_op: bool = True,
                 capturable: bool = False) -> None:
        # `mask`: a sequence of booleans, one per parameter, or a callable that makes one from
        # the parameters; False exempts a parameter from the decay (optim/adamw.py:60-63)
        self._mask = mask
        super().__init__(params, lr, betas, eps, weight_decay, eps_root=eps_root,
                         maximize=maximize, use_accelerated_op=use_accelerated_op,
                         capturable=capturable)


# Most rows a bias-correction table may have (16 bytes per float32 row): enough for b2 up to
# 0.99999, whose corrections settle after 3.7 million steps.
_MAX_BIAS_ROWS = 1 << 22


# the reference's class names (torchopt.Adam / torchopt.AdamW)
Adam = FusedAdam
AdamW = FusedAdamW
