"""``AdamOp``: the callable the Adam transformation applies to every leaf.

Counterpart of /root/reference/torchopt/accelerated_op/adam_op.py:33-181, bound to
``torchopt_amd._C.adam_op`` (hand-written gfx950 kernels) and to nothing else: there is no
pure-PyTorch fallback module behind it.

Contract kept from the reference:
  * ``AdamOp(b1, b2, eps, *, eps_root, inplace)(mu, nu, updates, count)`` returns
    ``(new_mu, new_nu, new_updates)``; ``updates is None`` returns ``(mu, nu, None)``
    untouched (:148-149);
  * ``inplace=True`` runs the fused ``forward_`` which overwrites all three tensors (:156-166);
  * ``inplace=False`` chains three autograd Functions -- ``MuOp``, ``NuOp``, ``UpdatesOp`` --
    whose backward passes call ``backward_mu`` / ``backward_nu`` / ``backward_updates`` with
    the tensors the reference saves (:36-121), so outer-loop gradients flow through the step;
  * non-tensor arguments (decay rates, the hyper-parameter tuple) get ``None`` gradients.
"""

from __future__ import annotations

from typing import Any

import torch

try:
    from torchopt_amd._C import adam_op
except ImportError as exc:  # no fallback module: the op is the compiled extension or nothing
    raise ImportError(
        'torchopt_amd._C, the compiled extension in front of libtoa_adam.so, cannot be '
        f'imported ({exc}); build it with `python torchopt_amd/build.py`. There is no '
        'pure-Python or CPU fallback.') from exc

# the same seven functions, visible to torch.compile while it traces (see library.py)
from torchopt_amd.accelerated_op.library import dispatch  # noqa: E402


class AdamOp:
    """Fused Adam scaling of one leaf: moments update plus bias-corrected step direction."""

    class MuOp(torch.autograd.Function):
        """First moment: ``new_mu = b1*mu + (1-b1)*updates``."""

        @staticmethod
        def forward(ctx: Any, updates: torch.Tensor, mu: torch.Tensor, b1: float) -> torch.Tensor:
            ctx.save_for_backward(updates, mu)
            ctx.b1 = b1
            return dispatch.forward_mu(updates, mu, b1)

        @staticmethod
        def backward(ctx: Any, dmu: torch.Tensor):
            updates, mu = ctx.saved_tensors
            dupdates, dmu_in = dispatch.backward_mu(dmu, updates, mu, ctx.b1)
            return dupdates, dmu_in, None

    class NuOp(torch.autograd.Function):
        """Second raw moment: ``new_nu = b2*nu + (1-b2)*updates**2``."""

        @staticmethod
        def forward(ctx: Any, updates: torch.Tensor, nu: torch.Tensor, b2: float) -> torch.Tensor:
            ctx.save_for_backward(updates, nu)
            ctx.b2 = b2
            return dispatch.forward_nu(updates, nu, b2)

        @staticmethod
        def backward(ctx: Any, dnu: torch.Tensor):
            updates, nu = ctx.saved_tensors
            dupdates, dnu_in = dispatch.backward_nu(dnu, updates, nu, ctx.b2)
            return dupdates, dnu_in, None

    class UpdatesOp(torch.autograd.Function):
        """Step direction ``mu_hat / (sqrt(nu_hat + eps_root) + eps)``; its backward is the
        reference's hand-derived formula, which needs the forward output."""

        @staticmethod
        def forward(ctx: Any, new_mu: torch.Tensor, new_nu: torch.Tensor, hyper: tuple):
            b1, b2, eps, eps_root, count = hyper
            new_updates = dispatch.forward_updates(new_mu, new_nu, b1, b2, eps, eps_root, count)
            ctx.save_for_backward(new_updates, new_mu, new_nu)
            ctx.hyper = hyper
            return new_updates

        @staticmethod
        def backward(ctx: Any, dupdates: torch.Tensor):
            new_updates, new_mu, new_nu = ctx.saved_tensors
            b1, b2, _eps, eps_root, count = ctx.hyper
            dnew_mu, dnew_nu = dispatch.backward_updates(
                dupdates, new_updates, new_mu, new_nu, b1, b2, eps_root, count)
            return dnew_mu, dnew_nu, None

    def __init__(
        self,
        b1: float = 0.9,
        b2: float = 0.999,
        eps: float = 1e-8,
        *,
        eps_root: float = 0.0,
        inplace: bool = True,
    ) -> None:
        self.b1 = b1
        self.b2 = b2
        self.eps = eps
        self.eps_root = eps_root
        self.inplace = inplace

    def __call__(self, mu, nu, updates, count):
        if updates is None:
            return mu, nu, None
        if self.inplace:
            # forward_ hands back [updates, mu, nu]; callers want (mu, nu, updates)
            new_updates, new_mu, new_nu = dispatch.forward_(
                updates, mu, nu, self.b1, self.b2, self.eps, self.eps_root, count)
            return new_mu, new_nu, new_updates
        new_mu = self.MuOp.apply(updates, mu, self.b1)
        new_nu = self.NuOp.apply(updates, nu, self.b2)
        hyper = (self.b1, self.b2, self.eps, self.eps_root, count)
        new_updates = self.UpdatesOp.apply(new_mu, new_nu, hyper)
        return new_mu, new_nu, new_updates


class MultiAdamOp:
    """`AdamOp` over whole lists of leaves.

    The reference applies `AdamOp` leaf by leaf from Python
    (/root/reference/torchopt/transform/scale_by_adam.py:325-332): one launch, and on the
    differentiable path three autograd nodes with three forward and three backward launches,
    per leaf.  This callable takes the flattened tree at once: the in-place branch is one
    `forward_multi_` call, and the differentiable branch is ONE autograd node whose forward
    (`forward_all_multi`) and backward (`backward_all_multi`) are one multi-tensor pass each, so
    a tree of any size costs two launches per step instead of six per leaf, and each direction
    reads its operands once.  Values and gradients are bit-identical to the per-leaf `AdamOp`.
    The node lives in the extension module (`adam_op.step_multi`, a C++ autograd node: no
    Python runs between autograd's engine and the launches); `StepOp` below is the same node
    written in Python, the route taken while `torch.compile` traces.

    All lists must be free of ``None`` and live on one device with one dtype; the caller groups
    leaves accordingly.  `counts` is one step number for all leaves or one per leaf (ints or
    0-dim integer tensors).
    """

    class StepOp(torch.autograd.Function):
        """(updates, mu, nu) -> (new_mu, new_nu, new_updates) for every leaf."""

        @staticmethod
        def forward(ctx: Any, hyper: tuple, k: int, *tensors: torch.Tensor):
            b1, b2, eps, eps_root, counts = hyper
            updates = list(tensors[:k])
            new_mu, new_nu, new_updates = adam_op.forward_all_multi(
                updates, list(tensors[k:2 * k]), list(tensors[2 * k:]), b1, b2, eps, eps_root,
                counts)
            ctx.save_for_backward(*new_updates, *new_mu, *updates)
            ctx.hyper, ctx.k = hyper, k
            ctx.set_materialize_grads(False)  # a missing gradient must stay missing, see below
            return (*new_mu, *new_nu, *new_updates)

        @staticmethod
        def backward(ctx: Any, *grads: torch.Tensor | None):
            saved, k = ctx.saved_tensors, ctx.k
            b1, b2, _eps, eps_root, counts = ctx.hyper
            new_updates, new_mu, updates = saved[:k], saved[k:2 * k], saved[2 * k:]
            g_mu, g_nu, g_u = grads[:k], grads[k:2 * k], grads[2 * k:]
            dupdates: list = [None] * k
            dmu: list = [None] * k
            dnu: list = [None] * k

            def pick(seq, idx):
                return [seq[i] for i in idx]

            def counts_of(idx):
                return pick(counts, idx) if isinstance(counts, (list, tuple)) else counts

            # Leaves whose new_updates received a gradient: the one-pass backward.
            live = [i for i in range(k) if g_u[i] is not None]
            if live:
                def outside(gs):
                    # Gradients reaching new_mu / new_nu from outside the step.  None at all:
                    # the kernel skips the addition, as autograd would.  Some: members without
                    # one get -0.0, the exact identity of IEEE addition (x + -0.0 is x for every
                    # x, signed zeros included), so they too come out as if nothing was added.
                    gs = pick(gs, live)
                    if all(g is None for g in gs):
                        return None
                    return [torch.full_like(new_mu[i], -0.0) if g is None else g
                            for g, i in zip(gs, live)]

                du, dm, dn = adam_op.backward_all_multi(
                    pick(g_u, live), outside(g_mu), outside(g_nu), pick(new_updates, live),
                    pick(new_mu, live), pick(updates, live), b1, b2, eps_root, counts_of(live))
                for j, i in enumerate(live):
                    dupdates[i], dmu[i], dnu[i] = du[j], dm[j], dn[j]

            # Leaves whose new_updates received none: the per-leaf chain never runs
            # backward_updates for them, so nothing of new_updates / new_mu (which may hold
            # infinities) enters; only the outside gradients flow on through backward_mu and
            # backward_nu, and a leaf with neither gets no gradient at all.
            dead = [i for i in range(k) if g_u[i] is None]
            via_mu = [i for i in dead if g_mu[i] is not None]
            via_nu = [i for i in dead if g_nu[i] is not None]
            if via_mu:
                du, dm = adam_op.backward_mu_multi(pick(g_mu, via_mu), pick(updates, via_mu),
                                                   pick(updates, via_mu), b1)
                for j, i in enumerate(via_mu):
                    dupdates[i], dmu[i] = du[j], dm[j]
            if via_nu:
                du, dn = adam_op.backward_nu_multi(pick(g_nu, via_nu), pick(updates, via_nu),
                                                   pick(updates, via_nu), b2)
                for j, i in enumerate(via_nu):
                    # autograd adds the two contributions to d(updates) where both exist
                    dupdates[i] = du[j] if dupdates[i] is None else dupdates[i] + du[j]
                    dnu[i] = dn[j]
            return (None, None, *dupdates, *dmu, *dnu)

    # False routes the differentiable branch through the Python `StepOp` even outside
    # `torch.compile` (the tests hold both routes to the per-leaf chain)
    use_native_node = True

    def __init__(
        self,
        b1: float = 0.9,
        b2: float = 0.999,
        eps: float = 1e-8,
        *,
        eps_root: float = 0.0,
        inplace: bool = True,
    ) -> None:
        self.b1 = b1
        self.b2 = b2
        self.eps = eps
        self.eps_root = eps_root
        self.inplace = inplace

    def __call__(self, mus, nus, updates, counts):
        """Returns ``(new_mus, new_nus, new_updates)`` as lists."""
        mus, nus, updates = list(mus), list(nus), list(updates)
        k = len(updates)
        if k == 0:
            return [], [], []
        if self.inplace:
            adam_op.forward_multi_(updates, mus, nus, self.b1, self.b2, self.eps, self.eps_root,
                                   counts)
            return mus, nus, updates
        if self.use_native_node and not torch.compiler.is_compiling():
            return adam_op.step_multi(updates, mus, nus, self.b1, self.b2, self.eps,
                                      self.eps_root, counts)
        hyper = (self.b1, self.b2, self.eps, self.eps_root, counts)
        out = self.StepOp.apply(hyper, k, *updates, *mus, *nus)
        return list(out[:k]), list(out[k:2 * k]), list(out[2 * k:])
