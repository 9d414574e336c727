"""Availability probe of the accelerated Adam operator
(counterpart of /root/reference/torchopt/accelerated_op/__init__.py:30-50)."""

from __future__ import annotations

import warnings
from typing import Iterable, Union

import torch

from torchopt_amd.accelerated_op.adam_op import AdamOp, MultiAdamOp

__all__ = ['AdamOp', 'MultiAdamOp', 'is_available']

Device = Union[torch.device, str, int]

_warned_default = False


def is_available(devices: Device | Iterable[Device] | None = None) -> bool:
    """True iff the fused op runs on every device asked about.

    As in the reference, the probe really runs the op: a 0-dim fp32 tensor passed as mu, nu
    and updates at once with count 1, and any exception means "not available".  With no
    argument the reference asks about ``cuda`` and ``cpu``
    (/root/reference/torchopt/accelerated_op/__init__.py:35-36); this build serves GPUs only, so
    the default asks about ``cuda`` alone and says so in a `UserWarning` (once per process), and
    asking about ``cpu`` answers False with a `UserWarning` naming the reason (``meta`` and other
    devices answer False silently, as in the reference).
    """
    global _warned_default
    if devices is None:
        if not _warned_default:
            _warned_default = True
            warnings.warn(
                'torchopt_amd.accelerated_op.is_available() without arguments asks about "cuda" '
                'only: this build has no CPU kernels (TorchOpt asks about "cuda" and "cpu").',
                UserWarning, stacklevel=2)
        devices = [torch.device('cuda')]
    elif isinstance(devices, (torch.device, int, str)):
        devices = [devices]
    try:
        devices = [torch.device(dev) for dev in devices]
    except Exception:  # noqa: BLE001 - not a device: not available
        return False
    if any(dev.type == 'cpu' for dev in devices):
        warnings.warn(
            'torchopt_amd has no CPU kernels: is_available() answers False for "cpu", where '
            'TorchOpt, which ships a CPU implementation of the operator, answers True.',
            UserWarning, stacklevel=2)
        return False

    op = AdamOp()
    try:
        for dev in devices:
            dev = torch.device(dev)
            if dev.type == 'cuda' and not torch.cuda.is_available():
                return False
            probe = torch.tensor(1.0, device=dev)
            op(probe, probe, probe, 1)
    except Exception:  # noqa: BLE001 - the reference swallows everything here too
        return False
    return True
