"""Availability probe of the accelerated Adam operator
(counterpart of /root/reference/torchopt/accelerated_op/__init__.py:30-50)."""

from __future__ import annotations

from typing import Iterable, Union

import torch

from torchopt_amd.accelerated_op.adam_op import AdamOp, MultiAdamOp

__all__ = ['AdamOp', 'MultiAdamOp', 'is_available']

Device = Union[torch.device, str, int]


def is_available(devices: Device | Iterable[Device] | None = None) -> bool:
    """True iff the fused op runs on every device asked about.

    As in the reference, the probe really runs the op: a 0-dim fp32 tensor passed as mu, nu
    and updates at once with count 1, and any exception means "not available".  With no
    argument the reference asks about ``cuda`` and ``cpu``; this build serves GPUs only, so
    the default asks about ``cuda`` alone, and asking about ``cpu`` (or ``meta``, ...)
    answers False.
    """
    if devices is None:
        devices = [torch.device('cuda')]
    elif isinstance(devices, (torch.device, int, str)):
        devices = [devices]

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
