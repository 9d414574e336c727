"""Where optimizer state goes in device memory.

The reference's ``init_fn`` makes its moments with ``zeros_like``
(/root/reference/torchopt/transform/scale_by_adam.py:401-414) and gets whatever address the
allocator hands out: for a large tensor a block on a 2 MiB boundary, so gradient, mu and nu share
their address modulo 16 KiB.  The in-place step streams all three at once, and on MI355X its rate
moves with how those streams fall on the memory channels: with the two moments 8 KiB off the
gradient's phase the float32 step on 2^28 elements runs 0.8-1.0 % faster, 4 and 12 KiB are the
slow distances, and nothing measured is slower at 8 KiB than at 0.  The state this package
allocates therefore starts at that phase (``toa_adam_state_shift`` of the C ABI names it);
values, shapes, dtypes and contiguity are those of ``zeros_like``.
"""

from __future__ import annotations

import torch

from torchopt_amd import _lib

# below this a tensor shares allocator blocks with its neighbours at 512-byte granularity, its
# phase is anybody's, and 16 KiB of slack would be a visible share of it
MIN_BYTES = 1 << 20


def _placed(t: torch.Tensor, zero: bool, requires_grad: bool) -> torch.Tensor:
    size = t.numel() * t.element_size()
    if (not t.is_cuda or size < MIN_BYTES or not t.is_contiguous()
            or t.layout != torch.strided):
        make = torch.zeros_like if zero else torch.empty_like
        return make(t, requires_grad=requires_grad)
    lib = _lib.load()
    slack = lib.toa_adam_state_slack() // t.element_size()
    make = torch.zeros if zero else torch.empty
    block = make(t.numel() + slack, dtype=t.dtype, device=t.device)
    skip = lib.toa_adam_state_shift(block.data_ptr()) // t.element_size()
    out = block[skip:skip + t.numel()].view(t.shape)
    return out.requires_grad_(requires_grad)


def state_zeros_like(t: torch.Tensor, *, requires_grad: bool = False) -> torch.Tensor:
    """``zeros_like(t)`` at the preferred phase (a view into a slightly larger block when `t` is
    a contiguous GPU tensor of 1 MiB or more, plain ``zeros_like`` otherwise)."""
    return _placed(t, True, requires_grad)


def state_empty_like(t: torch.Tensor, *, requires_grad: bool = False) -> torch.Tensor:
    """``empty_like(t)`` at the preferred phase."""
    return _placed(t, False, requires_grad)
