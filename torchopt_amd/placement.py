"""Where optimizer state goes in device memory.

The reference's ``init_fn`` makes its moments with ``zeros_like``
(/root/reference/torchopt/transform/scale_by_adam.py:401-414) and gets whatever address the
allocator hands out: for a large tensor a block on a 2 MiB boundary, so gradient, mu and nu share
their address modulo 16 KiB.  The in-place step streams all three at once, and on MI355X its rate
moves with how those streams fall on the memory channels.  Measured on the float32 step over 2^28
elements: with the two moments 8 KiB apart modulo 16 KiB it runs at 85.0-85.8 % of the HBM peak
whatever the gradient's own phase (84.2-84.9 % with all three at one phase, as the allocator
leaves them; 84.0-85.7 % with both moments at one phase 8 KiB off, depending on the gradient's).
The state this package allocates therefore starts 8 KiB past a multiple of 16 KiB for first
moments and at a multiple of 16 KiB for second moments (``toa_adam_state_shift`` of the C ABI
names the phases); values, shapes, dtypes and contiguity are those of ``zeros_like``.

A tree's moments come from ONE block per (device, dtype): every mu, then every nu, each leaf at
its phase, so the slack is 16 KiB per leaf instead of what the allocator's rounding would add to
separate blocks (2 MiB on a 16 MiB leaf), and a leaf's two moments lie a whole even number of MiB
between 4 and 12, plus those 8 KiB, apart modulo 16 MiB (8 MiB where that costs little): the
distances the step streams fastest at, and clear of the multiples of 16 MiB at which arrays meet
in the same DRAM banks.

What a caller can observe of this, beside the speed: the moments of such a tree are views into a
shared storage (non-zero ``storage_offset()``), so (a) ``torch.save`` of the whole state writes
the block once -- sharing is preserved in the file -- but saving ONE moment leaf on its own writes
the whole block (``unshared(t)`` gives a leaf a storage of its own first); (b) dropping or
replacing one leaf's state frees nothing while a sibling is alive; (c) state that comes back from
``torch.load`` (or from anywhere else) lies where the loader put it: `FusedAdam.load_state_dict`
and `placed_like_tree` move it to the preferred placement again, one copy per leaf.  Setting the
environment variable ``TORCHOPT_AMD_STATE_PLACEMENT=0`` (read at every allocation) switches all
of it off: every moment is then a plain ``zeros_like`` allocation, as in the reference.
"""

from __future__ import annotations

import os

import torch

from torchopt_amd import _lib

# below this a tensor shares allocator blocks with its neighbours at 512-byte granularity, its
# phase is anybody's, and 16 KiB of slack would be a visible share of it
MIN_BYTES = 1 << 20


def placement_enabled() -> bool:
    """False when TORCHOPT_AMD_STATE_PLACEMENT=0: state then comes from plain ``zeros_like``."""
    return os.environ.get('TORCHOPT_AMD_STATE_PLACEMENT', '1') != '0'


def _placed(t: torch.Tensor, zero: bool, requires_grad: bool, moment: int) -> torch.Tensor:
    size = t.numel() * t.element_size()
    if (not t.is_cuda or size < MIN_BYTES or not t.is_contiguous()
            or t.layout != torch.strided or not placement_enabled()):
        make = torch.zeros_like if zero else torch.empty_like
        return make(t, requires_grad=requires_grad)
    lib = _lib.load()
    slack = lib.toa_adam_state_slack() // t.element_size()
    make = torch.zeros if zero else torch.empty
    block = make(t.numel() + slack, dtype=t.dtype, device=t.device)
    skip = lib.toa_adam_state_shift(block.data_ptr(), moment) // t.element_size()
    out = block[skip:skip + t.numel()].view(t.shape)
    return out.requires_grad_(requires_grad)


def state_zeros_like(t: torch.Tensor, *, requires_grad: bool = False,
                     moment: int = 0) -> torch.Tensor:
    """``zeros_like(t)`` at the preferred phase of a first (``moment=0``) or second
    (``moment=1``) moment: a view into a slightly larger block when `t` is a contiguous GPU tensor
    of 1 MiB or more, plain ``zeros_like`` otherwise."""
    return _placed(t, True, requires_grad, moment)


def state_empty_like(t: torch.Tensor, *, requires_grad: bool = False,
                     moment: int = 0) -> torch.Tensor:
    """``empty_like(t)`` at the preferred phase of a first or second moment."""
    return _placed(t, False, requires_grad, moment)


# How far apart the two moments of a leaf lie inside the block, modulo 16 MiB.  Measured on the
# float32 step over 2^28 elements with both moments in one block (GB/s by distance beyond 1 GiB):
# 0 MiB 6812, 1 6716, 2 6790, 3 6668, 4 6836, 5 6650, 6 6827, 7 6733, 8 6856, 10 6838, 12 6837,
# 14 6805, 16 6785 -- whole even numbers of MiB from 4 to 12 are the fast ones, 8 the fastest,
# odd ones cost 2 %, and multiples of 16 MiB are where arrays collide in the same DRAM banks.
_DISTANCE_PERIOD = 16 << 20
_DISTANCES = (8 << 20, 10 << 20, 6 << 20, 12 << 20, 4 << 20)  # in order of preference


def _second_moment_offset(end: int, largest: int, period: int) -> int:
    """Where the second moments start, `end` being the size of the first moments' region: the
    nearest preferred distance that costs at most 1/32 of the region (2 MiB for small ones) in
    slack, else the cheapest preferred one (small leaves sit in cache: no distance to arrange) --
    plus the 8 KiB that put the second moments at their own phase."""
    second = -(-end // period) * period
    if largest >= (4 << 20):
        budget = max(2 << 20, end // 32)
        gaps = [(want - second) % _DISTANCE_PERIOD for want in _DISTANCES]
        within = [g for g in gaps if g <= budget]
        second += within[0] if within else min(gaps)
    return second + period // 2  # second moments half a period off the first moments' phase


def _eligible(t) -> bool:
    return (t is not None and t.is_cuda and t.layout == torch.strided and t.is_contiguous()
            and t.numel() * t.element_size() >= MIN_BYTES and placement_enabled())


def is_placed(t: torch.Tensor, moment: int) -> bool:
    """Does `t` start at the preferred address phase of a first (0) or second (1) moment?"""
    return _lib.load().toa_adam_state_shift(t.data_ptr(), moment) == 0


def unshared(t: torch.Tensor) -> torch.Tensor:
    """`t` itself if its storage holds nothing else, a copy with a storage of its own otherwise:
    what to hand to ``torch.save`` when ONE state leaf is to be written (a view into a tree's
    block would take the whole block along)."""
    if t.untyped_storage().nbytes() <= t.numel() * t.element_size() + 512:
        return t
    return t.detach().clone().requires_grad_(t.requires_grad)


def placed_like_tree(mu_leaves, nu_leaves):
    """The moments `mu_leaves`, `nu_leaves` of a flattened tree (``None`` leaves stay ``None``)
    at the placement `state_zeros_like_tree` would have given them: leaves that are eligible (GPU,
    contiguous, 1 MiB or more) and not already at their phases are copied into a fresh block,
    the others are returned as they are.  Values, shapes, dtypes and ``requires_grad`` are kept.
    For state that arrives from ``torch.load`` or another process."""
    mu_leaves, nu_leaves = list(mu_leaves), list(nu_leaves)
    move = [k for k, (m, v) in enumerate(zip(mu_leaves, nu_leaves))
            if _eligible(m) and v is not None and not (is_placed(m, 0) and is_placed(v, 1))]
    if not move:
        return mu_leaves, nu_leaves
    fresh_mu, fresh_nu = state_zeros_like_tree([mu_leaves[k] for k in move])
    with torch.no_grad():
        for k, m, v in zip(move, fresh_mu, fresh_nu):
            m.copy_(mu_leaves[k])
            v.copy_(nu_leaves[k])
            mu_leaves[k] = m.requires_grad_(mu_leaves[k].requires_grad)
            nu_leaves[k] = v.requires_grad_(nu_leaves[k].requires_grad)
    return mu_leaves, nu_leaves


def state_zeros_like_tree(leaves, *, requires_grad: bool = False):
    """``([zeros_like(t) for t in leaves], [zeros_like(t) for t in leaves])`` -- both moments of
    a flattened tree (``None`` leaves stay ``None``).  The large contiguous GPU leaves of one
    device and dtype share one block: all first moments, then all second moments, every leaf at
    the preferred phase.  Other leaves get plain ``zeros_like``."""
    leaves = list(leaves)
    mu = [None] * len(leaves)
    nu = [None] * len(leaves)
    groups: dict = {}
    for k, t in enumerate(leaves):
        if t is None:
            continue
        if _eligible(t):
            groups.setdefault((t.device, t.dtype), []).append(k)
        else:
            mu[k] = torch.zeros_like(t, requires_grad=requires_grad)
            nu[k] = torch.zeros_like(t, requires_grad=requires_grad)
    if not groups:
        return mu, nu
    lib = _lib.load()
    period = lib.toa_adam_state_slack()
    for (device, dtype), members in groups.items():
        es = leaves[members[0]].element_size()
        sizes = [leaves[k].numel() * es for k in members]
        # byte offsets from the first leaf's start, every leaf a whole number of periods on
        offsets, end = [], 0
        for n in sizes:
            end = -(-end // period) * period
            offsets.append(end)
            end += n
        second = _second_moment_offset(end, max(sizes), period)
        try:
            block = torch.zeros((second + end + period) // es, dtype=dtype, device=device)
        except torch.cuda.OutOfMemoryError:
            # no room for one block of that size: a block per moment and leaf, as zeros_like would
            for k in members:
                mu[k] = state_zeros_like(leaves[k], requires_grad=requires_grad, moment=0)
                nu[k] = state_zeros_like(leaves[k], requires_grad=requires_grad, moment=1)
            continue
        first = lib.toa_adam_state_shift(block.data_ptr(), 0)
        for k, off in zip(members, offsets):
            n, shape = leaves[k].numel(), leaves[k].shape
            a, b = (first + off) // es, (first + second + off) // es
            mu[k] = block[a:a + n].view(shape).requires_grad_(requires_grad)
            nu[k] = block[b:b + n].view(shape).requires_grad_(requires_grad)
    return mu, nu
