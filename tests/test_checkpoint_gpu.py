"""Optimizer state through torch.save -> torch.load -> load_state_dict -> step: bit-equal to an
uninterrupted run, for the fused optimizer and for the functional transformation, with leaves
large enough to get this package's state placement (views into one block per tree) and leaves
too small for it.  Mirrors what /root/reference/torchopt/optim/base.py:126-135 offers
(`state_dict` / `load_state_dict` hand the state tuples through)."""

from __future__ import annotations

import io

import pytest
import torch

import torchopt_amd as topt
from torchopt_amd.placement import is_placed, placed_like_tree, unshared
from torchopt_amd.transform import scale_by_accelerated_adam

pytestmark = pytest.mark.gpu

SHAPES = [(300_000,), (17, 5), (1024, 300), (3,)]  # two leaves beyond 1 MiB, two small ones


def params_and_grads(steps, seed=0):
    g = torch.Generator(device='cpu').manual_seed(seed)
    params = [torch.randn(s, generator=g).cuda() for s in SHAPES]
    grads = [[torch.randn(s, generator=g).cuda() for s in SHAPES] for _ in range(steps)]
    return params, grads


def through_a_file(obj):
    """torch.save into memory, torch.load back onto the GPU (a file this test wrote itself)."""
    buf = io.BytesIO()
    torch.save(obj, buf)
    size = buf.tell()
    buf.seek(0)
    return torch.load(buf, map_location='cuda', weights_only=False), size


def same_bits(a, b, what):
    assert a.shape == b.shape and a.dtype == b.dtype, what
    assert torch.equal(a.contiguous().view(torch.int32), b.contiguous().view(torch.int32)), what


@pytest.mark.parametrize('capturable', [False, True])
def test_fused_adam_resumes_bit_for_bit(capturable):
    params, grads = params_and_grads(5)

    def make(ps):
        ps = [p.clone().requires_grad_(True) for p in ps]
        return ps, topt.FusedAdam(ps, lr=1e-2, eps_root=1e-8, weight_decay=1e-3,
                                  capturable=capturable)

    def run(ps, opt, which):
        for k in which:
            for p, g in zip(ps, grads[k]):
                p.grad = g.clone()
            opt.step()

    straight, opt = make(params)
    run(straight, opt, range(5))

    first, opt_a = make(params)
    run(first, opt_a, range(3))
    print('FusedAdam: three steps, save, load, two more steps', flush=True)
    (state, saved_params), size = through_a_file((opt_a.state_dict(), [p.detach() for p in first]))
    # the block of the tree is written once: the file holds the state, not a copy per view
    state_bytes = sum(2 * p.numel() * 4 for p in first)
    assert size < state_bytes + sum(p.numel() * 4 for p in first) + (1 << 20), size
    resumed, opt_b = make(saved_params)
    opt_b.load_state_dict(state)
    # what torch.load allocated has been moved to the placement the package's init produces
    for mu, nu, p in zip(opt_b.state_dict()[0].mu, opt_b.state_dict()[0].nu, resumed):
        if p.numel() * 4 >= (1 << 20):
            assert is_placed(mu, 0) and is_placed(nu, 1)
    run(resumed, opt_b, range(3, 5))
    for a, b, shape in zip(resumed, straight, SHAPES):
        same_bits(a.detach(), b.detach(), f'parameters {shape}')
    for sa, sb in zip(opt_b.state_dict(), opt.state_dict()):
        for a, b, shape in zip(sa.mu, sb.mu, SHAPES):
            same_bits(a, b, f'mu {shape}')
        for a, b, shape in zip(sa.nu, sb.nu, SHAPES):
            same_bits(a, b, f'nu {shape}')
        assert [int(c) for c in sa.count] == [int(c) for c in sb.count] == [5] * len(SHAPES)


@pytest.mark.parametrize('inplace', [True, False])
def test_functional_state_resumes_bit_for_bit(inplace):
    _, grads = params_and_grads(4, seed=1)
    tr = scale_by_accelerated_adam(0.9, 0.999, 1e-8, 1e-8)
    tree = {'w': grads[0][0], 'rest': (grads[0][1], grads[0][2], grads[0][3])}

    def as_tree(leaves):
        return {'w': leaves[0].clone(), 'rest': tuple(x.clone() for x in leaves[1:])}

    state = tr.init(tree)
    outs = []
    for k in range(4):
        u, state = tr.update(as_tree(grads[k]), state, inplace=inplace)
        outs.append(u)

    state2 = tr.init(tree)
    for k in range(2):
        _, state2 = tr.update(as_tree(grads[k]), state2, inplace=inplace)
    print(f'scale_by_accelerated_adam inplace={inplace}: two steps, save, load, two more',
          flush=True)
    loaded, _ = through_a_file(state2)
    assert type(loaded).__name__ == 'ScaleByAdamState' and isinstance(loaded.mu, dict)
    for k in range(2, 4):
        u, loaded = tr.update(as_tree(grads[k]), loaded, inplace=inplace)
        same_bits(u['w'], outs[k]['w'], f'update w at step {k + 1}')
        for a, b in zip(u['rest'], outs[k]['rest']):
            same_bits(a, b, f'update at step {k + 1}')
    same_bits(loaded.mu['w'], state.mu['w'], 'mu w')
    same_bits(loaded.nu['rest'][1], state.nu['rest'][1], 'nu')
    assert int(loaded.count['w']) == int(state.count['w']) == 4


def test_one_leaf_of_a_placed_tree_saved_alone():
    """A moment of a large leaf is a view into its tree's block: saved as it is, the file takes
    the whole block; `unshared` gives it a storage of its own first.  `placed_like_tree` puts
    loaded leaves back where init would have put them, values untouched."""
    leaves = [torch.randn(s, device='cuda') for s in SHAPES]
    mu, nu = topt.state_zeros_like_tree(leaves)
    mu[0].normal_()
    nu[0].uniform_()
    big = SHAPES[0][0] * 4
    _, whole = through_a_file(mu[0])
    alone, small = through_a_file(unshared(mu[0]))
    assert whole > 2 * big and small < big + 4096, (whole, small)
    same_bits(alone, mu[0], 'the leaf saved alone')
    assert unshared(alone) is alone
    loaded_nu, _ = through_a_file(unshared(nu[0]))
    back_mu, back_nu = placed_like_tree([alone, None, mu[1]], [loaded_nu, None, nu[1]])
    assert back_mu[1] is None and back_mu[2] is mu[1] and back_nu[2] is nu[1]  # small: untouched
    assert is_placed(back_mu[0], 0) and is_placed(back_nu[0], 1)
    same_bits(back_mu[0], mu[0], 'mu after placement')
    same_bits(back_nu[0], nu[0], 'nu after placement')


def test_placement_can_be_switched_off(monkeypatch):
    """TORCHOPT_AMD_STATE_PLACEMENT=0: every moment is a plain zeros_like allocation (offset 0, a
    storage of its own), as the reference's init makes them."""
    leaves = [torch.randn(s, device='cuda') for s in SHAPES]
    monkeypatch.setenv('TORCHOPT_AMD_STATE_PLACEMENT', '0')
    mu, nu = topt.state_zeros_like_tree(leaves)
    for t, leaf in zip(mu + nu, leaves + leaves):
        assert t.storage_offset() == 0 and t.shape == leaf.shape and not t.any()
    assert mu[0].untyped_storage().data_ptr() != mu[2].untyped_storage().data_ptr()
    assert topt.state_zeros_like(leaves[0]).storage_offset() == 0
    monkeypatch.delenv('TORCHOPT_AMD_STATE_PLACEMENT')
    mu, nu = topt.state_zeros_like_tree(leaves)
    assert mu[0].untyped_storage().data_ptr() == mu[2].untyped_storage().data_ptr()
