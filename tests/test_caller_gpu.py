"""`scale_by_accelerated_adam` and `MultiAdamOp` on the GPU: tree handling, count bookkeeping,
in-place and differentiable branches, against the CPU oracle leaf by leaf, against the per-leaf
`AdamOp`, and against `torch.optim.Adam` as the library routine the whole chain reduces to."""

from __future__ import annotations

import collections

import numpy as np
import pytest
import torch

from conftest import assert_bit_equal
from oracle import adam_oracle as O
from torchopt_amd import AdamOp, MultiAdamOp
from torchopt_amd.transform import scale_by_accelerated_adam
from torchopt_amd.transform.scale_by_adam import _host_value

import bench

pytestmark = pytest.mark.gpu

B1, B2, EPS = 0.9, 0.999, 1e-8
Point = collections.namedtuple('Point', 'w b')


@pytest.fixture(scope='module', autouse=True)
def _gpu():
    assert torch.cuda.is_available(), 'these tests need a GPU; there is no fallback path'
    yield
    torch.cuda.synchronize()


def host(t):
    return t.detach().cpu().numpy()


def dev(a):
    return torch.as_tensor(np.array(a)).cuda()  # keeps 0-dim leaves 0-dim


def make_tree(dtype, seed):
    rng = np.random.default_rng(seed)
    r = lambda *s: np.asarray(rng.standard_normal(s), dtype=dtype)  # noqa: E731
    return {'conv': Point(r(8, 3, 3, 3), r(8)), 'skip': None, 'head': [r(5, 40), r(5)],
            'scalar': r()}


def tree_leaves(tree):
    return [tree['conv'].w, tree['conv'].b, tree['head'][0], tree['head'][1], tree['scalar']]


def to_dev(tree):
    return {'conv': Point(dev(tree['conv'].w), dev(tree['conv'].b)), 'skip': None,
            'head': [dev(tree['head'][0]), dev(tree['head'][1])], 'scalar': dev(tree['scalar'])}


@pytest.mark.parametrize('dtype', [np.float32, np.float64], ids=['f32', 'f64'])
def test_inplace_steps_on_a_nested_tree(dtype):
    """Five optimizer steps; one leaf misses its gradient on steps 2 and 3, so its count lags."""
    t = scale_by_accelerated_adam(B1, B2, EPS, eps_root=0.0)
    params = to_dev(make_tree(dtype, 0))
    state = t.init(params)
    h_mu = [np.zeros_like(a) for a in tree_leaves(make_tree(dtype, 0))]
    h_nu = [np.zeros_like(a) for a in h_mu]
    h_count = [0] * 5
    for step in range(1, 6):
        h_grads = make_tree(dtype, 100 + step)
        grads = to_dev(h_grads)
        missing = step in (2, 3)
        if missing:
            grads['head'][1] = None
        old_state = state
        updates, state = t.update(grads, state, params=params, inplace=True)
        # structure and identity: in place, the outputs are the inputs
        assert isinstance(updates['conv'], Point) and updates['skip'] is None
        assert updates['conv'].w is grads['conv'].w
        assert state.mu['conv'].w is old_state.mu['conv'].w
        if missing:
            assert updates['head'][1] is None
            assert state.count['head'][1] is old_state.count['head'][1]
        for k, (g, got_u, got_m, got_v, got_c) in enumerate(zip(
                tree_leaves(h_grads), tree_leaves(updates), tree_leaves(state.mu),
                tree_leaves(state.nu), tree_leaves(state.count))):
            if missing and k == 3:
                pass
            else:
                h_count[k] += 1
                g = np.ascontiguousarray(g).reshape(-1).copy()
                O.forward_inplace(g, h_mu[k].reshape(-1), h_nu[k].reshape(-1), B1, B2, EPS, 0.0,
                                  h_count[k])
                assert_bit_equal(host(got_u).reshape(-1), g, f'step {step} leaf {k} updates')
            assert_bit_equal(host(got_m), h_mu[k], f'step {step} leaf {k} mu')
            assert_bit_equal(host(got_v), h_nu[k], f'step {step} leaf {k} nu')
            assert got_c.dim() == 0 and got_c.dtype == torch.int64 and got_c.is_cuda
            assert int(got_c) == h_count[k] == _host_value(got_c)
    assert h_count == [5, 5, 5, 3, 5]


def test_flat_variant_matches_tree_variant():
    dtype = np.float32
    sizes = [bench.numel(s) for s in bench.maml_shapes()]
    rng = np.random.default_rng(3)
    grads = [rng.standard_normal(n).astype(dtype) for n in sizes]
    flat = scale_by_accelerated_adam.flat(B1, B2, EPS, 1e-8)
    tree = scale_by_accelerated_adam(B1, B2, EPS, 1e-8)
    p_flat = tuple(dev(g) for g in grads)
    p_tree = {'p': [dev(g) for g in grads]}
    s_flat, s_tree = flat.init(p_flat), tree.init(p_tree)
    assert isinstance(s_flat.mu, tuple)
    for _ in range(3):
        u_flat, s_flat = flat.update(tuple(dev(g) for g in grads), s_flat, inplace=True)
        u_tree, s_tree = tree.update({'p': [dev(g) for g in grads]}, s_tree, inplace=True)
    assert isinstance(u_flat, tuple) and isinstance(s_flat.nu, tuple)
    for a, b in zip(u_flat, u_tree['p']):
        assert torch.equal(a, b)
    for a, b in zip(s_flat.nu, s_tree.nu['p']):
        assert torch.equal(a, b)


@pytest.mark.parametrize('kind', [dict, collections.OrderedDict])
@pytest.mark.parametrize('inplace', [True, False])
def test_dicts_of_tensors_step_like_tuples_whatever_their_key_order(kind, inplace):
    """A plain dict of tensors (`dict(module.named_parameters())`) is flattened without the
    general tree walk; it must step exactly as the tuple of its values does, keep its type and
    keys, and line gradients up with the state BY NAME when their dict was built in another
    order (the reference's pytree library sorts dict keys, so order never matters there)."""
    torch.manual_seed(8)
    names = ['w2', 'b2', 'w1', 'b1', 'emb']
    shapes = [(7, 5), (7,), (5, 3), (5,), (300,)]
    params = kind((n, torch.randn(s, device='cuda')) for n, s in zip(names, shapes))
    t = scale_by_accelerated_adam(B1, B2, EPS, 1e-8)
    as_dict, as_tuple = t.init(params), t.init(tuple(params.values()))
    assert type(as_dict.mu) is kind and list(as_dict.mu) == names and list(as_dict.count) == names
    for step in range(3):
        grads = [torch.randn(s, device='cuda') for s in shapes]
        order = list(range(len(names))) if step != 1 else [3, 0, 4, 2, 1]  # shuffled once
        gd = kind((names[k], grads[k].clone()) for k in order)
        ud, as_dict = t.update(gd, as_dict, inplace=inplace)
        ut, as_tuple = t.update(tuple(g.clone() for g in grads), as_tuple, inplace=inplace)
        assert type(ud) is kind and sorted(ud) == sorted(names)
        for k, n in enumerate(names):
            assert torch.equal(ud[n], ut[k]), (step, n)
            assert torch.equal(as_dict.mu[n], as_tuple.mu[k])
            assert torch.equal(as_dict.nu[n], as_tuple.nu[k])
            assert int(as_dict.count[n]) == int(as_tuple.count[k]) == step + 1
    bad = kind((n + '_', g) for n, g in zip(names, grads))
    with pytest.raises(ValueError, match='different keys'):
        t.update(bad, as_dict, inplace=inplace)


def test_count_state_restored_from_elsewhere_is_read_once():
    """Counts that did not come from this transformation (a loaded checkpoint) carry no host
    mirror: they are read from the device, and the step uses their value."""
    t = scale_by_accelerated_adam(B1, B2, EPS)
    g = np.random.default_rng(1).standard_normal(1000).astype(np.float32)
    state = t.init([dev(g)])
    restored = state._replace(count=[torch.tensor(41, device='cuda')])
    updates, new_state = t.update([dev(g)], restored, inplace=True)
    assert int(new_state.count[0]) == 42
    e = g.copy()
    O.forward_inplace(e, np.zeros_like(g), np.zeros_like(g), B1, B2, EPS, 0.0, 42)
    assert_bit_equal(host(updates[0]), e, 'count 42')


@pytest.fixture(params=['native_node', 'python_node'])
def node(request, monkeypatch):
    """Both routes of the differentiable list step: the C++ autograd node of the extension
    module (the default) and the same node written in Python (what `torch.compile` traces)."""
    monkeypatch.setattr(MultiAdamOp, 'use_native_node', request.param == 'native_node')
    return request.param


def test_differentiable_branch_matches_per_leaf_adam_op(node):
    """inplace=False: the list-level autograd node gives the same values and the same
    gradients as the reference-shaped per-leaf AdamOp, bit for bit."""
    shapes = bench.maml_shapes()
    rng = np.random.default_rng(11)
    data = [[rng.standard_normal(s).astype(np.float32) for _ in range(3)] for s in shapes]
    cots = [[rng.standard_normal(s).astype(np.float32) for _ in range(3)] for s in shapes]
    count, eps_root = 5, 1e-8

    def leaves():
        return [[dev(a).requires_grad_(True) for a in (g, 0.1 * m, np.abs(0.01 * v))]
                for g, m, v in data]

    # per leaf
    single = leaves()
    op = AdamOp(B1, B2, EPS, eps_root=eps_root, inplace=False)
    outs = [op(m, v, g, count) for g, m, v in single]
    torch.autograd.backward([o for out in outs for o in out],
                            [dev(c) for ct in cots for c in ct])
    # whole list
    multi = leaves()
    mop = MultiAdamOp(B1, B2, EPS, eps_root=eps_root, inplace=False)
    new_mu, new_nu, new_u = mop([x[1] for x in multi], [x[2] for x in multi],
                                [x[0] for x in multi], count)
    flat_out = [o for trio in zip(new_mu, new_nu, new_u) for o in trio]
    assert all(o.requires_grad for o in flat_out)
    torch.autograd.backward(flat_out, [dev(c) for ct in cots for c in ct])
    for k in range(len(shapes)):
        for a, b, what in zip(outs[k], (new_mu[k], new_nu[k], new_u[k]), ('mu', 'nu', 'updates')):
            assert torch.equal(a, b), f'leaf {k} new {what}'
        for a, b, what in zip(single[k], multi[k], ('updates', 'mu', 'nu')):
            assert torch.equal(a.grad, b.grad), f'leaf {k} grad wrt {what}'


@pytest.mark.parametrize('which', ['updates_only', 'updates_and_mu', 'ragged'])
def test_differentiable_branch_with_missing_outside_gradients(which, node):
    """Only some outputs feed the loss: the one-pass backward must give what the per-leaf chain
    gives when autograd has nothing to add at new_mu / new_nu (for all leaves, or for some)."""
    shapes = [(7, 5), (300,), (3, 4, 5), ()]
    rng = np.random.default_rng(21)
    data = [[np.asarray(rng.standard_normal(s), dtype=np.float64) for _ in range(3)]
            for s in shapes]
    cots = [[np.asarray(rng.standard_normal(s), dtype=np.float64) for _ in range(3)]
            for s in shapes]

    def leaves():
        return [[dev(a).requires_grad_(True) for a in (g, 0.1 * m, np.abs(0.01 * v) + 1e-3)]
                for g, m, v in data]

    def loss_terms(outs):
        terms = []
        for k, (new_mu, new_nu, new_u) in enumerate(outs):
            terms.append((new_u * dev(cots[k][2])).sum())
            if which == 'updates_and_mu' or (which == 'ragged' and k % 2 == 0):
                terms.append((new_mu * dev(cots[k][0])).sum())
            if which == 'ragged' and k == 1:
                terms.append((new_nu * dev(cots[k][1])).sum())
        return sum(terms)

    single = leaves()
    op = AdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)
    loss_terms([op(m, v, g, 3) for g, m, v in single]).backward()
    multi = leaves()
    mop = MultiAdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)
    new_mu, new_nu, new_u = mop([x[1] for x in multi], [x[2] for x in multi],
                                [x[0] for x in multi], 3)
    loss_terms(list(zip(new_mu, new_nu, new_u))).backward()
    for k in range(len(shapes)):
        for a, b, what in zip(single[k], multi[k], ('updates', 'mu', 'nu')):
            assert_bit_equal(host(b.grad), host(a.grad), f'{which} leaf {k} grad wrt {what}')


@pytest.mark.parametrize('which', ['no_update_gradient', 'mu_only', 'nothing_for_one_leaf'])
def test_leaf_whose_update_receives_no_gradient(which, node):
    """A leaf whose new_updates does not feed the loss: the per-leaf chain never runs
    backward_updates for it, so the infinities its new_updates / new_mu ratio may hold must not
    reach the gradients of the one-pass node either (0 * inf would be NaN), and a -0 outside
    gradient must stay -0."""
    rng = np.random.default_rng(33)
    shapes = [(40,), (9,), (6, 3)]
    data = [[np.asarray(rng.standard_normal(s), dtype=np.float32) for _ in range(3)]
            for s in shapes]
    # leaf 1: a tiny non-zero new_mu under a huge update -> new_updates / new_mu overflows
    data[1][0][:] = 0.0
    data[1][1][:] = 1e-38
    data[1][2][:] = 0.0
    cots = [[np.asarray(rng.standard_normal(s), dtype=np.float32) for _ in range(3)]
            for s in shapes]
    cots[1][0][:3] = -0.0

    def leaves():
        return [[dev(g).requires_grad_(True), dev(m).requires_grad_(True),
                 dev(np.abs(v)).requires_grad_(True)] for g, m, v in data]

    def loss_terms(outs):
        terms = []
        for k, (new_mu, new_nu, new_u) in enumerate(outs):
            if k != 1:
                terms.append((new_u * dev(cots[k][2])).sum())
                terms.append((new_nu * dev(cots[k][1])).sum())
            if k == 1 and which == 'nothing_for_one_leaf':
                continue
            terms.append((new_mu * dev(cots[k][0])).sum())
            if k == 1 and which == 'no_update_gradient':
                terms.append((new_nu * dev(cots[k][1])).sum())
        return sum(terms)

    single = leaves()
    op = AdamOp(B1, B2, 0.0, eps_root=0.0, inplace=False)
    loss_terms([op(m, v, g, 2) for g, m, v in single]).backward()
    multi = leaves()
    mop = MultiAdamOp(B1, B2, 0.0, eps_root=0.0, inplace=False)
    new_mu, new_nu, new_u = mop([x[1] for x in multi], [x[2] for x in multi],
                                [x[0] for x in multi], 2)
    assert not torch.isfinite(new_u[1] / new_mu[1]).all()  # the case is what it claims to be
    loss_terms(list(zip(new_mu, new_nu, new_u))).backward()
    for k in range(len(shapes)):
        for a, b, what in zip(single[k], multi[k], ('updates', 'mu', 'nu')):
            if a.grad is None:
                assert b.grad is None, f'{which} leaf {k}: {what} got a gradient from nowhere'
            else:
                assert_bit_equal(host(b.grad), host(a.grad), f'{which} leaf {k} grad wrt {what}')


def test_differentiable_branch_with_a_step_count_per_leaf(node):
    """Leaves that have fallen out of step carry their own count (ints or 0-dim tensors); values
    and gradients still equal the per-leaf chain's, also for a leaf whose update gets no
    gradient while its neighbours' counts differ."""
    rng = np.random.default_rng(44)
    shapes = [(12, 3), (5,), (2, 2, 2), (31,)]
    counts = [3, torch.tensor(7, device='cuda'), 3, 1]
    data = [[np.asarray(rng.standard_normal(s), dtype=np.float64) for _ in range(3)]
            for s in shapes]
    cots = [np.asarray(rng.standard_normal(s), dtype=np.float64) for s in shapes]

    def leaves():
        return [[dev(a).requires_grad_(True) for a in (g, 0.1 * m, np.abs(0.01 * v) + 1e-3)]
                for g, m, v in data]

    def loss(outs):
        # leaf 2 contributes through new_mu only: it takes the backward_mu route on its own
        return sum((o[2] * dev(c)).sum() if k != 2 else (o[0] * dev(c)).sum()
                   for k, (o, c) in enumerate(zip(outs, cots)))

    single = leaves()
    op = AdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)
    loss([op(m, v, g, int(c)) for (g, m, v), c in zip(single, counts)]).backward()
    multi = leaves()
    mop = MultiAdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)
    out = mop([x[1] for x in multi], [x[2] for x in multi], [x[0] for x in multi], counts)
    loss(list(zip(*out))).backward()
    for k in range(len(shapes)):
        for a, b, what in zip(single[k], multi[k], ('updates', 'mu', 'nu')):
            if a.grad is None:
                assert b.grad is None, f'leaf {k}: {what} got a gradient from nowhere'
            else:
                assert_bit_equal(host(b.grad), host(a.grad), f'leaf {k} grad wrt {what}')


def test_native_node_contract():
    """What autograd sees of `adam_op.step_multi`: outputs that require grad exactly when an
    input does, no graph under no_grad, fresh non-overlapping outputs of the inputs' layout, and
    list lengths checked before anything is launched."""
    from torchopt_amd._C import adam_op

    g = [torch.randn(5, 7, device='cuda'), torch.randn(3, device='cuda')]
    mu = [torch.zeros_like(x) for x in g]
    nu = [torch.zeros_like(x) for x in g]
    new_mu, new_nu, new_u = adam_op.step_multi(g, mu, nu, B1, B2, EPS, 0.0, 1)
    assert isinstance(new_mu, list) and len(new_mu) == len(new_nu) == len(new_u) == 2
    assert not any(t.requires_grad for t in new_mu + new_nu + new_u)
    gl = [x.clone().requires_grad_(True) for x in g]
    out = adam_op.step_multi(gl, mu, nu, B1, B2, EPS, 0.0, 1)
    assert all(t.requires_grad and t.grad_fn is not None for lst in out for t in lst)
    with torch.no_grad():
        out = adam_op.step_multi(gl, mu, nu, B1, B2, EPS, 0.0, 1)
    assert not any(t.requires_grad for lst in out for t in lst)
    # outputs do not overlap one another or the inputs, and keep the inputs' shapes
    spans = sorted((t.data_ptr(), t.data_ptr() + t.numel() * t.element_size())
                   for lst in (out[0], out[1], out[2], g, mu, nu) for t in lst)
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    assert [t.shape for t in out[2]] == [x.shape for x in g]
    assert all(t.data_ptr() % 16 == 0 for lst in out for t in lst)
    with pytest.raises(RuntimeError, match='differ in length'):
        adam_op.step_multi(g, mu[:1], nu, B1, B2, EPS, 0.0, 1)
    with pytest.raises(RuntimeError, match='counts'):
        adam_op.step_multi(g, mu, nu, B1, B2, EPS, 0.0, [1, 2, 3])
    assert adam_op.step_multi([], [], [], B1, B2, EPS, 0.0, 1) == ([], [], [])


def test_native_node_behaves_like_any_autograd_node():
    """The node is written against autograd's Node interface directly, so what a Function gets
    for free is checked here: saved tensors released after a backward without retain_graph (and
    the usual error on a second one), identical gradients from repeated backwards with
    retain_graph, the version check on saved tensors, saved-tensor hooks, a layout-converted
    input, and no reference cycle between the node and the outputs it saves."""
    import gc

    from torchopt_amd._C import adam_op

    def fresh():
        torch.manual_seed(3)
        g = [torch.randn(64, 3, device='cuda', requires_grad=True),
             torch.randn(17, device='cuda', requires_grad=True)]
        mu = [torch.randn_like(x).mul_(0.1).requires_grad_(True) for x in g]
        nu = [torch.rand_like(x).mul_(0.01).requires_grad_(True) for x in g]
        return g, mu, nu

    def loss_of(out):
        return sum((t * t).sum() for lst in out for t in lst)

    g, mu, nu = fresh()
    out = adam_op.step_multi(g, mu, nu, B1, B2, EPS, 1e-8, 2)
    assert out[0][0].grad_fn.name() == 'AdamStepBackward'
    assert all(t.grad_fn is out[0][0].grad_fn for lst in out for t in lst)
    loss = loss_of(out)
    first = torch.autograd.grad(loss, g + mu + nu, retain_graph=True)
    second = torch.autograd.grad(loss, g + mu + nu)
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    with pytest.raises(RuntimeError, match='second time'):
        torch.autograd.grad(loss, g + mu + nu)

    # a saved tensor modified in place between forward and backward is caught
    g, mu, nu = fresh()
    out = adam_op.step_multi(g, mu, nu, B1, B2, EPS, 1e-8, 2)
    loss = loss_of(out)
    with torch.no_grad():
        out[0][1].add_(1.0)  # new_mu of the second leaf, saved for backward
    with pytest.raises(RuntimeError, match='modified by an inplace operation'):
        loss.backward()

    # saved-tensor hooks see the 3 tensors per leaf the reference's Functions save
    g, mu, nu = fresh()
    packed = []

    def pack(t):
        packed.append(t.shape)
        return t

    with torch.autograd.graph.saved_tensors_hooks(pack, lambda t: t):
        out = adam_op.step_multi(g, mu, nu, B1, B2, EPS, 1e-8, 2)
    assert len(packed) == 3 * len(g)
    want = torch.autograd.grad(loss_of(out), g + mu + nu)
    for a, b in zip(first, want):
        assert torch.equal(a, b)

    # an expanded gradient (what sum().backward() hands on): converted inside, its gradient
    # comes back in the input's own shape
    base = torch.randn(1, device='cuda', requires_grad=True)
    ge = [base.expand(64, 3), g[1]]
    out = adam_op.step_multi(ge, mu, nu, B1, B2, EPS, 1e-8, 2)
    (d_base,) = torch.autograd.grad(loss_of(out), [base])
    dense = base.detach().expand(64, 3).contiguous().requires_grad_(True)
    out2 = adam_op.step_multi([dense, g[1]], mu, nu, B1, B2, EPS, 1e-8, 2)
    (d_dense,) = torch.autograd.grad(loss_of(out2), [dense])
    torch.testing.assert_close(d_base, d_dense.sum().reshape(1), rtol=1e-5, atol=0)

    # dropping the outputs frees their memory at once: the node holds its saved outputs
    # without a cycle through their grad_fn
    del out, out2, loss, want, first, second
    gc.collect()
    gc.disable()
    try:
        big = [torch.randn(1 << 20, device='cuda', requires_grad=True)]
        zeros = [torch.zeros(1 << 20, device='cuda')]
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        held = adam_op.step_multi(big, zeros, zeros, B1, B2, EPS, 1e-8, 1)
        assert torch.cuda.memory_allocated() >= before + 3 * (1 << 22)  # the three outputs
        del held
        assert torch.cuda.memory_allocated() == before
    finally:
        gc.enable()


def test_meta_step_through_the_transformation():
    """A MAML-style inner step: params' = params - lr * adam(grad); the outer loss
    differentiates through the update, the moments and the step."""
    torch.manual_seed(0)
    w = torch.randn(6, 4, device='cuda', dtype=torch.float64, requires_grad=True)
    b = torch.randn(6, device='cuda', dtype=torch.float64, requires_grad=True)
    x = torch.randn(16, 4, device='cuda', dtype=torch.float64)
    y = torch.randn(16, 6, device='cuda', dtype=torch.float64)
    t = scale_by_accelerated_adam(B1, B2, EPS, eps_root=1e-8, moment_requires_grad=True)
    state = t.init((w, b))

    def inner_loss(w_, b_):
        return ((x @ w_.t() + b_ - y) ** 2).mean()

    grads = torch.autograd.grad(inner_loss(w, b), (w, b), create_graph=True)
    updates, state = t.update(grads, state, params=(w, b), inplace=False)
    assert isinstance(updates, tuple) and updates[0].requires_grad
    w1, b1 = w - 0.1 * updates[0], b - 0.1 * updates[1]
    outer = inner_loss(w1, b1)
    gw, gb = torch.autograd.grad(outer, (w, b))
    assert torch.isfinite(gw).all() and torch.isfinite(gb).all() and gw.abs().sum() > 0
    # same computation through the per-leaf reference-shaped op
    op = AdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)
    grads2 = torch.autograd.grad(inner_loss(w, b), (w, b), create_graph=True)
    z = [torch.zeros_like(p, requires_grad=True) for p in (w, b)]
    z2 = [torch.zeros_like(p, requires_grad=True) for p in (w, b)]
    u2 = [op(m, v, g, 1)[2] for m, v, g in zip(z, z2, grads2)]
    outer2 = inner_loss(w - 0.1 * u2[0], b - 0.1 * u2[1])
    gw2, gb2 = torch.autograd.grad(outer2, (w, b))
    # three gradient paths meet at w; their summation order may differ between the two graphs
    torch.testing.assert_close(gw, gw2, rtol=1e-12, atol=1e-14)
    torch.testing.assert_close(gb, gb2, rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize('inplace', [True, False])
def test_chain_reduces_to_torch_optim_adam(inplace):
    """With eps_root = 0 the chain scale_by_adam -> scale(-lr) -> apply is torch.optim.Adam;
    the reference pins its accelerated path the same way, in float64, at 25x the default
    tolerance (/root/reference/tests/test_alias.py:207-270, tests/helpers.py:202-229)."""
    torch.manual_seed(1)
    lr = 1e-2
    model = torch.nn.Sequential(torch.nn.Linear(20, 32), torch.nn.Tanh(),
                                torch.nn.Linear(32, 5)).to('cuda', torch.float64)
    ref = torch.nn.Sequential(torch.nn.Linear(20, 32), torch.nn.Tanh(),
                              torch.nn.Linear(32, 5)).to('cuda', torch.float64)
    ref.load_state_dict(model.state_dict())
    base = [p.detach().clone() for p in model.parameters()]
    optim_ref = torch.optim.Adam(ref.parameters(), lr, betas=(B1, B2), eps=EPS)
    t = scale_by_accelerated_adam(B1, B2, EPS, eps_root=0.0)
    params = tuple(model.parameters())
    state = t.init(params)
    for step in range(5):
        x = torch.randn(64, 20, device='cuda', dtype=torch.float64)
        y = torch.randint(0, 5, (64,), device='cuda')
        loss = torch.nn.functional.cross_entropy(model(x), y)
        grads = torch.autograd.grad(loss, params)
        updates, state = t.update(grads, state, params=params, inplace=inplace)
        with torch.no_grad():
            for p, u in zip(params, updates):
                p.add_(u, alpha=-lr)
        optim_ref.zero_grad()
        torch.nn.functional.cross_entropy(ref(x), y).backward()
        optim_ref.step()
    for p, q, p0 in zip(model.parameters(), ref.parameters(), base):
        torch.testing.assert_close(p - p0, q - p0, rtol=25 * 1e-7, atol=25 * 1e-7)


def test_expanded_and_permuted_gradients_on_the_differentiable_branch(node):
    """Gradients straight out of `torch.autograd.grad` may be expanded (stride 0, as the
    gradient of a sum is) or laid out differently from the moments; the list ops bring them to
    the moments' memory order instead of misreading them."""
    torch.manual_seed(5)
    shapes = [(6, 40), (33,), (4, 3, 5, 5)]
    mu = [0.1 * torch.randn(s, device='cuda', dtype=torch.float64) for s in shapes]
    nu = [(0.01 * torch.randn(s, device='cuda', dtype=torch.float64)).abs_() for s in shapes]
    grads = [torch.tensor(0.5, device='cuda', dtype=torch.float64).expand(shapes[0]),  # stride 0
             torch.randn(66, device='cuda', dtype=torch.float64)[::2],  # strided slice
             torch.randn(shapes[2], device='cuda', dtype=torch.float64).contiguous(
                 memory_format=torch.channels_last)]
    assert not grads[0].is_contiguous() and not grads[1].is_contiguous()
    leaves = [g.detach().clone().requires_grad_(True) for g in grads]  # dense stand-ins
    op = MultiAdamOp(B1, B2, EPS, eps_root=1e-8, inplace=False)
    want = op([m.clone() for m in mu], [v.clone() for v in nu], leaves, 4)
    got = op([m.clone() for m in mu], [v.clone() for v in nu], grads, 4)
    for a, b in zip(sum(map(list, got), []), sum(map(list, want), [])):
        assert a.shape == b.shape
        assert_bit_equal(host(a.contiguous()), host(b.contiguous()), 'values')
    # and the backward pass reads the saved non-dense gradients correctly
    gl = [g.detach().requires_grad_(True) for g in grads]
    out = op([m.clone() for m in mu], [v.clone() for v in nu], gl, 4)
    total = sum((u * u).sum() for u in out[2])
    dg = torch.autograd.grad(total, gl)
    total_ref = sum((u * u).sum() for u in want[2])
    dg_ref = torch.autograd.grad(total_ref, leaves)
    for a, b in zip(dg, dg_ref):
        assert_bit_equal(host(a.contiguous()), host(b.contiguous()), 'gradients')


def test_inplace_branch_refuses_gradients_it_cannot_overwrite():
    mu = [torch.zeros(6, 40, device='cuda')]
    nu = [torch.zeros(6, 40, device='cuda')]
    g = [torch.tensor(0.5, device='cuda').expand(6, 40)]
    with pytest.raises(RuntimeError, match='dense'):
        MultiAdamOp(inplace=True)(mu, nu, g, 1)


def test_availability_probe_on_the_gpu():
    """tests/test_accelerated_op.py:47-54 of the reference, for the devices this build serves."""
    from torchopt_amd import accelerated_op_available

    assert accelerated_op_available()
    assert accelerated_op_available('cuda')
    assert accelerated_op_available('cuda:0')
    assert accelerated_op_available(0)
    assert accelerated_op_available(torch.device('cuda', 0))
    assert accelerated_op_available(['cuda', 'cuda:0', 0])
    assert not accelerated_op_available(['cuda', 'meta'])
    assert not accelerated_op_available(['cpu', 'cuda'])  # the CPU is not served here


@pytest.mark.parametrize('dtype', [torch.float32, torch.float64, torch.bfloat16],
                         ids=['f32', 'f64', 'bf16'])
def test_state_of_large_leaves_is_placed_and_steps_like_any_other(dtype):
    """init puts the moments of a large GPU leaf 8 KiB off the 16 KiB address phase (a view into
    a slightly larger block), leaves small and non-contiguous leaves to zeros_like, and the steps
    that follow are the oracle's bit for bit either way."""
    from torchopt_amd import FusedAdam, state_zeros_like

    n_big = (3 << 20) // torch.empty(0, dtype=dtype).element_size() + 5  # 3 MiB and a ragged end
    params = [torch.randn(n_big, device='cuda').to(dtype),
              torch.randn(7, 33, device='cuda').to(dtype),
              torch.randn(1024, 600, device='cuda').to(dtype).t()]  # large, not contiguous
    t = scale_by_accelerated_adam(B1, B2, 1e-3, eps_root=0.0)
    state = t.init(params)
    for moments, phase in ((state.mu, 8 << 10), (state.nu, 0)):
        big, small, strided = moments
        assert big.data_ptr() % (16 << 10) == phase and big.is_contiguous()
        assert big.shape == params[0].shape and big.dtype == dtype and not big.any()
        assert small.storage_offset() == 0 and small.shape == (7, 33)
        assert strided.stride() == params[2].stride() and strided.storage_offset() == 0
    assert state_zeros_like(params[0], requires_grad=True).requires_grad
    # the large leaves of a tree share one block: first moments, then second moments, disjoint,
    # a leaf's two moments clear of the multiples of 16 MiB at which arrays collide in DRAM
    from torchopt_amd import state_zeros_like_tree
    tree = [params[0], None, params[1], torch.empty(5 << 20, device='cuda', dtype=dtype), params[2]]
    mu, nu = state_zeros_like_tree(tree, requires_grad=True)
    assert mu[1] is None and nu[1] is None and mu[2].shape == (7, 33) and mu[4].stride() == params[2].stride()
    placed = [mu[0], mu[3], nu[0], nu[3]]
    assert len({x.untyped_storage().data_ptr() for x in placed}) == 1
    spans = sorted((x.data_ptr(), x.data_ptr() + x.numel() * x.element_size()) for x in placed)
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    assert [x.data_ptr() for x in placed] == sorted(x.data_ptr() for x in placed)
    for got, like, phase in zip(placed, (tree[0], tree[3], tree[0], tree[3]),
                                (8 << 10, 8 << 10, 0, 0)):
        assert got.data_ptr() % (16 << 10) == phase and got.shape == like.shape
        assert got.requires_grad and got.dtype == dtype and not got.any()
    apart = (nu[3].data_ptr() - mu[3].data_ptr()) % (16 << 20) - (8 << 10)
    assert nu[0].data_ptr() - mu[0].data_ptr() == nu[3].data_ptr() - mu[3].data_ptr()
    assert apart % (2 << 20) == 0 and (4 << 20) <= apart <= (12 << 20)  # the fast distances
    if dtype == torch.bfloat16:
        return  # values of the 16-bit step are covered where its oracle is (test_low_precision_gpu)
    np_dtype = {torch.float32: np.float32, torch.float64: np.float64}[dtype]
    h_mu, h_nu = np.zeros(n_big, np_dtype), np.zeros(n_big, np_dtype)
    for step in (1, 2, 3):
        g = torch.randn(n_big, device='cuda').to(dtype)
        h_g = host(g).copy()
        updates, state = t.update([g, None, None], state, params=params, inplace=True)
        O.forward_inplace(h_g, h_mu, h_nu, B1, B2, 1e-3, 0.0, step)
        assert_bit_equal(host(updates[0]), h_g, f'step {step} updates')
        assert_bit_equal(host(state.mu[0]), h_mu, f'step {step} mu')
        assert_bit_equal(host(state.nu[0]), h_nu, f'step {step} nu')
    opt = FusedAdam([torch.nn.Parameter(params[0].clone())], lr=1e-3)
    opt.param_groups[0][0].grad = torch.randn(n_big, device='cuda').to(dtype)
    opt.step()
    s = opt.state_groups[0]
    assert s.mu[0].data_ptr() % (16 << 10) == 8 << 10 and s.nu[0].data_ptr() % (16 << 10) == 0


@pytest.mark.parametrize('seed', [0, 1, 2])
def test_tree_state_allocation_invariants_on_random_trees(seed):
    """Random trees (sizes from empty to 24 MiB, three dtypes, missing leaves): whatever the mix,
    every moment has its leaf's shape and dtype, holds zeros, shares no byte with another, and
    the large leaves of one dtype sit at the preferred phase in one block."""
    from torchopt_amd import state_zeros_like_tree

    rng = np.random.default_rng(seed)
    dtypes = (torch.float32, torch.float64, torch.bfloat16)
    tree = []
    for _ in range(int(rng.integers(1, 40))):
        kind = rng.integers(0, 10)
        if kind == 0:
            tree.append(None)
            continue
        n = int(rng.choice([0, 1, 7, 4096, 1 << 18, (1 << 20) + 3, 3 << 20, 6 << 20]))
        tree.append(torch.empty(n, device='cuda', dtype=dtypes[int(rng.integers(0, 3))]))
    mu, nu = state_zeros_like_tree(tree)
    spans, blocks = [], {}
    for t, a, b in zip(tree, mu, nu):
        if t is None:
            assert a is None and b is None
            continue
        for x in (a, b):
            assert x.shape == t.shape and x.dtype == t.dtype and x.device == t.device
            assert x.is_contiguous() and not x.any()
            if x.numel():
                spans.append((x.data_ptr(), x.data_ptr() + x.numel() * x.element_size()))
            if t.numel() * t.element_size() >= (1 << 20):
                assert x.data_ptr() % (16 << 10) == (8 << 10 if x is a else 0)
                blocks.setdefault(t.dtype, set()).add(x.untyped_storage().data_ptr())
    spans.sort()
    assert all(p[1] <= q[0] for p, q in zip(spans, spans[1:])), 'two moments overlap'
    assert all(len(b) == 1 for b in blocks.values()), 'one block per dtype'
