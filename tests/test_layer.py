"""`flex_rnn_amd.layer`: a layer function's per-timestep preparation moves into the compiled step.  Checked on the
CPU with the plain loop standing in for the kernels (`jit.apply = jit.naive`, as a user debugging a layer would):
the rewritten graph must compute what the layer computes eagerly, values and gradients, and must have moved
what the docstring says it moves."""
import pytest
import torch as th
import torch.nn.functional as F

import flex_rnn_amd
from flex_rnn_amd import examples, ops
from oracle import recurrence

DIMS = dict(B=2, T=6, D=32, C=16)


def _eager(layer, steps, inputs, dtype=th.float64):
    """The layer as written, every step on the plain loop in `dtype`, with gradients of the sum of squares of the results."""
    saved = {k: s.apply for k, s in steps.items()}
    for s in steps.values():
        s.apply = (lambda *a, s=s: s.naive(*a, dtype=dtype))
    try:
        xs = [i.detach().clone().requires_grad_() for i in inputs]
        res = layer(*xs)
        res = res if isinstance(res, tuple) else (res,)
        loss = sum((r.double() ** 2).sum() for r in res)
        grads = th.autograd.grad(loss, xs, allow_unused=True)
        return [r.detach() for r in res], [th.zeros_like(x) if g is None else g for g, x in zip(grads, xs)]
    finally:
        for k, s in steps.items():
            s.apply = saved[k]


def _through_layer(lay, steps, inputs, dtype=th.float64):
    lay.graph(*inputs)
    for c in lay.calls:
        c.fused.apply = (lambda *a, f=c.fused: f.naive(*a, dtype=dtype))
    saved = {k: s.apply for k, s in steps.items()}
    for s in steps.values():
        s.apply = (lambda *a, s=s: s.naive(*a, dtype=dtype))
    try:
        xs = [i.detach().clone().requires_grad_() for i in inputs]
        res = lay(*xs)
        res = res if isinstance(res, tuple) else (res,)
        loss = sum((r.double() ** 2).sum() for r in res)
        grads = th.autograd.grad(loss, xs, allow_unused=True)
        return [r.detach() for r in res], [th.zeros_like(x) if g is None else g for g, x in zip(grads, xs)]
    finally:
        for k, s in steps.items():
            s.apply = saved[k]


# what must have moved into the step, per raw-projection layer (operator names as the tracer records them)
MOVED = {
    'rwkv7': {'softplus', 'sigmoid', 'div', 'neg'},
    'gla': {'softplus', 'div', 'mul'},
    'delta_rule': {'div', 'sigmoid'},
    'gated_delta_rule': {'div', 'softplus', 'sigmoid', 'add'},
    'mamba2': {'softplus', 'add'},
    'mamba': {'softplus', 'add'},
    'hgrn': {'sigmoid', 'softplus', 'rsub'},
}


@pytest.mark.parametrize('reductions', [False, True])
@pytest.mark.parametrize('op', examples.RAW_OPS)
def test_preparation_moves_into_the_step(op, reductions):
    inputs, layer, steps = examples.build(op, DIMS['B'], DIMS['T'], DIMS['D'], DIMS['C'], 'cpu', raw=True)
    inputs = [i.double() for i in inputs]
    lay = flex_rnn_amd.layer(layer, reductions=reductions)
    got, ggot = _through_layer(lay, steps, inputs)
    assert len(lay.calls) == 1 and MOVED[op] <= set(lay.calls[0].moved), lay.calls and lay.calls[0].moved
    # norms along the column axis move only on request; otherwise they stay in the graph
    normalises = op in ('rwkv7', 'delta_rule', 'gated_delta_rule')
    assert ('linalg_vector_norm' in lay.calls[0].moved) == (normalises and reductions)
    assert ('linalg_vector_norm' in lay.graph(*inputs).code) == (normalises and not reductions)
    want, gwant = _eager(layer, steps, inputs)
    recurrence.assert_all_close(got + ggot, want + gwant, 1e-10, op)


def test_time_invariant_preparation_stays_outside():
    """`-exp(A_log)` of a per-head parameter does not vary with time: it is evaluated once, eagerly, and enters the
    fused step as a raw input; what varies with time (softplus of the step size plus a bias) moves."""
    inputs, layer, steps = examples.build('mamba2', 2, 6, 32, 16, 'cpu', raw=True)
    lay = flex_rnn_amd.layer(layer)
    gm = lay.graph(*inputs)
    assert 'exp' in gm.code and 'exp' not in lay.calls[0].moved
    assert 'softplus' not in gm.code and 'softplus' in lay.calls[0].moved


@pytest.mark.parametrize('op', examples.OPS)
def test_adapters_without_preparation_run_unchanged(op):
    """The reference's own adapters (views only, chained steps with eager operations between them): nothing moves,
    results are those of the adapter itself."""
    inputs, layer, steps = examples.build(op, 2, 6, 32, 16, 'cpu')
    inputs = [i.double() for i in inputs]
    lay = flex_rnn_amd.layer(layer)
    got, ggot = _through_layer(lay, steps, inputs)
    want, gwant = _eager(layer, steps, inputs)
    moved = {m for c in lay.calls for m in c.moved}
    assert moved <= {'softmax', 'div', 'mul', 'add', 'abs', 'maximum', 'exp', 'neg', 'reciprocal', 'rsub', 'pow'}, moved
    recurrence.assert_all_close(got + ggot, want + gwant, 1e-10, op)


def test_reduction_over_rows_is_left_in_the_graph():
    """A value normalised over the axis that becomes the state's *row* axis cannot move (a step may only sum along
    columns): the norm stays eager, the division by it moves."""
    st = flex_rnn_amd.jit(ops.gla)

    def layer(q, k, v, g, s):
        v = F.normalize(v, dim=-1) * 2.0
        g = -F.softplus(g)
        q, k, v, g = [i.unsqueeze(-2) for i in (q, k, v, g)]
        y, s = st(q, k, v.mT, g, s.mT)
        return y, s.mT

    gen = th.Generator().manual_seed(1)
    inputs = [th.randn(2, 5, 2, 8, generator=gen, dtype=th.float64) for _ in range(4)] + [th.randn(2, 2, 8, 8, generator=gen, dtype=th.float64)]
    lay = flex_rnn_amd.layer(layer)
    got, ggot = _through_layer(lay, {'s': st}, inputs)
    assert 'linalg_vector_norm' in lay.graph(*inputs).code and 'linalg_vector_norm' not in lay.calls[0].moved
    assert {'softplus', 'div'} <= set(lay.calls[0].moved)
    want, gwant = _eager(layer, {'s': st}, inputs)
    recurrence.assert_all_close(got + ggot, want + gwant, 1e-10, 'row normalisation')


def test_merged_head_axis_and_shared_raw_tensor():
    """Projections arrive as [B, T, H*C]; the reshape that splits the head axis follows the preparation, and one raw
    tensor feeds two step inputs (key and, negated and gated, the removal direction)."""
    st = flex_rnn_amd.jit(ops.rwkv7_decay)
    B, T, H, C = 2, 5, 2, 8

    def layer(r, w, k, v, g, s):
        w = th.exp(-th.exp(w))
        kk = F.normalize(k.view(B, T, H, C), dim=-1).view(B, T, H * C)
        a, b = -kk, kk * th.sigmoid(g)
        r, w, k, v, a, b = [i.view(B, T, H, 1, C) for i in (r, w, k, v, a, b)]
        y, s = st(r, w, k, v.mT, a, b, s.mT)
        return y.reshape(B, T, H * C), s.mT

    gen = th.Generator().manual_seed(2)
    inputs = [th.randn(B, T, H * C, generator=gen, dtype=th.float64) * 0.5 for _ in range(5)] + [th.randn(B, H, C, C, generator=gen, dtype=th.float64)]
    lay = flex_rnn_amd.layer(layer, reductions=True)
    got, ggot = _through_layer(lay, {'s': st}, inputs)
    assert len(lay.calls[0].raw_signatures) == 5, lay.calls[0].raw_signatures      # r, w, k (once), v, g
    assert {'exp', 'linalg_vector_norm', 'sigmoid', 'neg'} <= set(lay.calls[0].moved)
    want, gwant = _eager(layer, {'s': st}, inputs)
    recurrence.assert_all_close(got + ggot, want + gwant, 1e-10, 'merged heads')
