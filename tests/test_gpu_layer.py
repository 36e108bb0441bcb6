"""`flex_rnn_amd.layer` on the GPU: the 14 example layers through their unmodified adapters, and the raw-projection
layers whose preparation moves into the kernels, against the oracle loop applied to the eager layer in fp64
(tolerances of the parity tests: 1e-4 for fp32 I/O, 1e-2 for bf16 I/O)."""
import pytest
import torch as th

import flex_rnn_amd
from flex_rnn_amd import examples
from oracle import recurrence

import warm

pytestmark = pytest.mark.gpu


def _oracle_apply(step_obj):
    def run(*args):
        xs, ss = args[:step_obj.ninputs], args[step_obj.ninputs:]
        outs, st = recurrence.run_loop(step_obj.step, xs, ss, dtype=th.float64)
        return (*outs, *st)
    return run


@pytest.mark.parametrize('op,raw,dtype,reductions', warm.LAYER_CASES)
def test_layer_against_oracle(op, raw, dtype, reductions):
    print(f'case layer {op} raw={raw} {dtype} reductions={reductions}', flush=True)
    a = warm.EXAMPLE_ARGS
    inputs, layer, steps = examples.build(op, a['B'], a['T'], a['D'], a['C'], 'cuda', raw=raw)
    inputs = [i.to(dtype) for i in inputs]
    lay = flex_rnn_amd.layer(layer, reductions=reductions)
    xs = [i.clone().requires_grad_() for i in inputs]
    res = lay(*xs)
    res = res if isinstance(res, tuple) else (res,)
    if raw:
        assert len(lay.calls) == 1 and lay.calls[0].moved, 'nothing moved into the step'
    g = th.Generator().manual_seed(7)
    douts = [th.randn(r.shape, generator=g).to(r.device, r.dtype) for r in res]
    grads = th.autograd.grad(res, xs, grad_outputs=douts, allow_unused=True)
    # reference: the layer as written, on fp64 copies of the same inputs, every step on the oracle loop
    saved = {k: s.apply for k, s in steps.items()}
    for s in steps.values():
        s.apply = _oracle_apply(s)
    try:
        xr = [i.double().requires_grad_() for i in inputs]
        want = layer(*xr)
        want = want if isinstance(want, tuple) else (want,)
        gwant = th.autograd.grad(want, xr, grad_outputs=[d.double() for d in douts], allow_unused=True)
    finally:
        for k, s in steps.items():
            s.apply = saved[k]
    zero = lambda gs, ps: [th.zeros_like(p) if g_ is None else g_ for g_, p in zip(gs, ps)]
    recurrence.assert_all_close(list(res) + zero(grads, xs), list(want) + zero(gwant, xr),
                                1e-2 if dtype == th.bfloat16 else 1e-4, f'layer {op} raw={raw}')
