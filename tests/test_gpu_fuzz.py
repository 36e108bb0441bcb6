"""Random recurrences (tests/cases.py: random_step) on the GPU against the oracle: the same seeds and
sizes that tests/test_emit_sim.py runs through the emitted kernels on the CPU, where every buffer
sits against a guard page.  On the GPU they additionally cover what the CPU harness replaces: the DPP
and lane-swap reductions, the hardware exp2 / log2, and the timed choice among candidate builds."""
import pytest
import torch as th

import flex_rnn_amd
from oracle import recurrence

import cases

pytestmark = pytest.mark.gpu
TOL = {th.float32: 1e-4, th.bfloat16: 1e-2}


@pytest.mark.parametrize('seed', cases.FUZZ_SEEDS)
def test_random_recurrence(seed):
    dtype = (th.float32, th.bfloat16)[(seed // 6) % 2]
    print(f'case random recurrence {seed} {cases.FUZZ_DIMS[seed % 6]} {dtype}', flush=True)
    step, xs, ss = cases.fuzz_case(seed, dtype)
    f = flex_rnn_amd.jit(step, n_step_args=len(xs) + len(ss))
    xg = [x.cuda().requires_grad_() for x in xs]
    sg = [s.cuda().requires_grad_() for s in ss]
    out = f(*xg, *sg)
    g = th.Generator().manual_seed(11)
    dout = [th.randn(o.shape, generator=g).to(o.dtype) for o in out]
    grads = th.autograd.grad(out, xg + sg, [d.cuda() for d in dout], allow_unused=True)
    want = recurrence.loop_with_grads(step, xs, ss, dout[:f.noutputs], dout[f.noutputs:])
    want = [*want[0], *want[1], *want[2], *want[3]]
    got = [o.detach().cpu() for o in out] + [th.zeros_like(x) if gr is None else gr.cpu() for gr, x in zip(grads, xs + ss)]
    recurrence.assert_all_close(got, want, TOL[dtype], f'seed {seed}')
    # the inference kernel agrees with the training forward
    lean = f.infer(*[x.cuda() for x in xs], *[s.cuda() for s in ss])
    for a, b in zip(lean, out):
        assert recurrence.rel_err(a.float(), b.detach().float()) < 1e-5 or th.equal(a, b.detach())
