"""Runs one recurrence through the emitted kernels on the CPU (hipsim) and compares with the
oracle.  Executed as a subprocess by tests/test_emit_sim.py so that a guard-page hit (SIGSEGV)
fails one test instead of the whole session.

usage: run_case.py <case> B,T,H,M,N <f32|bf16|f16> <against_end 0|1> [tol]
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

if os.environ.get('HIPSIM_CANDIDATES', '0') == '1':
    # every candidate is run; the choice among them goes to a scratch directory, never to the product's cache
    import tempfile
    os.environ['FLEX_RNN_CACHE'] = tempfile.mkdtemp(prefix='frnn_hipsim_picks_')
    os.environ['FLEX_RNN_RETUNE'] = '1'
os.environ.setdefault('FLEX_RNN_CHECK', '1')        # the product's launch audit runs on every simulated launch

import torch as th

import cases
from flex_rnn_amd import configs, planner
from hipsim import SimPlan
from oracle import recurrence


def main():
    name, dims, dt, end = sys.argv[1], tuple(int(v) for v in sys.argv[2].split(',')), sys.argv[3], int(sys.argv[4])
    dtype = {'f32': th.float32, 'bf16': th.bfloat16, 'f16': th.float16, 'f64': th.float64}[dt]
    tol = float(sys.argv[5]) if len(sys.argv) > 5 else {'f32': 2e-5, 'f64': 2e-5, 'bf16': 1e-2, 'f16': 3e-3}[dt]
    if name.startswith('pattern:'):
        # gated linear attention with a per-step scalar gain; inputs q, k, v, g, c with the given spans
        def step(q, k, v, g, c, S):
            S = S * th.sigmoid(g) + c * (v * k)
            return (S * q).sum(-1, True), S
        spec = [tuple(p.split(':')) for p in name[len('pattern:'):].split(',')]
        table = {'pat': (step, [(c, sp) for c, sp in spec], 1)}
        step, xs, ss = cases.make_inputs('pat', *dims, dtype=dtype, table=table)
        ss = [th.randn(dims[0], dims[2], dims[3], dims[4], generator=th.Generator().manual_seed(3)).to(dtype) * 0.3]
    elif name.startswith('gen:'):
        step, spec, nst, src = cases.random_step(int(name[4:]))
        print(src)
        step, xs, ss = cases.make_inputs('gen', *dims, dtype=dtype, table={'gen': (step, spec, nst)})
    elif name.startswith('layer:') or name.startswith('layer+:'):
        # the step a traced layer runs instead of the user's (flex_rnn_amd.layer: input preparation moved into the step;
        # `layer+:` also moves norms along the column axis), on the raw tensors the rewritten layer hands it
        full, name = name.startswith('layer+:'), 'layer:' + name.split(':', 1)[1]
        import flex_rnn_amd
        from flex_rnn_amd import examples
        B, T, H, M, N = dims
        assert M == N or name[6:] in ('mamba', 'hgrn')
        inputs, layer, _ = examples.build(name[6:], B, T, H * M, M, 'cpu', raw=True)
        inputs = [i.to(dtype) for i in inputs]
        lay = flex_rnn_amd.layer(layer, reductions=full)
        lay.graph(*inputs)
        call, = lay.calls
        seen = {}

        def capture(*a):
            seen['args'] = a
            return call.fused.naive(*a)

        call.fused.apply = capture
        lay(*inputs)
        step = call.fused.step
        xs, ss = list(seen['args'][:call.fused.ninputs]), list(seen['args'][call.fused.ninputs:])
        ss = [(th.randn(s.shape, generator=th.Generator().manual_seed(4)) * 0.3).to(dtype) for s in ss]
    elif name.startswith('cfg:'):
        wl = configs.make(name[4:], dims=dims, dtype=dtype)
        step, xs, ss = wl.step, wl.inputs, wl.states
    else:
        step, xs, ss = cases.make_inputs(name, *dims, dtype=dtype)
    plan, fm, bm = planner.make_plan(step, xs, ss)
    nout, nst = plan.part.noutputs, plan.part.nstates
    sp = SimPlan(plan, state_meta=fm[nout:nout + nst], against_end=bool(end))
    res = sp.forward(tuple(xs), tuple(ss))
    outs, stT, sck, aux = res[:nout], res[nout:nout + nst], res[nout + nst:nout + 2 * nst], res[-1]
    # the inference kernel (no checkpoints, no saved sums) must give the same outputs and final states
    lean = sp.forward_only(tuple(xs), tuple(ss))
    for a, b in zip(lean, list(outs) + list(stT)):
        assert th.equal(a, b) or recurrence.rel_err(a, b) < 1e-6, 'forward_only differs from forward'
    g = th.Generator().manual_seed(11)
    dy = [th.randn(o.shape, generator=g) for o in outs]
    dS = [th.randn(s.shape, generator=g) for s in ss]
    dins, dst0 = sp.backward(tuple(d.to(o.dtype) for d, o in zip(dy, outs)),
                             tuple(d.to(s.dtype) for d, s in zip(dS, stT)), tuple(xs), sck, aux)
    dyq = [d.to(o.dtype) for d, o in zip(dy, outs)]
    dSq = [d.to(s.dtype) for d, s in zip(dS, stT)]
    want = recurrence.loop_with_grads(step, xs, ss, dyq, dSq)
    got = list(outs) + list(stT) + list(dins) + list(dst0)
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    print(f'{name} {dims} {dt} tile={plan.tile}', flush=True)
    worst = max(recurrence.assert_all_close(got, want, tol, name))
    ran = sorted({f'{k}#{i}' for k, i in sp.launches})
    print(f'{name} {dims} {dt} tile={plan.tile} worst={worst:.3e} lds={sp.lds_peak} candidate launches compared with the first: {getattr(sp, "compared", 0)} builds run: {" ".join(ran)}')


if __name__ == '__main__':
    main()
