"""GPU parity: the compiled HIP path against the CPU oracle on the five benchmark
workloads (reduced B, T, H; same state shape M x N as the full configurations).

Tolerances (max over outputs, final states and all gradients of ||a-b|| / ||b||, b = oracle
in fp64 on the same cast inputs): 1e-4 for fp32 I/O, 1e-2 for bf16 I/O.
"""
import pytest
import torch as th

import flex_rnn_amd
from flex_rnn_amd import configs, prebuild
from oracle import recurrence

pytestmark = pytest.mark.gpu

TOL = {th.float32: 1e-4, th.bfloat16: 1e-2, th.float16: 1e-2}


def run_case(name, dims, dtype, seed=0):
    wl = configs.make(name, dims=dims, dtype=dtype, seed=seed)
    dy, dS = configs.upstream_grads(wl, seed=seed + 1)
    # oracle on the CPU, fp64 arithmetic on the (already cast) input values
    want = recurrence.loop_with_grads(wl.step, wl.inputs, wl.states, dy, dS, dtype=th.float64)
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    f = flex_rnn_amd.jit(wl.step)
    xs = [x.cuda().requires_grad_() for x in wl.inputs]
    ss = [s.cuda().requires_grad_() for s in wl.states]
    res = f(*xs, *ss)
    grads = th.autograd.grad(res, xs + ss, grad_outputs=[g.cuda().to(r.dtype) for g, r in zip(dy + dS, res)])
    th.cuda.synchronize()
    got = list(res) + list(grads)
    errs = recurrence.assert_all_close(got, want, TOL[wl.dtype], f'{name} {dims}')
    return errs, got, wl


@pytest.mark.parametrize('name,dims,dtype', [(n, d, t) for n, d, t in prebuild.CASES if d is not None or n == 'delta_rule'])
def test_parity_reduced(name, dims, dtype):
    print(f'case {name} {dims} {dtype}', flush=True)
    errs, got, wl = run_case(name, dims, dtype)
    tol = TOL[wl.dtype]
    print('rel errors', ['%.2e' % e for e in errs], flush=True)
    assert max(errs) < tol, (name, errs)


@pytest.mark.parametrize('name', ['delta_rule', 'mamba1', 'mamba2', 'rwkv7', 'gated_delta_rule'])
def test_committed_vectors(name):
    """The compiled path on the inputs of tests/golden/five_configs_fp64.npz (fp32 I/O) against the
    stored fp64 results: <= 1e-4."""
    import os
    import numpy as np
    print(f'case golden {name}', flush=True)
    z = np.load(os.path.join(os.path.dirname(__file__), 'golden', 'five_configs_fp64.npz'))

    def arrs(key):
        out, i = [], 0
        while f'{name}.{key}{i}' in z:
            out.append(th.from_numpy(z[f'{name}.{key}{i}']))
            i += 1
        return out
    step = configs.make(name, dims=(1, 2, 1, 2, 2), dtype=th.float32).step
    xs = [x.float().cuda().requires_grad_() for x in arrs('in')]
    ss = [s.float().cuda().requires_grad_() for s in arrs('st')]
    res = flex_rnn_amd.jit(step)(*xs, *ss)
    grads = th.autograd.grad(res, xs + ss, [g.float().cuda() for g in arrs('dy') + arrs('dS')])
    want = arrs('out') + arrs('stT') + arrs('din') + arrs('dst')
    recurrence.assert_all_close(list(res) + list(grads), want, 1e-4, f'golden {name}')
