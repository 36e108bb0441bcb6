"""TEST INFRASTRUCTURE ONLY - CPU oracle for the recurrence.

`run_loop` restates the reference's `jit.naive` (/root/reference/flex_rnn/jit.py:23-36;
README.md:28-38 `simplified_naive`): for every timestep, slice each `[B|1,T|1,H|1,M|1,N|1]`
input at `t` (broadcasting a size-1 time axis), cast inputs (not the state) to `dtype`,
call the user's single-step function on `[B|1,H|1,m,n]` tensors, collect the `[B,H,M,1]`
outputs into `[B,T,H,M]`.

Pinned by (tests/test_oracle.py):
  * closed form of decay-only linear attention  S_t = S_{t-1}*w_t + v_t k_t^T   (masked matmul),
  * closed form of the N=1 gated scan            s_t = g_t s_{t-1} + x_t         (cumulative products),
  * one-step delta rule                          a single rank-1 update,
  * Mamba with constant delta, A                 geometric series,
  * invariants: batch/head permutation, broadcast vs materialised input, chunked call with
    state hand-off.
Gradients of the oracle are `torch.autograd.grad` through this loop (what
/root/reference/flex_rnn/check_grad.py:30-35 does), pinned by `torch.autograd.gradcheck`
in fp64 on tiny shapes.
"""
from __future__ import annotations

import torch


def _tup(x):
    return tuple(x) if isinstance(x, (tuple, list)) else (x,)


def run_loop(step, inputs, states, dtype=torch.float64):
    """Returns (outputs [B,T,H,M] each, final states [B,H,M,N] each), all in `dtype`
    arithmetic (states are promoted by the arithmetic, as in the reference)."""
    T = max(x.shape[1] for x in inputs)
    st = tuple(states)
    cols = None
    for t in range(T):
        xs = []
        for x in inputs:
            xt = x[:, t] if x.shape[1] == T and T != 1 else x[:, 0]
            xs.append(xt.to(dtype))
        y, st = step(*xs, *st)
        y, st = _tup(y), _tup(st)
        if cols is None:
            cols = [[] for _ in y]
        for acc, v in zip(cols, y):
            acc.append(v.squeeze(-1))
    outs = tuple(torch.stack(c, dim=1) for c in cols)
    return outs, st


def rel_err(a, b):
    """Error metric of the reference's checker (/root/reference/flex_rnn/check_grad.py:20):
    ||a-b||_2 / max(||b||_2, 1e-30), `b` being the trusted value."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    return float((a - b).norm() / max(float(b.norm()), 1e-30))


def loop_with_grads(step, inputs, states, douts, dstates, dtype=torch.float64):
    """Forward through `run_loop` and gradients of sum(<out,dout>) + sum(<stateT,dstate>)
    with respect to every input and initial state.  Returns (outs, final_states, dinputs, dstates0)."""
    xs = [x.detach().clone().to(dtype).requires_grad_() for x in inputs]
    ss = [s.detach().clone().to(dtype).requires_grad_() for s in states]
    outs, fin = run_loop(step, xs, ss, dtype)
    ys = list(outs) + list(fin)
    gs = [g.to(dtype) for g in list(douts) + list(dstates)]
    grads = torch.autograd.grad(ys, xs + ss, grad_outputs=gs, allow_unused=True)
    grads = [torch.zeros_like(p) if g is None else g for g, p in zip(grads, xs + ss)]
    return outs, fin, grads[:len(xs)], grads[len(xs):]
