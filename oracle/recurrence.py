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

`rel_err` / `assert_close` are the metric and the assertion of every parity test
(/root/reference/flex_rnn/check_grad.py:20).  Pinned by known values (3-4-5 triangle, the 1e-30
floor for a zero reference, promotion of bf16 operands to double, asymmetry in its arguments) and
by negative tests: a result off by twice the tolerance must fail `assert_close`.

`chunked_loop_with_grads` is `loop_with_grads` with bounded memory for long sequences: the same
loop and the same autograd, one chunk of timesteps at a time, the gradient of the chunk's entry
state handed back to the chunk before.  Pinned by equality (fp64, 1e-12) with `loop_with_grads`
on short sequences, chunk lengths that do not divide T and time-broadcast inputs included.
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


def assert_close(got, want, tol, what=''):
    """The parity assertion: `rel_err(got, want) < tol` (and equal shapes); returns the error."""
    assert tuple(got.shape) == tuple(want.shape), f'{what}: shape {tuple(got.shape)} != {tuple(want.shape)}'
    e = rel_err(got, want)
    assert e == e and e < tol, f'{what}: relative error {e:.3e} is not below {tol:.1e}'
    return e


def assert_all_close(got, want, tol, what=''):
    """`assert_close` over two equally long sequences of tensors; returns the list of errors."""
    got, want = list(got), list(want)
    assert len(got) == len(want), f'{what}: {len(got)} results, {len(want)} expected'
    return [assert_close(a, b, tol, f'{what} #{i}') for i, (a, b) in enumerate(zip(got, want))]


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


def chunked_loop_with_grads(step, inputs, states, douts, dstates, chunk, dtype=torch.float64):
    """Same results as `loop_with_grads`, holding the autograd graph of only `chunk` timesteps at
    a time: a forward sweep without graph keeps the state at every chunk boundary; a reverse sweep
    re-runs each chunk from its boundary state with a graph, differentiates
    sum(<out_chunk, dout_chunk>) + <state at chunk end, its gradient> and hands the gradient of
    the chunk's entry state to the chunk before.  Gradients of inputs without a time axis are
    summed over the chunks.  Returns (outs, final_states, dinputs, dstates0)."""
    T = max(x.shape[1] for x in inputs)
    xs = [x.detach().to(dtype) for x in inputs]
    timed = [x.shape[1] == T and T != 1 for x in xs]
    bounds = list(range(0, T, chunk))
    entry, outs_c = [], []
    st = tuple(s.detach().to(dtype) for s in states)
    with torch.no_grad():
        for t0 in bounds:
            entry.append(st)
            sl = [x[:, t0:t0 + chunk] if td else x for x, td in zip(xs, timed)]
            o, st = run_loop(step, sl, st, dtype)
            outs_c.append(o)
    outs = tuple(torch.cat([o[k] for o in outs_c], dim=1) for k in range(len(outs_c[0])))
    fin = st
    dins = [torch.zeros_like(x) for x in xs]
    dst = [g.detach().to(dtype) for g in dstates]
    gouts = [g.detach().to(dtype) for g in douts]
    for ci in range(len(bounds) - 1, -1, -1):
        t0 = bounds[ci]
        sl = [(x[:, t0:t0 + chunk] if td else x).clone().requires_grad_() for x, td in zip(xs, timed)]
        s_in = [s.clone().requires_grad_() for s in entry[ci]]
        o, s_out = run_loop(step, sl, s_in, dtype)
        ys = list(o) + list(s_out)
        gs = [g[:, t0:t0 + chunk] for g in gouts] + list(dst)
        grads = torch.autograd.grad(ys, sl + s_in, grad_outputs=gs, allow_unused=True)
        grads = [torch.zeros_like(p) if g is None else g for g, p in zip(grads, sl + s_in)]
        for i, td in enumerate(timed):
            if td:
                dins[i][:, t0:t0 + chunk] = grads[i]
            else:
                dins[i] += grads[i]
        dst = [g.detach() for g in grads[len(sl):]]
    return outs, fin, dins, dst
