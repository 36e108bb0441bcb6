"""TEST INFRASTRUCTURE ONLY - CPU executor of the partitioned plan.

Runs the dataflow the three GPU kernels implement, with torch ops on whole
`[B,H,M,N]` tensors, so that the *graph partition* (which sums are saved as `aux` /
`daux`, what is recomputed from checkpoints, how sums over the row axis are
accumulated and post-processed) is checked against autograd of the plain loop
before any kernel is involved.  The dataflow restated here is the reference's
two-pass scheme, /root/reference/flex_rnn/twopass.py:202-220 (forward with state
checkpoints every dT steps and per-step aux), 245-273 (reverse d_state scan with
d_state checkpoints, column grads, daux) and 285-339 (per-chunk recompute, per-row
accumulation of row/scalar/matrix grads).

Pinned by tests/test_partition.py: equality (fp64, 1e-10) with
`oracle.recurrence.loop_with_grads` on every example step function.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch

_UN = {
    'exp': torch.exp, 'neg': torch.neg, 'reciprocal': torch.reciprocal, 'log': torch.log,
    'sqrt': torch.sqrt, 'rsqrt': torch.rsqrt, 'sigmoid': torch.sigmoid, 'tanh': torch.tanh,
    'abs': torch.abs, 'relu': torch.relu, 'sign': torch.sign, 'log1p': torch.log1p,
    'expm1': torch.expm1, 'copy': lambda x: x, 'sin': torch.sin, 'cos': torch.cos, 'erf': torch.erf,
    'log2': torch.log2, 'exp2': torch.exp2,
}
_BIN = {
    'mul': torch.mul, 'add': torch.add, 'sub': torch.sub, 'div': torch.div,
    'lt': torch.lt, 'gt': torch.gt, 'le': torch.le, 'ge': torch.ge, 'eq': torch.eq, 'ne': torch.ne,
    'maximum': torch.maximum, 'minimum': torch.minimum,
}


def eval_graph(g, env: Dict[str, torch.Tensor], dtype) -> List[torch.Tensor]:
    """Evaluate IR graph `g`; `env` maps its (used) input names to tensors whose last two
    dims are the value's [m|1, n|1]."""
    env = dict(env)

    def get(a):
        if isinstance(a, str):
            return env[a]
        return torch.tensor(float(a), dtype=dtype)

    for n in g.nodes:
        if n.op == 'const':
            r = torch.full((1, 1), float(n.args[0]), dtype=dtype)
        elif n.op in _UN:
            r = _UN[n.op](get(n.args[0]))
        elif n.op in _BIN:
            r = _BIN[n.op](get(n.args[0]), get(n.args[1]))
            if r.dtype == torch.bool:
                r = r.to(dtype)
        elif n.op == 'where':
            r = torch.where(get(n.args[0]) != 0, get(n.args[1]), get(n.args[2]))
        elif n.op == 'sum':
            r = get(n.args[0]).sum(dim=tuple(d - 2 for d in n.dims), keepdim=True)
        else:
            raise NotImplementedError(n.op)
        env[n.name] = r
    return [env[o] for o in g.outputs]


def _slice_t(x, t):
    return x[:, t] if x.shape[1] > 1 else x[:, 0]


def run_plan(part, inputs: Sequence[torch.Tensor], states: Sequence[torch.Tensor],
             douts: Sequence[torch.Tensor], dstatesT: Sequence[torch.Tensor], DT: int,
             dtype=torch.float64):
    """Returns (outs, final_states, dinputs, dstates0) computed through the partition."""
    B = max(x.shape[0] for x in inputs)
    T = max(x.shape[1] for x in inputs)
    H = max(x.shape[2] for x in inputs)
    M, N = states[0].shape[-2:]
    assert T % DT == 0
    nin, nst, nout = part.ninputs, part.nstates, part.noutputs
    xs = [x.to(dtype) for x in inputs]
    naux, ndaux = len(part.aux), len(part.daux)

    def bind_inputs(g, t):
        return {name: _slice_t(x, t) for name, x in zip(part.in_names, xs)}

    # ------------------------------------------------------------------ forward
    S = [s.to(dtype) for s in states]
    ckpt, aux_hist, outs = [], [], [[] for _ in range(nout)]
    for t in range(T):
        if t % DT == 0:
            ckpt.append([s.clone() for s in S])
        env = bind_inputs(part.fw, t)
        env.update(dict(zip(part.st_names, S)))
        res = eval_graph(part.fw, env, dtype)
        y, S, aux = res[:nout], res[nout:nout + nst], res[nout + nst:]
        S = [s.expand(B, H, M, N) for s in S]
        aux_hist.append(aux)
        for acc, v in zip(outs, y):
            acc.append(v.expand(B, H, M, 1).squeeze(-1))
    outs = tuple(torch.stack(o, dim=1) for o in outs)
    final = tuple(S)

    # ------------------------------------------------------------------ reverse scan
    def recompute_chunk(c):
        hist = [ckpt[c]]
        for t in range(c * DT, c * DT + DT - 1):
            env = bind_inputs(part.restep, t)
            env.update(dict(zip(part.st_names, hist[-1])))
            env.update(dict(zip(part.aux, aux_hist[t])))
            hist.append([s.expand(B, H, M, N) for s in eval_graph(part.restep, env, dtype)])
        return hist

    D = [d.to(dtype) for d in dstatesT]
    dmat = {i: torch.zeros(B, H, M, N, dtype=dtype) for i in part.mat_idx}
    dck = [None] * (T // DT)
    dcol = {i: [None] * T for i in part.col_idx}
    daux_hist = [None] * T
    hist, hist_c = None, -1
    for t in range(T - 1, -1, -1):
        if (t + 1) % DT == 0:
            dck[t // DT] = [d.clone() for d in D]
        env = bind_inputs(part.dstep, t)
        if part.dstep_needs_state:
            if hist_c != t // DT:
                hist, hist_c = recompute_chunk(t // DT), t // DT
            env.update(dict(zip(part.st_names, hist[t % DT])))
        env.update(dict(zip(part.aux, aux_hist[t])))
        env.update({n: _slice_t(d.to(dtype).unsqueeze(-1), t) for n, d in zip(part.dout_names, douts)})
        env.update(dict(zip(part.dnst_names, D)))
        res = eval_graph(part.dstep, env, dtype)
        D = [d.expand(B, H, M, N) for d in res[:nst]]
        for k, i in enumerate(part.col_idx):
            dcol[i][t] = res[nst + k].expand(B, H, M, 1)
        daux_hist[t] = res[nst + len(part.col_idx):nst + len(part.col_idx) + ndaux]
        if part.mat_in_dstep:
            for k, i in enumerate(part.mat_idx):
                dmat[i] = dmat[i] + res[nst + len(part.col_idx) + ndaux + k].expand(B, H, M, N)
    dstate0 = tuple(D)

    # ------------------------------------------------------------------ gradient pass
    nm = part.joint.node_map()
    rs = part.row_idx + part.scalar_idx
    drs = {i: [None] * T for i in rs}
    mats_drow = [] if part.mat_in_dstep else list(part.mat_idx)
    for c in range(T // DT):
        hist = recompute_chunk(c)
        D = dck[c]
        for t in range(c * DT + DT - 1, c * DT - 1, -1):
            env = bind_inputs(part.drow, t)
            env.update(dict(zip(part.st_names, hist[t % DT])))
            env.update(dict(zip(part.aux, aux_hist[t])))
            env.update(dict(zip(part.daux, daux_hist[t])))
            env.update({n: _slice_t(d.to(dtype).unsqueeze(-1), t) for n, d in zip(part.dout_names, douts)})
            env.update(dict(zip(part.dnst_names, D)))
            res = eval_graph(part.drow, env, dtype)
            D = [d.expand(B, H, M, N) for d in res[:nst]]
            for k, i in enumerate(mats_drow):
                dmat[i] = dmat[i] + res[nst + k].expand(B, H, M, N)
            ops = res[nst + len(mats_drow):]
            # accumulate the sums over the row axis, then run the epilogue
            eenv = bind_inputs(part.epi, t)
            eenv.update(dict(zip(part.aux, aux_hist[t])))
            for name, operand in zip(part.msums, ops):
                node = nm[name]
                em, en = part.joint.ext(node.args[0])
                full = operand.expand(B, H, M if em else 1, N if en else 1)
                eenv[name] = full.sum(dim=tuple(d - 2 for d in node.dims), keepdim=True)
            eres = eval_graph(part.epi, eenv, dtype)
            for k, i in enumerate(rs):
                drs[i][t] = eres[k]

    # ------------------------------------------------------------------ assemble, reduce broadcast dims
    def finish(i, per_t):
        x = inputs[i]
        tgt = (B, H) + tuple(x.shape[-2:])
        g = torch.stack([p.expand(B, H, *p.shape[-2:]).expand(*tgt) if p.shape[-2:] == x.shape[-2:]
                         else p.expand(B, H, *x.shape[-2:]) for p in per_t], dim=1)   # [B,T,H,m,n]
        for d in range(3):
            if x.shape[d] == 1 and g.shape[d] != 1:
                g = g.sum(dim=d, keepdim=True)
        return g

    dinputs = []
    for i in range(nin):
        if i in part.col_idx:
            dinputs.append(finish(i, dcol[i]))
        elif i in rs:
            dinputs.append(finish(i, drs[i]))
        else:
            g = dmat[i].unsqueeze(1)
            x = inputs[i]
            for d in (0, 2):
                if x.shape[d] == 1 and g.shape[d] != 1:
                    g = g.sum(dim=d, keepdim=True)
            dinputs.append(g)
    return outs, final, dinputs, dstate0
