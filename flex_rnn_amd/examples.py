"""Command-line examples: the 14 recurrences the reference demonstrates, written against
layer-shaped tensors ([B,T,H,C] etc.) with the unsqueeze / `.mT` adapters, and checked against
the pure-PyTorch loop or benchmarked.

    python -m flex_rnn_amd.examples --op rwkv7 --check-flex
    python -m flex_rnn_amd.examples --op mamba2 --benchmark-flex [--forward] [--torch-compile]

Counterpart of /root/reference/tests/examples.py (ops 37-426, modes 433-466).  The comparisons
with third-party kernels (fla, mamba_ssm, ...) are not available here; `--check-flex` compares
the compiled kernels with `naive_fp64`, as the reference's own check does.
"""
import argparse

import torch as th
import torch.nn.functional as F

import flex_rnn_amd
from flex_rnn_amd import ops

OPS = ['rwkv7', 'rwkv6', 'gla', 'retention', 'delta_rule', 'gated_delta_rule', 'mamba2', 'longhorn', 'rwkv4',
       'hgrn', 'mamba', 's4d', 'gsa', 'mlstm']


RAW_OPS = ['rwkv7', 'gla', 'delta_rule', 'gated_delta_rule', 'mamba2', 'mamba', 'hgrn']


def build(op, B, T, D, C, device, raw=False):
    """Returns (inputs, layer, steps) where layer(*inputs) calls jit-compiled steps through adapters.  With `raw`
    (ops in RAW_OPS) the layer takes the projections as a model produces them and prepares them itself - sigmoid
    and softplus gates, L2-normalised keys, decay parameters - before it adapts shapes and calls the step: the
    form `flex_rnn_amd.layer` is for."""
    H = D // C
    g = th.Generator().manual_seed(0)

    def randn(*shape):
        return th.randn(*shape, generator=g).to(device)

    steps = {}

    def jit(name, fn):
        steps[name] = flex_rnn_amd.jit(fn)
        return steps[name]

    if raw:
        assert op in RAW_OPS, f'no raw-projection form of {op}'
        if op == 'rwkv7':
            inputs = tuple(randn(B, T, H, C) for _ in range(6)) + (randn(B, H, C, C),)
            st = jit('step', ops.rwkv7)

            def layer(r, w, k, v, a, b, s):
                w = -F.softplus(-w) - 0.5                       # log of a decay in (0, exp(-0.5))
                a = F.normalize(a, dim=-1)
                b = -a * th.sigmoid(b)
                r, w, k, v, a, b = [i.unsqueeze(-2) for i in (r, w, k, v, a, b)]
                y, s = st(r, w, k, v.mT, a, b, s.mT)
                return y, s.mT
        elif op == 'gla':
            inputs = tuple(randn(B, T, H, C) for _ in range(4)) + (randn(B, H, C, C),)
            st = jit('step', ops.gla)

            def layer(q, k, v, g_, s):
                g_ = -F.softplus(-g_) / 16                      # log-sigmoid gate with the usual normaliser
                q = q * C ** -0.5
                q, k, v, g_ = [i.unsqueeze(-2) for i in (q, k, v, g_)]
                y, s = st(q, k, v.mT, g_, s.mT)
                return y, s.mT
        elif op in ('delta_rule', 'gated_delta_rule'):
            q, k, v = [randn(B, T, H, C) for _ in range(3)]
            beta = randn(B, T, H)
            if op == 'delta_rule':
                inputs = (q, k, v, beta, randn(B, H, C, C))
                st = jit('step', ops.delta_rule)

                def layer(q, k, v, beta, s):
                    k = F.normalize(k, dim=-1)
                    beta = th.sigmoid(beta)
                    q, k, v, beta = [i.unsqueeze(-2) for i in (q, k, v, beta.unsqueeze(-1))]
                    y, s = st(q, k, v.mT, beta, s.mT)
                    return y, s.mT
            else:
                inputs = (q, k, v, randn(B, T, H), beta, randn(H), randn(H), randn(B, H, C, C))
                st = jit('step', ops.gated_delta_rule)

                def layer(q, k, v, a, beta, A_log, dt_bias, s):
                    q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
                    gate = -A_log.exp() * F.softplus(a + dt_bias)          # log of the gate
                    beta = th.sigmoid(beta)
                    q, k, v, gate, beta = [i.unsqueeze(-2) for i in (q, k, v, gate.unsqueeze(-1), beta.unsqueeze(-1))]
                    y, s = st(q, k, v.mT, gate, beta, s.mT)
                    return y, s.mT
        elif op == 'mamba2':
            inputs = (randn(B, T, H, C), randn(B, T, H), randn(H), randn(H), randn(B, T, 1, C), randn(B, T, 1, C), randn(B, H, C, C))
            st = jit('step', ops.mamba2)

            def layer(x, dt, dt_bias, A_log, b, c, s):
                dt = F.softplus(dt + dt_bias)
                A = -A_log.exp()
                x, dt, A, b, c = [i.unsqueeze(-2) for i in (x, dt.unsqueeze(-1), A[None, None, :, None], b, c)]
                return st(x.mT, dt, A, b, c, s)
        elif op == 'mamba':
            N = 16
            inputs = (randn(B, D, T), randn(B, D, T), randn(D), randn(D, N), randn(B, N, T), randn(B, N, T))
            st = jit('step', ops.mamba)

            def layer(u, dt, dt_bias, A_log, b, c):
                dt = F.softplus(dt + dt_bias[:, None])
                A = -A_log.exp()
                u, dt, b, c = [i.mT[:, :, None, :, None] for i in (u, dt, b, c)]
                s = th.zeros(B, 1, D, N, device=u.device, dtype=u.dtype)
                return st(u, dt, A[None, None, None], b.mT, c.mT, s)[0].squeeze(2).mT
        else:
            inputs = (randn(B, T, D), randn(B, T, D))
            st = jit('step', ops.hgrn)

            def layer(x, gate):
                f = th.sigmoid(gate)
                x, gate = (1 - f) * x, -F.softplus(-gate)       # input gate tied to the forget gate, whose log drives the state
                s = th.zeros(B, 1, D, 1, device=x.device, dtype=x.dtype)
                x, gate = [i[:, :, None, :, None] for i in (x, gate)]
                return st(x, gate, s)[0].squeeze(2)
        return inputs, layer, steps

    if op == 'rwkv7':
        r, w, k, v, a, b = [randn(B, T, H, C) for _ in range(6)]
        w, a = -th.sigmoid(w), F.normalize(a, dim=-1)
        b = -a * th.sigmoid(b)
        inputs = (r, w, k, v, a, b, randn(B, H, C, C))
        st = jit('step', ops.rwkv7)

        def layer(r, w, k, v, a, b, s):
            r, w, k, v, a, b = [i.unsqueeze(-2) for i in (r, w, k, v, a, b)]
            y, s = st(r, w, k, v.mT, a, b, s.mT)
            return y, s.mT
    elif op in ('rwkv6', 'gla'):
        q, k, v, w = [randn(B, T, H, C) for _ in range(4)]
        w = -th.sigmoid(w)
        if op == 'rwkv6':
            inputs = (q, k, v, w, randn(H, C), randn(B, H, C, C))
            st = jit('step', ops.rwkv6)

            def layer(q, k, v, w, u, s):
                q, k, v, w, u = [i.unsqueeze(-2) for i in (q, k, v, w, u[None, None])]
                y, s = st(q, k, v.mT, w, u, s.mT)
                return y, s.mT
        else:
            inputs = (q, k, v, w, randn(B, H, C, C))
            st = jit('step', ops.gla)

            def layer(q, k, v, g_, s):
                q, k, v, g_ = [i.unsqueeze(-2) for i in (q, k, v, g_)]
                y, s = st(q, k, v.mT, g_, s.mT)
                return y, s.mT
    elif op == 'retention':
        q, k, v = [randn(B, T, H, C) for _ in range(3)]
        inputs = (q, k, v, randn(B, H, C, C))
        st = jit('step', ops.retention)
        decay = (1 - 2 ** (-5 - th.arange(H).float())).view(1, 1, H, 1, 1).expand(B, T, H, 1, 1).contiguous().to(device)

        def layer(q, k, v, s):
            q, k, v = [i.unsqueeze(-2) for i in (q, k, v)]
            y, s = st(decay.to(q.dtype), q, k, v.mT, s.mT)
            return y, s.mT
    elif op in ('delta_rule', 'gated_delta_rule'):
        q, k, v = [randn(B, T, H, C) for _ in range(3)]
        k = F.normalize(k, dim=-1)
        beta = randn(B, T, H)
        if op == 'delta_rule':
            inputs = (q, k, v, beta, randn(B, H, C, C))
            st = jit('step', ops.delta_rule)

            def layer(q, k, v, beta, s):
                q, k, v, beta = [i.unsqueeze(-2) for i in (q, k, v, beta.unsqueeze(-1))]
                y, s = st(q, k, v.mT, beta, s.mT)
                return y, s.mT
        else:
            gate = -th.sigmoid(randn(B, T, H))
            inputs = (q, k, v, gate, beta, randn(B, H, C, C))
            st = jit('step', ops.gated_delta_rule)

            def layer(q, k, v, gate, beta, s):
                q, k, v, gate, beta = [i.unsqueeze(-2) for i in (q, k, v, gate.unsqueeze(-1), beta.unsqueeze(-1))]
                y, s = st(q, k, v.mT, gate, beta, s.mT)
                return y, s.mT
    elif op == 'mamba2':
        inputs = (randn(B, T, H, C), th.sigmoid(randn(B, T, H)), -th.rand(H, generator=g).to(device),
                  randn(B, T, 1, C), randn(B, T, 1, C), randn(B, H, C, C))
        st = jit('step', ops.mamba2)

        def layer(x, dt, A, b, c, s):
            x, dt, A, b, c = [i.unsqueeze(-2) for i in (x, dt.unsqueeze(-1), A[None, None, :, None], b, c)]
            return st(x.mT, dt, A, b, c, s)
    elif op == 'longhorn':
        inputs = (randn(B, H * C, T), randn(B, C, T), randn(B, C, T), randn(B, H * C, T))
        st = jit('step', ops.longhorn)

        def layer(u, q, k, dt):
            u, q, k, dt = [i.mT.view(B, T, -1, 1, C) for i in (u, q, k, dt)]
            s = th.zeros(B, H, C, C, device=u.device, dtype=u.dtype)
            return st(u.mT, q, k, dt.mT, s)[0].view(B, T, H * C).mT
    elif op == 'rwkv4':
        s = randn(B, 3, 1, D)
        s[:, 2] = -1e30
        inputs = (randn(D), randn(D), randn(B, T, D), randn(B, T, D), s)
        st = jit('step', ops.rwkv4)

        def layer(w, u, k, v, s):
            w, u, k, v = [i[:, :, None, :, None] for i in (w[None, None], u[None, None], k, v)]
            sa, sb, sc = s.unsqueeze(-1).unbind(1)
            y, sa, sb, sc = st(w, u, k, v, sa, sb, sc)
            return y.squeeze(2), th.stack((sa, sb, sc), dim=1).squeeze(-1)
    elif op == 'hgrn':
        inputs = (randn(B, T, D), -th.sigmoid(randn(B, T, D)))
        st = jit('step', ops.hgrn)

        def layer(x, gate):
            s = th.zeros(B, 1, D, 1, device=x.device, dtype=x.dtype)
            x, gate = [i[:, :, None, :, None] for i in (x, gate)]
            return st(x, gate, s)[0].squeeze(2)
    elif op == 'mamba':
        N = 16
        inputs = (randn(B, D, T), th.sigmoid(randn(B, D, T)), -th.sigmoid(randn(D, N)), randn(B, N, T), randn(B, N, T))
        st = jit('step', ops.mamba)

        def layer(u, dt, A, b, c):
            u, dt, b, c = [i.mT[:, :, None, :, None] for i in (u, dt, b, c)]
            s = th.zeros(B, 1, D, N, device=u.device, dtype=u.dtype)
            return st(u, dt, A[None, None, None], b.mT, c.mT, s)[0].squeeze(2).mT
    elif op == 's4d':
        N = C // 2
        inputs = (randn(B, T, D), 0.9 * th.cos(randn(D, N)), 0.4 * th.sin(randn(D, N)), randn(D, N), randn(D, N), randn(D))
        st = jit('step', ops.s4d)

        def layer(u, Ar, Ai, Qr, Qi, Dp):
            u = u[:, :, None, :, None]
            Ar, Ai, Qr, Qi = [i[None, None, None] for i in (Ar, Ai, Qr, Qi)]
            Sr, Si = [th.zeros(B, 1, D, N, device=u.device, dtype=u.dtype) for _ in range(2)]
            return st(u, Ar, Ai, Qr, Qi, Dp[None, None, None, :, None], Sr, Si)[0].squeeze(2)
    elif op == 'gsa':
        q, k, v, x, gate = [randn(B, T, H, C) for _ in range(5)]
        gate = -th.sigmoid(gate)
        inputs = (q, k, v, x, gate, randn(B, H, C, C), randn(B, H, C, C))
        s1, s2 = jit('step1', ops.gsa_slot), jit('step2', ops.gsa_value)

        def layer(q, k, v, x, gate, sa, sb):
            q, k, v, x, gate = [i.unsqueeze(-2) for i in (q, k, v, x, gate)]
            qv, sa = s1(q, k, x.mT, gate.mT, sa.mT)
            qv = qv.softmax(-1).unsqueeze(-2)
            y, sb = s2(qv, x, v.mT, gate, sb.mT)
            return y, sa.mT, sb.mT
    elif op == 'mlstm':
        inputs = (randn(B, H, T, C), randn(B, H, T, C), randn(B, H, T, C), randn(B, H, T), randn(B, H, T),
                  randn(B, H, C, C), randn(B, H, C), randn(B, H, 1))
        s1, s2, s3 = jit('step1', ops.mlstm_gates), jit('step2', ops.mlstm_norm), jit('step3', ops.mlstm_cell)

        def layer(q, k, v, i, f, sa, sb, sc):
            i, f, sb, sc = [x.unsqueeze(-1) for x in (i, f, sb, sc)]
            q, k, v, i, f = [x.transpose(1, 2).unsqueeze(-2) for x in (q, k, v, i, f)]
            i, f, sc, scT = s1(i, f, sc)
            i, f = i.unsqueeze(-1), f.unsqueeze(-1)
            sb_q, sbT = s2(k, q, i, f, sb.mT)
            norm = 1 / (th.maximum(th.abs(sb_q), (-sc).exp() * C ** .5) + 1e-6 * C ** .5).unsqueeze(-1)
            y, saT = s3(q, k, v.mT, i, f, norm, sa.mT)
            return y.transpose(1, 2), saT.mT, sbT.squeeze(-2), scT.squeeze(-1)
    else:
        raise KeyError(op)
    return inputs, layer, steps


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument('--batchsz', type=int, default=8)
    ap.add_argument('--modeldim', type=int, default=None)
    ap.add_argument('--headsz', type=int, default=128)
    ap.add_argument('--seqlen', type=int, default=None)
    ap.add_argument('--op', default='rwkv7', choices=OPS)
    ap.add_argument('--benchmark-flex', action='store_true')
    ap.add_argument('--check-flex', action='store_true')
    ap.add_argument('--torch-compile', action='store_true')
    ap.add_argument('--forward', action='store_true', help='forward pass only')
    ap.add_argument('--raw', action='store_true', help='the layer takes raw projections and prepares them itself (ops: ' + ', '.join(RAW_OPS) + ')')
    ap.add_argument('--fuse', action='store_true', help='run the layer through flex_rnn_amd.layer (input preparation moves into the step)')
    ap.add_argument('--fuse-reductions', action='store_true', help='with --fuse: also move sums and norms along the column axis')
    a = ap.parse_args(argv)
    check = a.check_flex or not a.benchmark_flex
    D = a.modeldim or (256 if check else 4096)
    T = a.seqlen or (256 if check else 1024)
    print(f'Testing {a.op}\nInput sizes B={a.batchsz}, T={T}, H={D // a.headsz}, C={a.headsz}')
    inputs, layer, steps = build(a.op, a.batchsz, T, D, a.headsz, 'cuda', raw=a.raw)
    eager_layer = layer
    if a.fuse:
        layer = flex_rnn_amd.layer(layer, reductions=a.fuse_reductions)
    if not check:
        if a.op not in ('s4d', 'mamba'):
            inputs = tuple(i.to(th.bfloat16) for i in inputs)
        fn = th.compile(layer) if a.torch_compile else layer
        print('Benchmarking flex compiled kernel')
        flex_rnn_amd.benchmark(fn, list(inputs), backward=not a.forward)
        return

    def ref(*args):
        saved = {k: s.apply for k, s in steps.items()}
        for s in steps.values():
            s.apply = s.naive_fp64
        try:
            return eager_layer(*args)
        finally:
            for k, s in steps.items():
                s.apply = saved[k]

    print('Verifying flex compiled kernel')
    fn = th.compile(layer) if a.torch_compile else layer
    flex_rnn_amd.check_grad(fn, ref, list(inputs), backward=not a.forward)


if __name__ == '__main__':
    main()
