"""Step functions and input layouts used across the tests (the 14 example recurrences the
reference ships in /root/reference/tests/examples.py, with their broadcast patterns)."""
import torch as th
import torch.nn.functional as F

from flex_rnn_amd import ops

# spec per input: (class, spans) with class in row/col/scalar/mat and spans a subset of 'BTH'
CASES = {
    'rwkv7': (ops.rwkv7, [('row', 'BTH'), ('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('row', 'BTH'), ('row', 'BTH')], 1),
    'rwkv7_decay': (ops.rwkv7_decay, [('row', 'BTH')] * 3 + [('col', 'BTH')] + [('row', 'BTH')] * 2, 1),
    'rwkv6': (ops.rwkv6, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('row', 'BTH'), ('row', 'H')], 1),
    'gla': (ops.gla, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('row', 'BTH')], 1),
    'retention': (ops.retention, [('scalar', 'BTH'), ('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH')], 1),
    'delta_rule': (ops.delta_rule, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('scalar', 'BTH')], 1),
    'delta_rule_fused': (ops.delta_rule_fused, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('scalar', 'BTH')], 1),
    'gated_delta_rule': (ops.gated_delta_rule, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('scalar', 'BTH'), ('scalar', 'BTH')], 1),
    'mamba2': (ops.mamba2, [('col', 'BTH'), ('scalar', 'BTH'), ('scalar', 'H'), ('row', 'BT'), ('row', 'BT')], 1),
    'mamba': (ops.mamba, [('col', 'BTH'), ('col', 'BTH'), ('mat', 'H'), ('row', 'BT'), ('row', 'BT')], 1),
    'longhorn': (ops.longhorn, [('col', 'BTH'), ('row', 'BT'), ('row', 'BT'), ('col', 'BTH')], 1),
    's4d': (ops.s4d, [('col', 'BT'), ('mat', ''), ('mat', ''), ('mat', ''), ('mat', ''), ('col', '')], 2),
    'gsa_slot': (ops.gsa_slot, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('col', 'BTH')], 1),
    'mlstm_norm': (ops.mlstm_norm, [('row', 'BTH'), ('row', 'BTH'), ('scalar', 'BTH'), ('scalar', 'BTH')], 1),
    'mlstm_cell': (ops.mlstm_cell, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('scalar', 'BTH'), ('scalar', 'BTH'), ('col', 'BTH')], 1),
}


def _zoo(x, g, c, S):
    """Exercises the emitter's op table: sigmoid, tanh, softplus, where, relu, abs, sqrt, rsqrt, log,
    reciprocal, maximum/minimum, comparisons, pow, division."""
    gate = th.sigmoid(g) * th.tanh(x) + F.softplus(x) * 0.1
    S = S * th.sigmoid(g) + c * th.where(x > 0, gate, 0.2 * gate) + F.relu(x) * 0.05
    S = S + th.minimum(th.maximum(c, -c), th.ones_like(c)) * th.sqrt(x.abs() + 1.0) / (1.0 + x ** 2)
    y = (S * th.rsqrt(1.0 + x * x)).sum(-1, True) + th.log(1.0 + c * c) - (1.0 / (2.0 + g.abs())).sum(-1, True)
    return y, S


CASES['zoo'] = (_zoo, [('row', 'BTH'), ('row', 'BT'), ('col', 'BTH')], 1)


def _zoo2(x, g, c, S):
    """More of the op table: clamp / hardtanh, leaky_relu, elu, gelu (both forms), silu, sin, cos, erf,
    log2, exp2, integer and fractional powers, logical and / or / not on comparisons."""
    gate = th.sigmoid(F.gelu(g) + F.gelu(x, approximate='tanh') * 0.5 + F.silu(g) * 0.1)
    upd = F.leaky_relu(x, 0.1) + F.elu(x) * 0.3 + x.clamp(-0.7, 0.9) + F.hardtanh(g, -0.5, 0.5) + g.clamp(min=-0.2) * 0.1
    upd = upd + th.sin(x) * th.cos(g) + th.erf(x) * 0.2 + th.log2(1.5 + x * x) * th.exp2(-g.abs())
    upd = upd + (x.abs() + 0.5) ** 1.5 * 0.1 + (0.5 * x) ** 4 + (1.0 + g * g) ** -2
    inside = (x > -0.3) & (x < 0.6)
    outside = (g > 1.0) | ~(g > -1.0)
    S = S * gate + c * th.where(inside, upd, 0.5 * upd) + th.where(outside, g, x) * 0.05 * F.relu6(c + 1.0)
    y = (S * th.tanh(x)).sum(-1, True) + F.hardsigmoid(c) * F.hardswish(c) * 0.1
    return y, S


CASES['zoo2'] = (_zoo2, [('row', 'BTH'), ('row', 'BT'), ('col', 'BTH')], 1)



def _matgain(q, k, v, w, G, S):
    """Gated linear attention with a per-element gain on the update: a matrix input whose gradient
    does not read the state (it is formed by the per-chunk gradient kernel, not by the reverse scan)."""
    S = S * th.sigmoid(w) + G * (v * k)
    return (S * q).sum(-1, True), S


CASES['matgain'] = (_matgain, [('row', 'BTH'), ('row', 'BTH'), ('col', 'BTH'), ('row', 'BTH'), ('mat', 'BH')], 1)
# Mamba-1 with a decay matrix per (batch, head): a matrix input that is broadcast over nothing
CASES['mamba_bh'] = (ops.mamba, [('col', 'BTH'), ('col', 'BTH'), ('mat', 'BH'), ('row', 'BT'), ('row', 'BT')], 1)

# vector-state recurrences (N == 1)
VECTOR_CASES = {
    'hgrn': (ops.hgrn, [('col', 'BT'), ('col', 'BT')], 1),
    'rwkv4': (ops.rwkv4, [('col', ''), ('col', ''), ('col', 'BT'), ('col', 'BT')], 3),
    'mlstm_gates': (ops.mlstm_gates, [('col', 'BTH'), ('col', 'BTH')], 1),
}


def make_inputs(name, B, T, H, M, N, dtype=th.float64, seed=0, table=None):
    step, spec, nst = (table or {**CASES, **VECTOR_CASES})[name]
    g = th.Generator().manual_seed(seed)
    xs = []
    for cls, spans in spec:
        shape = [B if 'B' in spans else 1, T if 'T' in spans else 1, H if 'H' in spans else 1,
                 M if cls in ('col', 'mat') else 1, N if cls in ('row', 'mat') else 1]
        xs.append((th.randn(*shape, generator=g) * 0.5).to(dtype))
    # keep the recurrences contractive so fp32 comparisons stay meaningful
    if name in ('rwkv7', 'rwkv6', 'gla', 'gated_delta_rule', 'gsa_slot', 'hgrn'):
        i = {'rwkv7': 1, 'rwkv6': 3, 'gla': 3, 'gated_delta_rule': 3, 'gsa_slot': 3, 'hgrn': 1}[name]
        xs[i] = -th.sigmoid(xs[i].double()).to(dtype)
    if name == 'rwkv7_decay':
        xs[1] = th.exp(-th.exp(xs[1].double())).to(dtype)
    if name in ('rwkv7', 'rwkv7_decay'):
        kk = F.normalize(xs[4].double(), dim=-1)
        xs[4], xs[5] = (-kk).to(dtype), (kk * th.sigmoid(xs[5].double())).to(dtype)
    if name in ('delta_rule', 'gated_delta_rule'):
        xs[1] = F.normalize(xs[1].double(), dim=-1).to(dtype)
        j = 3 if name == 'delta_rule' else 4
        xs[j] = th.sigmoid(xs[j].double()).to(dtype)
    if name == 'retention':
        xs[0] = th.sigmoid(xs[0].double() + 2).to(dtype)
    if name in ('mamba', 'mamba2', 'mamba_bh'):
        xs[1] = F.softplus(xs[1].double() - 1).to(dtype)
        xs[2] = -th.sigmoid(xs[2].double()).to(dtype)
    if name == 's4d':
        xs[1], xs[2] = (0.9 * th.cos(xs[1].double())).to(dtype), (0.4 * th.sin(xs[2].double())).to(dtype)
    if name in ('mlstm_norm', 'mlstm_cell'):
        j = 2 if name == 'mlstm_norm' else 3
        xs[j], xs[j + 1] = th.sigmoid(xs[j].double()).to(dtype), th.sigmoid(xs[j + 1].double() + 1).to(dtype)
    Heff = H if any('H' in spans for _, spans in spec) else 1      # states follow the widest input
    ss = [(th.randn(B, Heff, M, N, generator=g) * 0.3).to(dtype) for _ in range(nst)]
    return step, xs, ss


# ------------------------------------------------------------------ random recurrences
_UNARY_SRC = ['th.sigmoid({0})', 'th.tanh({0})', '({0}).exp().clamp(max=4.0)', 'F.softplus({0})', '({0} * {0})',
              '(1.0 / (1.0 + ({0}).abs()))', 'th.where({0} > 0, {0}, 0.3 * {0})', '(-{0})', '({0} * 0.5 + 0.1)']


def random_step(seed):
    """A random but well-behaved linear-attention-like recurrence: a contractive decay built from
    a random mix of row / column / scalar inputs, one or two rank-1 updates, optionally a
    delta-rule style read-back (S k) and an in-step normalisation, and a read-out with an
    optional per-row skip term.  Returns (step, spec, nstates, source)."""
    import random
    rnd = random.Random(seed)
    ninp = rnd.randint(3, 6)
    classes = ['row', 'col'] + [rnd.choice(['row', 'col', 'scalar', 'row']) for _ in range(ninp - 2)]
    rnd.shuffle(classes)
    spec = []
    for c in classes:
        spans = ''.join(d for d in 'BTH' if rnd.random() < 0.8)
        spec.append((c, spans))
    spec[0] = (spec[0][0], 'BTH')
    names = [f'x{i}' for i in range(ninp)]
    by = {c: [n for n, (cc, _) in zip(names, spec) if cc == c] for c in ('row', 'col', 'scalar')}

    def pick(cls_list):
        pool = [n for c in cls_list for n in by[c]]
        return rnd.choice(pool)

    def expr(cls_list, depth=2):
        e = pick(cls_list)
        for _ in range(rnd.randint(0, depth)):
            e = rnd.choice(_UNARY_SRC).format(e)
            if rnd.random() < 0.3:
                e = f'({e} * {pick(cls_list)})'
        return e

    lines = []
    if rnd.random() < 0.4:          # in-step normalisation of a row input
        r0 = by['row'][0]
        lines.append(f'{r0} = {r0} * th.rsqrt(({r0} * {r0}).sum(-1, True) + 1.0)')
    dec = [rnd.choice([['row'], ['col'], ['row', 'scalar'] if by['scalar'] else ['row'], ['col', 'row']])]
    lines.append(f'decay = th.sigmoid({expr(dec[0])})' + (f' * th.sigmoid({expr(["col"])})' if rnd.random() < 0.4 else ''))
    lines.append(f'k = {expr(["row", "scalar"] if by["scalar"] else ["row"])}')
    lines.append(f'v = {expr(["col", "scalar"] if by["scalar"] else ["col"])}')
    if rnd.random() < 0.5:          # delta-rule style correction
        lines.append('S = S * decay')
        lines.append(f'S = S + 0.5 * th.sigmoid({pick(["row", "col", "scalar"] if by["scalar"] else ["row", "col"])}) * k * (v - (S * k).sum(-1, True))')
    else:
        lines.append('S = S * decay + v * k')
        if rnd.random() < 0.5:
            lines.append(f'S = S + 0.1 * (S * th.tanh({expr(["row"])})).sum(-1, True) * th.tanh({expr(["row"])})')
    lines.append(f'y = (S * {expr(["row"])}).sum(-1, True)')
    if rnd.random() < 0.5:
        lines.append(f'y = y + {expr(["col"])}')
    src = 'def step(' + ', '.join(names) + ', S):\n' + ''.join(f'    {ln}\n' for ln in lines) + '    return y, S\n'
    env = {'th': th, 'F': F}
    exec(src, env)
    return env['step'], spec, 1, src


# Random recurrences that run both through the emitted kernels on the CPU harness and on the GPU:
# seed -> B, T, H, M, N (widths that are no power of two included)
FUZZ_DIMS = [(2, 8, 2, 8, 16), (1, 19, 2, 5, 32), (2, 16, 1, 24, 128), (2, 8, 2, 8, 24), (1, 19, 2, 5, 48), (2, 16, 1, 12, 5)]
FUZZ_SEEDS = range(100, 112)


def fuzz_case(seed, dtype):
    """(step, inputs, states) of random recurrence `seed` at its size in FUZZ_DIMS."""
    step, spec, nst, _ = random_step(seed)
    return make_inputs('gen', *FUZZ_DIMS[seed % 6], dtype=dtype, table={'gen': (step, spec, nst)})
