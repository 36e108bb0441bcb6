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
    if name in ('mamba', 'mamba2'):
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
