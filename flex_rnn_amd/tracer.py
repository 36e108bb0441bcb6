"""Trace one timestep and its vector-Jacobian product into the Graph IR.

What is traced is the same joint function the reference traces
(/root/reference/flex_rnn/trace_isolated.py:31-39):

    fwbw(*inputs_t, *state, *d_outputs, *d_new_state)
        -> (*outputs, *new_state, *d_inputs_t, *d_state)

on meta tensors of shape [m, n] for a single (batch, head).  The reference
captures it with AOT-autograd and re-parses the printed code; here the FX graph
produced by `make_fx` (functionalized, core-ATen decomposed) is walked node by
node and every dtype cast is dropped, so all arithmetic is fp32 whatever the
I/O dtypes are (/root/reference/flex_rnn/graph.py:34-36 does the same by
aliasing `_to_copy`).
"""
from __future__ import annotations

from typing import Callable, Dict, List, Sequence, Tuple

import torch

from .ir import Graph, Node, broadcast_ext


class UnsupportedOp(NotImplementedError):
    pass


def _as_tuple(x):
    return tuple(x) if isinstance(x, (tuple, list)) else (x,)


def flat_step(step: Callable) -> Callable:
    def flat(*a):
        y, s = step(*a)
        return (*_as_tuple(y), *_as_tuple(s))
    return flat


def _needs_isolation() -> bool:
    """True when the calling thread is inside another tracer (fake-tensor mode, proxy
    tracing, functorch transform or a dispatcher callback with keys masked out)."""
    if torch._guards.detect_fake_mode() is not None:
        return True
    if torch.utils._python_dispatch._get_current_dispatch_mode_stack():
        return True
    excl = str(torch._C._dispatch_tls_local_exclude_set())
    return 'Functionalize' in excl or 'FuncTorchDynamicLayer' in excl


def _run_isolated(fn):
    """Dispatch-mode stacks, functorch layers and the dispatcher's include/exclude key sets are
    all thread-local, so a nested trace started from inside another tracer (torch.compile
    calling the op's fake implementation) runs on a fresh thread with default state.  The
    reference pickles the graph through a subprocess for the same purpose
    (/root/reference/flex_rnn/trace_isolated.py:3-14)."""
    import concurrent.futures
    with concurrent.futures.ThreadPoolExecutor(max_workers=1) as pool:
        return pool.submit(fn).result()


def trace_joint_fx(step: Callable, metas: Sequence[torch.Tensor]) -> Tuple[torch.fx.GraphModule, int]:
    """`metas`: tensors [m,n] (only shape and dtype are used) for inputs then states.  Returns
    the FX graph of the joint function and the number of forward results (outputs + states)."""
    import torch._decomp
    from torch.fx.experimental.proxy_tensor import make_fx

    flat = flat_step(step)
    nargs = len(metas)
    sig = [(tuple(m.shape), m.dtype) for m in metas]

    def run():
        args = tuple(torch.empty(s, dtype=d, device='meta') for s, d in sig)
        outs = flat(*args)

        def fwbw(*a):
            x, dy = a[:nargs], a[nargs:]
            y, pull = torch.func.vjp(flat, *x)
            return (*y, *pull(tuple(dy)))

        cot = tuple(torch.empty(o.shape, dtype=o.dtype, device='meta') for o in outs)
        gm = make_fx(torch.func.functionalize(fwbw),
                     decomposition_table=torch._decomp.core_aten_decompositions(),
                     tracing_mode='real')(*args, *cot)
        return gm, len(outs)

    return _run_isolated(run) if _needs_isolation() else run()


# --------------------------------------------------------------------------- FX -> IR

_ALIAS = {'aten::_to_copy', 'aten::clone', 'aten::expand', 'aten::alias', 'aten::detach', 'aten::view',
          'aten::reshape', 'aten::_unsafe_view', 'aten::contiguous', 'aten::lift_fresh_copy',
          'prims::convert_element_type', 'aten::to.dtype', 'aten::to.dtype_layout'}
_UNARY = {'aten::exp': 'exp', 'aten::neg': 'neg', 'aten::reciprocal': 'reciprocal', 'aten::log': 'log',
          'aten::sqrt': 'sqrt', 'aten::rsqrt': 'rsqrt', 'aten::sigmoid': 'sigmoid', 'aten::tanh': 'tanh',
          'aten::abs': 'abs', 'aten::relu': 'relu', 'aten::sign': 'sign', 'aten::sgn': 'sign',
          'aten::log1p': 'log1p', 'aten::expm1': 'expm1', 'aten::sin': 'sin', 'aten::cos': 'cos',
          'aten::erf': 'erf', 'aten::log2': 'log2', 'aten::exp2': 'exp2'}
_BINARY = {'aten::mul': 'mul', 'aten::add': 'add', 'aten::sub': 'sub', 'aten::div': 'div', 'aten::lt': 'lt',
           'aten::gt': 'gt', 'aten::le': 'le', 'aten::ge': 'ge', 'aten::eq': 'eq', 'aten::ne': 'ne',
           'aten::maximum': 'maximum', 'aten::minimum': 'minimum'}
_CONST_LIKE = {'aten::ones_like': 1.0, 'aten::zeros_like': 0.0}


class _Builder:
    """Builds the IR with value numbering (identical sub-expressions share a node)."""

    def __init__(self, name: str):
        self.name = name
        self.inputs: List[str] = []
        self.input_ext: Dict[str, Tuple[bool, bool]] = {}
        self.nodes: List[Node] = []
        self.ext: Dict[str, Tuple[bool, bool]] = {}
        self.memo: Dict[tuple, str] = {}
        self.counter = 0

    def add_input(self, name: str, ext):
        self.inputs.append(name)
        self.input_ext[name] = ext
        self.ext[name] = ext

    def emit(self, op: str, args: tuple, ext=None, dims: tuple = (), hint: str = 'v') -> str:
        key = (op, args, dims)
        if key in self.memo:
            return self.memo[key]
        if ext is None:
            ext = broadcast_ext(self.ext[a] for a in args if isinstance(a, str))
        name = f'{hint}{self.counter}'
        self.counter += 1
        self.nodes.append(Node(name, op, args, ext, dims))
        self.ext[name] = ext
        self.memo[key] = name
        return name

    def const(self, value: float) -> str:
        return self.emit('const', (float(value),), ext=(False, False), hint='c')


def _ext_of(val) -> Tuple[bool, bool]:
    shape = tuple(val.shape)
    if len(shape) != 2:
        raise UnsupportedOp(f'every value in the step must stay 2-D (use keepdim=True); got shape {list(shape)}')
    return (shape[0] != 1, shape[1] != 1)


def fx_to_graph(gm: torch.fx.GraphModule, name: str = 'joint') -> Graph:
    b = _Builder(name)
    env: Dict[str, object] = {}          # fx node name -> IR value name or python number

    def val(a):
        if isinstance(a, torch.fx.Node):
            return env[a.name]
        if isinstance(a, (int, float, bool)):
            return float(a)
        raise UnsupportedOp(f'unsupported argument {a!r}')

    def lift(a):
        """IR value name for `a` (numbers become const nodes)."""
        v = val(a)
        return v if isinstance(v, str) else b.const(v)

    outputs: List[str] = []
    for node in gm.graph.nodes:
        if node.op == 'placeholder':
            b.add_input(node.name, _ext_of(node.meta['val']))
            env[node.name] = node.name
            continue
        if node.op == 'output':
            for o in node.args[0]:
                outputs.append(lift(o))
            continue
        if node.op != 'call_function':
            raise UnsupportedOp(f'unsupported FX node {node.op} {node.target}')
        tgt = node.target
        full = tgt.name() if hasattr(tgt, 'name') else str(tgt)      # e.g. aten::mul.Tensor
        base = full.split('.')[0]
        a = node.args
        kw = node.kwargs

        if base in _ALIAS or full in _ALIAS:
            src = a[0]
            if base in ('aten::view', 'aten::reshape', 'aten::_unsafe_view'):
                if tuple(node.meta['val'].shape) != tuple(src.meta['val'].shape):
                    raise UnsupportedOp(f'{full}: reshaping {list(src.meta["val"].shape)} -> '
                                        f'{list(node.meta["val"].shape)} is not supported')
            env[node.name] = val(src)
        elif base in _UNARY:
            env[node.name] = b.emit(_UNARY[base], (lift(a[0]),), hint=_UNARY[base])
        elif base in _BINARY:
            x, y = val(a[0]), val(a[1])
            alpha = kw.get('alpha', a[2] if len(a) > 2 else 1)
            if base in ('aten::add', 'aten::sub') and alpha != 1:
                y = b.emit('mul', (y if isinstance(y, str) else b.const(y), float(alpha)), hint='mul')
            if base == 'aten::div' and kw.get('rounding_mode') is not None:
                raise UnsupportedOp('div with rounding_mode is not supported')
            if not isinstance(x, str) and not isinstance(y, str):
                x = b.const(x)
            if not isinstance(x, str):          # keep the tensor operand first where it commutes
                if _BINARY[base] in ('mul', 'add', 'maximum', 'minimum', 'eq', 'ne'):
                    x, y = y, x
                else:
                    x = b.const(x)
            env[node.name] = b.emit(_BINARY[base], (x, y), hint=_BINARY[base])
        elif base == 'aten::rsub':
            x, y = lift(a[0]), val(a[1])
            env[node.name] = b.emit('sub', (y if isinstance(y, str) else b.const(y), x), hint='sub')
        elif base == 'aten::pow':
            if full != 'aten::pow.Tensor_Scalar':
                raise UnsupportedOp(f'{full} is not supported (only tensor ** python number)')
            x, p = lift(a[0]), float(a[1])
            if p == 1.0:
                env[node.name] = x
            elif p == 2.0:
                env[node.name] = b.emit('mul', (x, x), hint='mul')
            elif p == 3.0:
                env[node.name] = b.emit('mul', (b.emit('mul', (x, x), hint='mul'), x), hint='mul')
            elif p == 0.5:
                env[node.name] = b.emit('sqrt', (x,), hint='sqrt')
            elif p == -1.0:
                env[node.name] = b.emit('reciprocal', (x,), hint='reciprocal')
            elif p == -0.5:
                env[node.name] = b.emit('rsqrt', (x,), hint='rsqrt')
            elif p == 0.0:
                env[node.name] = b.const(1.0)
            elif p == int(p) and abs(p) <= 8:
                r = x
                for _ in range(int(abs(p)) - 1):
                    r = b.emit('mul', (r, x), hint='mul')
                env[node.name] = r if p > 0 else b.emit('reciprocal', (r,), hint='reciprocal')
            else:       # positive bases only, like torch for a fractional exponent
                env[node.name] = b.emit('exp', (b.emit('mul', (b.emit('log', (x,), hint='log'), p), hint='mul'),), hint='exp')
        elif base == 'aten::where':
            env[node.name] = b.emit('where', (lift(a[0]), lift(a[1]), lift(a[2])), hint='where')
        elif base in _CONST_LIKE:
            env[node.name] = _CONST_LIKE[base]
        elif base in ('aten::full_like', 'aten::full', 'aten::scalar_tensor', 'aten::new_full'):
            v = a[1] if base in ('aten::full_like', 'aten::full') else (a[2] if base == 'aten::new_full' else a[0])
            env[node.name] = float(v)
        elif base in ('aten::zeros', 'aten::new_zeros'):
            env[node.name] = 0.0
        elif base in ('aten::ones', 'aten::new_ones'):
            env[node.name] = 1.0
        elif base in ('aten::empty_like', 'aten::empty', 'aten::empty_permuted', 'aten::empty_strided',
                      'aten::new_empty', 'aten::new_empty_strided'):
            env[node.name] = 0.0        # only ever consumed by *_like fills
        elif base == 'aten::sum':
            if full != 'aten::sum.dim_IntList':
                raise UnsupportedOp('Only torch.sum(x, dim=..., keepdim=True) is supported')
            keepdim = a[2] if len(a) > 2 else kw.get('keepdim', False)
            if not keepdim:
                raise UnsupportedOp('Only torch.sum(x, dim=-1, keepdim=True) is supported')
            x = lift(a[0])
            em, en = b.ext[x]
            shape = tuple(a[0].meta['val'].shape) if isinstance(a[0], torch.fx.Node) else (1, 1)
            dims = sorted({d % 2 for d in (a[1] if isinstance(a[1], (list, tuple)) else [a[1]])})
            # summing an axis the value does not vary along multiplies by that axis' length
            dims_eff = tuple(d for d in dims if (em, en)[d])
            scale = 1
            for d in dims:
                if not (em, en)[d]:
                    scale *= int(shape[d]) if len(shape) == 2 else 1
            if dims_eff:
                ext = (em and 0 not in dims_eff, en and 1 not in dims_eff)
                r = b.emit('sum', (x,), ext=ext, dims=dims_eff, hint='sum')
            else:
                r = x
            if scale != 1:
                r = b.emit('mul', (r, float(scale)), hint='mul')
            env[node.name] = r
        elif base in ('aten::clamp', 'aten::hardtanh', 'aten::clamp_min', 'aten::clamp_max'):
            r = lift(a[0])
            if base == 'aten::hardtanh':
                lo, hi = (a[1] if len(a) > 1 else kw.get('min_val', -1.0)), (a[2] if len(a) > 2 else kw.get('max_val', 1.0))
            elif base == 'aten::clamp_min':
                lo, hi = a[1], None
            elif base == 'aten::clamp_max':
                lo, hi = None, a[1]
            else:
                lo, hi = (a[1] if len(a) > 1 else kw.get('min')), (a[2] if len(a) > 2 else kw.get('max'))
            if lo is not None:
                r = b.emit('maximum', (r, val(lo)), hint='maximum')
            if hi is not None:
                r = b.emit('minimum', (r, val(hi)), hint='minimum')
            env[node.name] = r
        elif base == 'aten::hardtanh_backward':
            g, x = lift(a[0]), lift(a[1])
            inside = b.emit('mul', (b.emit('gt', (x, float(a[2])), hint='gt'), b.emit('lt', (x, float(a[3])), hint='lt')), hint='mul')
            env[node.name] = b.emit('mul', (g, inside), hint='mul')
        elif base in ('aten::logical_and', 'aten::bitwise_and', 'aten::logical_or', 'aten::bitwise_or'):
            # truth values are 0.0 / 1.0 floats here
            x, y = (b.emit('ne', (lift(v), 0.0), hint='ne') for v in a[:2])
            env[node.name] = b.emit('mul' if base.endswith('and') else 'maximum', (x, y), hint='and' if base.endswith('and') else 'or')
        elif base in ('aten::logical_not', 'aten::bitwise_not'):
            env[node.name] = b.emit('eq', (lift(a[0]), 0.0), hint='not')
        elif base == 'aten::leaky_relu':
            x, slope = lift(a[0]), float(a[1] if len(a) > 1 else kw.get('negative_slope', 0.01))
            env[node.name] = b.emit('where', (b.emit('gt', (x, 0.0), hint='gt'), x, b.emit('mul', (x, slope), hint='mul')), hint='where')
        elif base == 'aten::leaky_relu_backward':
            g, x, slope = lift(a[0]), lift(a[1]), float(a[2])
            env[node.name] = b.emit('where', (b.emit('gt', (x, 0.0), hint='gt'), g, b.emit('mul', (g, slope), hint='mul')), hint='where')
        elif base == 'aten::elu':
            x = lift(a[0])
            alpha, scale, iscale = (float(a[i]) if len(a) > i else 1.0 for i in (1, 2, 3))
            neg = b.emit('mul', (b.emit('expm1', (b.emit('mul', (x, iscale), hint='mul'),), hint='expm1'), alpha * scale), hint='mul')
            env[node.name] = b.emit('where', (b.emit('gt', (x, 0.0), hint='gt'), b.emit('mul', (x, scale), hint='mul'), neg), hint='where')
        elif base == 'aten::elu_backward':
            g, alpha, scale, iscale, is_result, x = lift(a[0]), float(a[1]), float(a[2]), float(a[3]), bool(a[4]), lift(a[5])
            if is_result:
                neg = b.emit('mul', (g, b.emit('mul', (b.emit('add', (x, alpha * scale), hint='add'), iscale), hint='mul')), hint='mul')
            else:
                e = b.emit('exp', (b.emit('mul', (x, iscale), hint='mul'),), hint='exp')
                neg = b.emit('mul', (g, b.emit('mul', (e, alpha * scale * iscale), hint='mul')), hint='mul')
            env[node.name] = b.emit('where', (b.emit('gt', (x, 0.0), hint='gt'), b.emit('mul', (g, scale), hint='mul'), neg), hint='where')
        elif base in ('aten::gelu', 'aten::gelu_backward'):
            bw = base.endswith('backward')
            g = lift(a[0]) if bw else None
            x = lift(a[1] if bw else a[0])
            approx = kw.get('approximate', a[2 if bw else 1] if len(a) > (2 if bw else 1) else 'none')
            mul = lambda u, v: b.emit('mul', (u, v), hint='mul')
            add = lambda u, v: b.emit('add', (u, v), hint='add')
            if approx == 'tanh':
                k, c = 0.7978845608028654, 0.044715
                x2 = mul(x, x)
                t = b.emit('tanh', (mul(mul(x, add(mul(x2, c), 1.0)), k),), hint='tanh')
                cdf = mul(add(t, 1.0), 0.5)
                if not bw:
                    env[node.name] = mul(x, cdf)
                else:
                    dt = mul(b.emit('sub', (b.const(1.0), mul(t, t)), hint='sub'), mul(add(mul(x2, 3.0 * c), 1.0), k))
                    env[node.name] = mul(g, add(cdf, mul(mul(x, 0.5), dt)))
            else:
                cdf = mul(add(b.emit('erf', (mul(x, 0.7071067811865476),), hint='erf'), 1.0), 0.5)
                if not bw:
                    env[node.name] = mul(x, cdf)
                else:
                    pdf = mul(b.emit('exp', (mul(mul(x, x), -0.5),), hint='exp'), 0.3989422804014327)
                    env[node.name] = mul(g, add(cdf, mul(x, pdf)))
        elif base == 'aten::sigmoid_backward':
            g, out = lift(a[0]), lift(a[1])
            t = b.emit('sub', (b.const(1.0), out), hint='sub')
            env[node.name] = b.emit('mul', (g, b.emit('mul', (out, t), hint='mul')), hint='mul')
        elif base == 'aten::tanh_backward':
            g, out = lift(a[0]), lift(a[1])
            t = b.emit('sub', (b.const(1.0), b.emit('mul', (out, out), hint='mul')), hint='sub')
            env[node.name] = b.emit('mul', (g, t), hint='mul')
        elif base == 'aten::threshold_backward':
            g, x, thr = lift(a[0]), lift(a[1]), float(a[2])
            env[node.name] = b.emit('mul', (g, b.emit('gt', (x, thr), hint='gt')), hint='mul')
        else:
            raise UnsupportedOp(f'flex_rnn: operation {full} is not supported in a step function')

    # outputs that are bare numbers were lifted; outputs may alias inputs or each other (fine).
    return Graph(name, b.inputs, b.input_ext, b.nodes, outputs)


def trace_step(step: Callable, metas: Sequence[torch.Tensor]) -> Tuple[Graph, int]:
    gm, nfw = trace_joint_fx(step, metas)
    return fx_to_graph(gm), nfw
