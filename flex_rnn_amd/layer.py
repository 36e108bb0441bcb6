"""Layer-level tracing: `flex_rnn_amd.layer(fn)`.

The reference's users call a compiled step through small adapters written against layer-shaped
tensors - `[B,T,H,C]` projections that are unsqueezed / transposed into the `[B,T,H,M|1,N|1]`
convention (/root/reference/README.md:17-23, every `flex()` in /root/reference/tests/examples.py,
e.g. 50-58, 165-174, 191-199, 298-307) - usually right after pointwise preparation of those
projections (a sigmoid gate, a softplus step size, an L2-normalised key, the negative exponential
of a decay parameter).  Run eagerly, every such operation reads and writes a whole `[B,T,H,C]`
tensor in the forward pass and again in the backward pass.

`layer(fn)` traces `fn` once per argument signature into an FX graph, finds the calls of `jit`
objects in it and, for every step input, follows the operations that produced it back towards the
layer's arguments.  Operations that act on one timestep of one head at a time - pointwise arithmetic,
dtype casts, and sums / means / L2 norms over the axis that becomes the state's column axis -
commute with slicing out a timestep, so they are moved *into* the step: a new step function
evaluates them on `[M|1, N|1]` tiles and then calls the user's step, and the `jit` object built from it
receives the raw tensors (as strided 5-D views, no copies).  The kernels then evaluate the preparation
while they stage a timestep's operands, the joint trace differentiates through it, and the gradients come
back with respect to the raw tensors.  View operations between preparation and step (unsqueeze, transpose,
expand, reshape that splits or merges whole axes) only relabel axes and disappear.  Whatever cannot be
moved (a softmax over time, a reduction over rows, an operation the step tracer does not know) stays in
the graph as it is and its result becomes a raw input of the fused step.

The result computes what `fn` computes; only the rounding differs where `fn` would have rounded
intermediate values to a 16-bit dtype (inside a step all arithmetic is fp32).
"""
from __future__ import annotations

import operator
import sys
from typing import Dict, List, Optional, Sequence, Tuple

import torch as th
import torch.fx as fx

AXES = 'BTHMN'


class Unfusable(Exception):
    """Raised during the analysis of one step input; `node` is the operation to leave in the graph."""

    def __init__(self, node, why=''):
        super().__init__(f'{node}: {why}')
        self.node = node


class _Atom:
    """One axis of the recurrence as it shows up in a dimension of some tensor.  `axis` is one of B, T, H, M, N, or
    None while unknown (the reduced axis of a sum, until another path to the same tensor names it); atoms
    found to be the same axis are linked (union-find)."""
    __slots__ = ('_axis', 'size', '_up')

    def __init__(self, axis, size):
        self._axis, self.size, self._up = axis, int(size), None

    def find(self):
        a = self
        while a._up is not None:
            a = a._up
        return a

    @property
    def axis(self):
        return self.find()._axis

    def unify(self, other) -> bool:
        a, b = self.find(), other.find()
        if a is b:
            return True
        if a.size != b.size or (a._axis and b._axis and a._axis != b._axis):
            return False
        if a._axis is None:
            a._up = b
        else:
            b._up = a
        return True

    def __repr__(self):
        return f'{self.axis or "?"}{self.size}'


def _unify(la, lb) -> bool:
    """Unifies two label lists (one tuple of atoms per dimension)."""
    if len(la) != len(lb):
        return False
    for ta, tb in zip(la, lb):
        if len(ta) != len(tb) or not all(x.unify(y) for x, y in zip(ta, tb)):
            return False
    return True


class _Leaf:
    def __init__(self, node, labels):
        self.node, self.labels = node, labels

    def signature(self):
        return tuple(tuple((a.axis, a.size) for a in t) for t in self.labels)


class _Op:
    """A pointwise operation: `target` applied to tiles (other arguments pass through)."""

    def __init__(self, node, args, kwargs):
        self.node, self.args, self.kwargs = node, args, kwargs


class _Reduce:
    def __init__(self, node, kind, child, atoms):
        self.node, self.kind, self.child, self.atoms = node, kind, child, atoms


_IDENTITY = {'_to_copy', 'clone', 'contiguous', 'alias', 'detach', 'lift_fresh_copy', 'to'}
_POINTWISE = {'sigmoid', 'exp', 'neg', 'mul', 'add', 'sub', 'div', 'reciprocal', 'log', 'sqrt', 'rsqrt', 'tanh', 'abs', 'relu',
              'sign', 'sgn', 'log1p', 'expm1', 'sin', 'cos', 'erf', 'log2', 'exp2', 'lt', 'gt', 'le', 'ge', 'eq', 'ne',
              'maximum', 'minimum', 'rsub', 'pow', 'where', 'clamp', 'clamp_min', 'clamp_max', 'hardtanh', 'leaky_relu',
              'elu', 'gelu', 'silu', 'softplus', 'logical_and', 'logical_or', 'logical_not', 'bitwise_and', 'bitwise_or',
              'bitwise_not', 'square', 'relu6', 'hardsigmoid', 'hardswish', 'mish'}
_REDUCE = {'sum': 'sum', 'mean': 'mean', 'linalg_vector_norm': 'norm'}


def _packet(node) -> str:
    t = node.target
    name = t.name() if hasattr(t, 'name') else getattr(t, '__name__', str(t))      # aten::mul.Tensor
    return name.split('::')[-1].split('.')[0]


def _shape(node):
    return tuple(int(s) for s in node.meta['val'].shape)


class _Analysis:
    """Follows the producers of the inputs of one `jit` call."""

    def __init__(self, cuts, reductions=False):
        self.cuts = cuts
        self.reductions = reductions
        self.ops: Dict[fx.Node, Tuple[object, list]] = {}      # operation nodes seen: node -> (expression, labels)
        self.leaves: List[_Leaf] = []

    def leaf(self, node, labels):
        for i, t in enumerate(labels):
            if not t and _shape(node)[i] != 1:
                raise Unfusable(node, 'a dimension longer than 1 that the step input does not have')
        lf = _Leaf(node, labels)
        self.leaves.append(lf)
        return lf

    def lift(self, node, labels):
        if not isinstance(node, fx.Node):
            raise Unfusable(node, 'not a tensor')
        if node.op != 'call_function' or node in self.cuts or not hasattr(node.target, 'name'):
            return self.leaf(node, labels)
        if node in self.ops:
            expr, seen = self.ops[node]
            if not _unify(seen, labels):
                raise Unfusable(node, 'used with two different axis assignments')
            return expr
        name = _packet(node)
        a = node.args
        shape = _shape(node)
        nd = len(shape)
        if name in _IDENTITY:
            return self.lift(a[0], labels)
        # ---- views: relabel and continue with the source
        if name == 'unsqueeze':
            d = a[1] % nd
            return self.lift(a[0], labels[:d] + labels[d + 1:])
        if name == 'squeeze':
            src = _shape(a[0])
            dims = range(len(src)) if len(a) == 1 else ([a[1]] if isinstance(a[1], int) else list(a[1]))
            dims = sorted(d % len(src) for d in dims if src[d % len(src)] == 1)
            out = list(labels)
            for d in dims:
                out.insert(d, ())
            return self.lift(a[0], out)
        if name in ('transpose', 't', 'mT', 'permute'):
            if name == 'permute':
                perm = [d % nd for d in a[1]]
            else:
                d0, d1 = (a[1] % nd, a[2] % nd) if name == 'transpose' else (nd - 2, nd - 1)
                perm = list(range(nd))
                perm[d0], perm[d1] = perm[d1], perm[d0]
            out = [None] * nd
            for i, p_ in enumerate(perm):       # output dim i is input dim perm[i]
                out[p_] = labels[i]
            return self.lift(a[0], out)
        if name == 'expand':
            src = _shape(a[0])
            off = nd - len(src)
            return self.lift(a[0], [labels[i + off] if src[i] == shape[i + off] else () for i in range(len(src))])
        if name == 'slice' and _shape(a[0]) == shape:
            return self.lift(a[0], labels)          # (a slice that keeps everything)
        if name in ('view', 'reshape', '_unsafe_view', 'unflatten', 'flatten'):
            return self.lift(a[0], self._regroup(node, _shape(a[0]), labels))
        # ---- arithmetic.  What does not vary with time stays in the graph: it is small there, and inside a step it
        # would be evaluated again at every timestep.
        if (name in _POINTWISE or name in _REDUCE) and not any(x.axis == 'T' for t in labels for x in t):
            return self.leaf(node, labels)
        if name in _POINTWISE:
            args = []
            for x in a:
                if isinstance(x, fx.Node):
                    xs = _shape(x)
                    off = nd - len(xs)
                    if off < 0:
                        raise Unfusable(node, 'operand with more dimensions than the result')
                    args.append(self.lift(x, [labels[i + off] if xs[i] == shape[i + off] else () for i in range(len(xs))]))
                elif isinstance(x, (int, float, bool)) or x is None:
                    args.append(x)
                else:
                    raise Unfusable(node, f'argument {x!r}')
            kwargs = {k: v for k, v in node.kwargs.items() if k not in ('dtype', 'layout', 'device', 'pin_memory', 'memory_format')}
            expr = _Op(node, args, kwargs)
            self.ops[node] = (expr, labels)
            return expr
        if name in _REDUCE and not self.reductions:
            return self.leaf(node, labels)
        if name in _REDUCE:
            src = _shape(a[0])
            if name == 'linalg_vector_norm':
                ord_ = a[1] if len(a) > 1 else node.kwargs.get('ord', 2)
                if ord_ not in (2, 2.0):
                    raise Unfusable(node, 'only the 2-norm')
                dims, keep = (a[2] if len(a) > 2 else node.kwargs.get('dim')), (a[3] if len(a) > 3 else node.kwargs.get('keepdim', False))
            else:
                if len(a) < 2:
                    raise Unfusable(node, 'reduction over everything')
                dims, keep = a[1], (a[2] if len(a) > 2 else node.kwargs.get('keepdim', False))
            if dims is None:
                raise Unfusable(node, 'reduction over everything')
            dims = sorted(d % len(src) for d in ([dims] if isinstance(dims, int) else dims))
            child, atoms = list(labels), []
            for d in dims:
                if src[d] == 1:
                    if not keep:
                        child.insert(d, ())
                    continue
                atom = _Atom(None, src[d])
                atoms.append(atom)
                if keep:
                    child[d] = (atom,)
                else:
                    child.insert(d, (atom,))
            expr = _Reduce(node, _REDUCE[name], self.lift(a[0], child), atoms)
            self.ops[node] = (expr, labels)
            return expr
        return self.leaf(node, labels)

    @staticmethod
    def _regroup(node, src, labels):
        """Labels of the source of a reshape: the atoms of the result, in order, dealt out to the source's dimensions."""
        atoms = [x for t in labels for x in t]
        out, k = [], 0
        for s in src:
            if s == 1:
                out.append(())
                continue
            take, prod = [], 1
            while prod < s:
                if k >= len(atoms):
                    raise Unfusable(node, 'reshape that does not keep whole axes')
                take.append(atoms[k])
                prod *= atoms[k].size
                k += 1
            if prod != s:
                raise Unfusable(node, 'reshape that splits an axis')
            out.append(tuple(take))
        if k != len(atoms):
            raise Unfusable(node, 'reshape that does not keep whole axes')
        return out

    def settle(self):
        """After all inputs of a call were followed: leaves reached several times name each other's unknown axes;
        every reduced axis must then be the state's column axis."""
        by_node: Dict[fx.Node, List[_Leaf]] = {}
        for lf in self.leaves:
            by_node.setdefault(lf.node, []).append(lf)
        for group in by_node.values():
            for lf in group:
                if any(x.axis is None for t in lf.labels for x in t):
                    for other in group:
                        if other is not lf and _structure_matches(lf.labels, other.labels):
                            _unify(lf.labels, other.labels)
                            break
        for node, (expr, _) in self.ops.items():
            if isinstance(expr, _Reduce):
                for atom in expr.atoms:
                    if atom.axis != 'N':
                        raise Unfusable(node, f'reduction over axis {atom.axis or "that never reaches the step"} (only sums along the '
                                              'state\'s column axis can move into a step)')
        for lf in self.leaves:
            axes = [x.axis for t in lf.labels for x in t]
            if None in axes or len(set(axes)) != len(axes):
                raise Unfusable(lf.node, 'an axis that is unknown or appears twice')


def _structure_matches(la, lb):
    return len(la) == len(lb) and all(len(ta) == len(tb) and all(x.size == y.size and (x.axis is None or y.axis is None or x.axis == y.axis)
                                                                   for x, y in zip(ta, tb)) for ta, tb in zip(la, lb))


def _to5d(v: th.Tensor, sig) -> th.Tensor:
    """The `[B|1, T|1, H|1, M|1, N|1]` view of a raw tensor whose dimensions carry the axes in `sig` (one tuple of
    (axis, size) pairs per dimension): merged dimensions are split, size-1 dimensions dropped, the rest ordered."""
    for d in range(len(sig) - 1, -1, -1):
        if len(sig[d]) > 1:
            v = v.unflatten(d, [s for _, s in sig[d]])
    flat = [ax for t in sig for ax, _ in (t if t else ((None, 1),))]
    drop = [i for i, ax in enumerate(flat) if ax is None]
    for i in reversed(drop):
        v = v.squeeze(i)
    have = [ax for ax in flat if ax is not None]
    v = v.permute([have.index(ax) for ax in AXES if ax in have])
    for i, ax in enumerate(AXES):
        if ax not in have:
            v = v.unsqueeze(i)
    return v


def _tile_eval(expr, tiles: Dict[int, th.Tensor], memo: dict):
    """Value of `expr` on one timestep of one head: tensors of shape `[M|1, N|1]`."""
    if not isinstance(expr, (_Leaf, _Op, _Reduce)):
        return expr
    key = id(expr)
    if key in memo:
        return memo[key]
    if isinstance(expr, _Leaf):
        r = tiles[id(expr)]
    elif isinstance(expr, _Op):
        args = [_tile_eval(x, tiles, memo) for x in expr.args]
        r = expr.node.target(*args, **expr.kwargs)
    else:
        x = _tile_eval(expr.child, tiles, memo)
        n = 1
        for atom in expr.atoms:
            n *= atom.size
        if not expr.atoms:
            r = x if expr.kind != 'norm' else x.abs()
        else:
            if x.shape[-1] == 1:        # constant along the reduced axis: the eager operation still adds up `n` copies
                x = x.expand(*x.shape[:-1], n)
            if expr.kind == 'norm':
                r = (x * x).sum(-1, True).sqrt()
            else:
                r = x.sum(-1, True)
                if expr.kind == 'mean':
                    r = r / n
    memo[key] = r
    return r


class FusedCall:
    """What became of one call of a `jit` object inside a traced layer."""

    def __init__(self, original, fused, raw_signatures, moved, metas):
        self.original = original            # the user's jit object
        self.fused = fused                  # the jit object that runs instead (takes the raw tensors)
        self.raw_signatures = raw_signatures
        self.moved = moved                  # names of the operations that moved into the step
        self.metas = metas                  # (inputs, states) of the fused step as meta tensors: what its kernels are planned for


class layer:
    """`layer(fn)`: a callable that computes what `fn` computes, with the per-timestep preparation of the inputs of
    every `jit` call inside `fn` moved into the compiled step.  `fn` takes and returns tensors (or tuples of
    tensors); it is traced once per signature of its tensor arguments (shape, strides, dtype, device).

    `reductions=True` also moves sums, means and L2 norms along the state's column axis (an L2-normalised key is
    then normalised inside the kernels).  By default they stay in the graph and only the arithmetic around them
    moves: a sum inside a step costs every kernel a reduction across lanes per timestep, in the gradient kernel also
    for its derivative, and measures slower than the eager reduction (gated delta rule layer with two normalised
    projections, B8 T1024 H32 128x128 on an MI355X: 3.5 ms eager, 4.5 ms with the norms moved)."""

    def __init__(self, fn, reductions=False):
        self.fn = fn
        self.reductions = bool(reductions)
        self._built = {}
        self.calls: List[FusedCall] = []        # of the most recently traced signature

    @staticmethod
    def _key(args):
        return tuple((tuple(a.shape), tuple(a.stride()), a.dtype, str(a.device)) if isinstance(a, th.Tensor) else ('const', a)
                     for a in args)

    def __call__(self, *args):
        key = self._key(args)
        hit = self._built.get(key)
        if hit is None:
            hit = self._built[key] = self._build(args)
        gm, calls = hit
        self.calls = calls
        return gm(*[a for a in args if isinstance(a, th.Tensor)])

    def graph(self, *args) -> fx.GraphModule:
        """The rewritten graph for these arguments (for inspection)."""
        key = self._key(args)
        if key not in self._built:
            self._built[key] = self._build(args)
        self.calls = self._built[key][1]
        return self._built[key][0]

    # ------------------------------------------------------------------ tracing and rewriting
    def _build(self, args):
        from torch.fx.experimental.proxy_tensor import make_fx
        from .jit import jit as jit_cls

        tensors = [a for a in args if isinstance(a, th.Tensor)]

        def flat(*ts):
            it = iter(ts)
            return self.fn(*[next(it) if isinstance(a, th.Tensor) else a for a in args])

        with th.no_grad():
            # (tensors the function closes over - a fixed decay table, say - enter the graph as constants)
            gm = make_fx(flat, tracing_mode='fake', _allow_non_fake_inputs=True)(*[t.detach() for t in tensors])
        calls = []
        for node in list(gm.graph.nodes):
            if node.op != 'call_function' or not hasattr(node.target, 'name'):
                continue
            obj = jit_cls.instance_of(node.target.name())
            if obj is None:
                continue
            done = self._fuse_call(gm, node, obj) if not obj.is_dynamic else None
            if done is not None:
                calls.append(done)
            else:
                self._reroute(gm, node, obj, obj, node.args)
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
        return gm, calls

    def _fuse_call(self, gm, node, obj) -> Optional[FusedCall]:
        from .jit import jit as jit_cls

        nin, nst = obj.ninputs, obj.nstates
        ins, states = list(node.args[:nin]), list(node.args[nin:])
        cuts = set()
        for _ in range(200):
            an = _Analysis(cuts, self.reductions)
            try:
                exprs = []
                for x in ins:
                    shape = _shape(x)
                    assert len(shape) == 5, f'a step input of shape {list(shape)}'
                    exprs.append(an.lift(x, [(_Atom(ax, s),) if s != 1 else () for ax, s in zip(AXES, shape)]))
                an.settle()
                break
            except Unfusable as e:
                if not isinstance(e.node, fx.Node) or e.node in cuts:
                    return None
                cuts.add(e.node)
        else:
            return None
        if not an.ops:
            return None                     # nothing but views between the layer's tensors and this call
        # distinct raw inputs: (graph node, axes of its dimensions)
        raw, slot_of = [], {}
        for lf in an.leaves:
            k = (lf.node, lf.signature())
            if k not in slot_of:
                slot_of[k] = len(raw)
                raw.append(k)
        leaf_slot = {id(lf): slot_of[(lf.node, lf.signature())] for lf in an.leaves}
        step, nraw = obj.step, len(raw)

        def fused_step(*a):
            tiles = {lid: a[s] for lid, s in leaf_slot.items()}
            memo = {}
            vals = [_tile_eval(e, tiles, memo) for e in exprs]
            return step(*vals, *a[nraw:])

        fused_step.__name__ = getattr(step, '__name__', 'step') + '_with_preparation'
        fused = jit_cls(fused_step, nraw + nst)
        # plan it now on shapes alone: what the step tracer or the planner refuses is not moved at all
        def meta_of(v):
            return th.empty_strided(v.shape, v.stride(), dtype=v.dtype, device='meta')

        metas = [meta_of(_to5d(k[0].meta['val'], k[1])) for k in raw], [meta_of(s_.meta['val']) for s_ in states]
        try:
            with th.no_grad():
                sys.modules[jit_cls.__module__].build_twopass(fused_step, *metas, dryrun=True)
        except (AssertionError, NotImplementedError, RuntimeError):
            return None

        with gm.graph.inserting_before(node):
            views = [gm.graph.call_function(_to5d, (k[0], k[1])) for k in raw]
        self._reroute(gm, node, obj, fused, (*views, *states))
        return FusedCall(obj, fused, [k[1] for k in raw], sorted({_packet(n) for n in an.ops}), metas)

    @staticmethod
    def _reroute(gm, node, obj, target, args):
        """Replaces the operator call `node` (a call of `obj`'s forward operator recorded by the tracer) with a call of
        `target.apply`: `apply` stays reassignable, as on every jit object (a layer can be run on the plain loop by
        setting it to `naive`)."""
        nvis = obj.noutputs + obj.nstates

        def run(*a):
            return tuple(target.apply(*a))

        run.__name__ = 'call_' + getattr(target.step, '__name__', 'step')
        for user in list(node.users):
            assert user.op == 'call_function' and user.target is operator.getitem, 'the result of a step call is used as a whole'
            if user.args[1] >= nvis:        # (the tracer names every result of the operator; the hidden ones have no readers)
                assert not user.users, 'a hidden result of a step call is used by the layer'
                gm.graph.erase_node(user)
        with gm.graph.inserting_before(node):
            new = gm.graph.call_function(run, tuple(args))
        node.replace_all_uses_with(new)
        gm.graph.erase_node(node)
