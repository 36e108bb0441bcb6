"""Graph IR for one recurrence timestep.

A `Graph` is an ordered SSA list of `Node`s over 2-D values.  Every value has an
*extent* `(em, en)`: whether it varies along the state's row axis (M) and along
the state's column axis (N).  The four extents are the four operand classes of
the programming model:

    (True,  True )  full   [M,N]   state-like tile
    (True,  False)  col    [M,1]   one value per state row
    (False, True )  row    [1,N]   one value per state column
    (False, False)  scalar [1,1]

Supported node kinds: elementwise unary/binary/ternary ops (with broadcasting),
constants, and `sum` over a subset of the two axes with keepdim.

The role of this file matches the reference's text-parsed IR
(/root/reference/flex_rnn/graph.py:7-88: SSA list, alias erasure, pruning with
an input mask, shape inference) but it is built from FX nodes and their meta
tensors instead of from printed code, and carries true broadcast extents.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Sequence, Tuple, Union

Arg = Union[str, float, int, bool]

# op name -> arity.  Semantics are fp32; comparisons yield 0.0 / 1.0.
UNARY_OPS = ('exp', 'neg', 'reciprocal', 'log', 'sqrt', 'rsqrt', 'sigmoid', 'tanh', 'abs',
             'relu', 'sign', 'log1p', 'expm1', 'copy', 'sin', 'cos', 'erf', 'log2', 'exp2')
BINARY_OPS = ('mul', 'add', 'sub', 'div', 'lt', 'gt', 'le', 'ge', 'eq', 'ne', 'maximum', 'minimum')
TERNARY_OPS = ('where',)
ALL_OPS = UNARY_OPS + BINARY_OPS + TERNARY_OPS + ('sum', 'const')


@dataclass
class Node:
    name: str
    op: str
    args: Tuple[Arg, ...]            # value names (str) or python numbers
    ext: Tuple[bool, bool]           # (varies along M, varies along N)
    dims: Tuple[int, ...] = ()       # for 'sum': axes reduced, subset of (0, 1)

    def value_args(self) -> List[str]:
        return [a for a in self.args if isinstance(a, str)]


@dataclass
class Graph:
    name: str
    inputs: List[str]
    input_ext: Dict[str, Tuple[bool, bool]]
    nodes: List[Node]
    outputs: List[str]

    # ----------------------------------------------------------------- queries
    def ext(self, v: str) -> Tuple[bool, bool]:
        if v in self.input_ext:
            return self.input_ext[v]
        return self.node_map()[v].ext

    def node_map(self) -> Dict[str, Node]:
        return {n.name: n for n in self.nodes}

    def ext_table(self) -> Dict[str, Tuple[bool, bool]]:
        t = dict(self.input_ext)
        for n in self.nodes:
            t[n.name] = n.ext
        return t

    def sums(self) -> List[Node]:
        return [n for n in self.nodes if n.op == 'sum']

    # ------------------------------------------------------------- transforms
    def extract(self, name: str, outputs: Sequence[str], cut: Iterable[str] = ()) -> 'Graph':
        """Sub-graph computing `outputs`, treating every value named in `cut`
        as a fresh input (appended after the original inputs, in node order).
        Unused original inputs are kept in the signature; `used_inputs` of the
        result tells which are live."""
        cut = set(cut)
        nm = self.node_map()
        need = set()
        stack = [o for o in outputs]
        while stack:
            v = stack.pop()
            if v in need:
                continue
            need.add(v)
            if v in cut or v in self.input_ext:
                continue
            stack.extend(nm[v].value_args())
        nodes = [n for n in self.nodes if n.name in need and n.name not in cut]
        cut_inputs = [n.name for n in self.nodes if n.name in cut and n.name in need]
        inputs = list(self.inputs) + cut_inputs
        input_ext = dict(self.input_ext)
        for c in cut_inputs:
            input_ext[c] = nm[c].ext
        g = Graph(name, inputs, input_ext, nodes, list(outputs))
        return g

    def used_inputs(self) -> List[bool]:
        used = set(self.outputs)
        for n in self.nodes:
            used.update(n.value_args())
        return [i in used for i in self.inputs]

    def uses(self, v: str) -> bool:
        if v in self.outputs:
            return True
        return any(v in n.value_args() for n in self.nodes)

    # ------------------------------------------------------------------ debug
    def code(self) -> str:
        cls = {(True, True): 'full', (True, False): 'col', (False, True): 'row', (False, False): 'scal'}
        lines = [f'def {self.name}(' + ', '.join(f'{i}:{cls[self.input_ext[i]]}' for i in self.inputs) + '):']
        for n in self.nodes:
            a = ', '.join(str(x) for x in n.args)
            d = f', dims={list(n.dims)}' if n.op == 'sum' else ''
            lines.append(f'    {n.name}:{cls[n.ext]} = {n.op}({a}{d})')
        lines.append('    return ' + ', '.join(self.outputs))
        return '\n'.join(lines)

    def signature(self) -> str:
        """Canonical text used for hashing (names are deterministic FX names)."""
        return self.code()


def broadcast_ext(exts: Iterable[Tuple[bool, bool]]) -> Tuple[bool, bool]:
    em = en = False
    for a, b in exts:
        em |= a
        en |= b
    return (em, en)
