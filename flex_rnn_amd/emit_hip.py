"""HIP (gfx950, wave64) code emitter for the three kernels of a plan.

Replaces the reference's CUDA text emitter (/root/reference/flex_rnn/to_cuda.py:7-124
`to_cuda`, 127-223 `parse_cuda`) and its three kernel templates
(/root/reference/flex_rnn/twopass.py:202-220 `fw`, 245-273 `bw1`, 285-339 `bw2`).
Nothing of their thread mapping is kept:

  * Row kernels (`fw`, `bw1`): a 64-lane wave is split into G = 64/L row groups of L
    lanes; a group holds R consecutive state rows in fp32 registers, C = N/L columns per
    lane.  `sum(-1)` is an in-lane chain over C followed by a DPP all-reduce inside the
    group (no LDS, no barrier).  Per-timestep operands are staged through LDS as fp32,
    TS timesteps at a time, by all threads of the workgroup (any stride / dtype is handled
    there); results go back the same way.
  * Gradient kernel (`bw2`): one lane per state column and DT timesteps per instance; a
    serial loop over the M rows recomputes the DT states of one element from its
    checkpoint (elementwise thanks to the saved row sums), runs the per-element backward,
    and accumulates the sums over rows in registers.  An epilogue maps them to row /
    scalar input gradients (column sums = wave all-reduce).

Shapes B, T, H, M and all strides are runtime kernel arguments; N, dtypes, operand
classes, broadcast pattern and tile sizes are baked into the source (and hence into the
cache key, which is a hash of the source).
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass, field
from typing import List, Sequence, Tuple

import torch as th

from .ir import Graph

# blocks a launch may have along grid y (hardware limit; the variable lets a test reach the folded form at small sizes)
MAX_GRID_Y = int(os.environ.get('FLEX_RNN_MAX_GRID_Y', '65535'))
DT_CODE = {th.float32: 0, th.bfloat16: 1, th.float16: 2, th.float64: 3}

PRELUDE = r'''
#include <hip/hip_runtime.h>
typedef long long i64;
typedef unsigned short u16_t;
struct TArg { void* p; i64 s[5]; };

template <int CTRL> __device__ __forceinline__ float dpp_mov(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
// Sum over the L (power of two) consecutive lanes of a group; every lane gets the total.
// quad_perm / row_half_mirror / row_mirror stay inside a 16-lane DPP row; wider groups
// cross rows with a lane permute.
// x + (x of the lane 16 / 32 away): the gfx950 row swaps exchange the odd 16-lane rows of one
// register with the even rows of another (the 32-lane halves for permlane32), so a register and
// its copy come back as "own rows twice" and "partner rows twice"; no trip through LDS.
__device__ __forceinline__ float xor16_sum(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}
__device__ __forceinline__ float xor32_sum(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}
template <int L> __device__ __forceinline__ float grp_allreduce(float x) {
  if constexpr (L >= 2) x += dpp_mov<0xB1>(x);    // quad_perm [1,0,3,2]
  if constexpr (L >= 4) x += dpp_mov<0x4E>(x);    // quad_perm [2,3,0,1]
  if constexpr (L >= 8) x += dpp_mov<0x141>(x);   // row_half_mirror
  if constexpr (L >= 16) x += dpp_mov<0x140>(x);  // row_mirror
  if constexpr (L >= 32) x = xor16_sum(x);
  if constexpr (L >= 64) x = xor32_sum(x);
  return x;
}

template <int DT> __device__ __forceinline__ float ldf(const void* p, i64 i);
template <> __device__ __forceinline__ float ldf<0>(const void* p, i64 i) { return ((const float*)p)[i]; }
template <> __device__ __forceinline__ float ldf<1>(const void* p, i64 i) {
  return __builtin_bit_cast(float, (unsigned)((const u16_t*)p)[i] << 16);
}
template <> __device__ __forceinline__ float ldf<2>(const void* p, i64 i) { return (float)((const _Float16*)p)[i]; }
template <> __device__ __forceinline__ float ldf<3>(const void* p, i64 i) { return (float)((const double*)p)[i]; }

// raw (unconverted) load into a 32-bit register and its conversion: lets a prefetch stay in flight
// without an instruction that consumes the loaded value
template <int DT> __device__ __forceinline__ unsigned ldr(const void* p, i64 i);
template <> __device__ __forceinline__ unsigned ldr<0>(const void* p, i64 i) { return ((const unsigned*)p)[i]; }
template <> __device__ __forceinline__ unsigned ldr<1>(const void* p, i64 i) { return ((const u16_t*)p)[i]; }
template <> __device__ __forceinline__ unsigned ldr<2>(const void* p, i64 i) { return ((const u16_t*)p)[i]; }
template <> __device__ __forceinline__ unsigned ldr<3>(const void* p, i64 i) {
  return __builtin_bit_cast(unsigned, (float)((const double*)p)[i]);
}
template <int DT> __device__ __forceinline__ float cvr(unsigned u);
template <> __device__ __forceinline__ float cvr<0>(unsigned u) { return __builtin_bit_cast(float, u); }
template <> __device__ __forceinline__ float cvr<1>(unsigned u) { return __builtin_bit_cast(float, u << 16); }
template <> __device__ __forceinline__ float cvr<2>(unsigned u) { return (float)__builtin_bit_cast(_Float16, (u16_t)u); }
template <> __device__ __forceinline__ float cvr<3>(unsigned u) { return __builtin_bit_cast(float, u); }

template <int DT> __device__ __forceinline__ void stf(void* p, i64 i, float v);
template <> __device__ __forceinline__ void stf<0>(void* p, i64 i, float v) { ((float*)p)[i] = v; }
template <> __device__ __forceinline__ void stf<1>(void* p, i64 i, float v) {
  ((u16_t*)p)[i] = __builtin_bit_cast(u16_t, (__bf16)v);
}
template <> __device__ __forceinline__ void stf<2>(void* p, i64 i, float v) { ((_Float16*)p)[i] = (_Float16)v; }
template <> __device__ __forceinline__ void stf<3>(void* p, i64 i, float v) { ((double*)p)[i] = (double)v; }

__device__ __forceinline__ void atomic_addf(void* p, i64 i, float v) {
  __hip_atomic_fetch_add(((float*)p) + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float f_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// a value that is the same on every lane of the wave, moved to a scalar register
__device__ __forceinline__ float wave_uniform(float x) { return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x))); }
// Division and friends at the precision of the reciprocal instruction (1 ulp; a quotient within about 2 ulp) instead of
// correctly rounded: 3-6 instructions instead of 10 for every quotient, 17 instead of 100 for log1p.  They sit in the per-timestep
// preparation of gates and norms and in its derivative, where they were most of the work.
__device__ __forceinline__ float f_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float f_div(float a, float b) {
  const float s = __builtin_fabsf(b) > 0x1p96f ? 0x1p-32f : 1.0f;      // keeps 1 / b out of the denormals
  return s * (a * f_rcp(b * s));
}
// log(1 + x) without cancellation: log(u) * x / (u - 1) with u = 1 + x as rounded, x itself where u rounds to 1
__device__ __forceinline__ float f_log1p(float x) {
  const float u = 1.0f + x, d = u - 1.0f;
  return d == 0.0f ? x : __logf(u) * (x * f_rcp(d));
}
__device__ __forceinline__ float f_sigmoid(float x) { return f_rcp(1.0f + __expf(-x)); }
__device__ __forceinline__ float f_tanh(float x) { return 1.0f - 2.0f * f_rcp(__expf(2.0f * x) + 1.0f); }
__device__ __forceinline__ float f_sign(float x) { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : 0.0f); }
'''


def _lit(v) -> str:
    v = float(v)
    if math.isinf(v):
        return '__builtin_inff()' if v > 0 else '(-__builtin_inff())'
    if math.isnan(v):
        return '__builtin_nanf("")'
    s = repr(v)
    if 'e' not in s and '.' not in s:
        s += '.0'
    return s + 'f'


_UNARY_EXPR = {
    'exp': '__expf({0})', 'neg': '(-{0})', 'reciprocal': 'f_rcp({0})', 'log': '__logf({0})',
    'sqrt': 'sqrtf({0})', 'rsqrt': 'rsqrtf({0})', 'sigmoid': 'f_sigmoid({0})', 'tanh': 'f_tanh({0})',
    'abs': '__builtin_fabsf({0})', 'relu': 'fmaxf({0}, 0.0f)', 'sign': 'f_sign({0})',
    'log1p': 'f_log1p({0})', 'expm1': 'expm1f({0})', 'copy': '({0})',
    'sin': 'sinf({0})', 'cos': 'cosf({0})', 'erf': 'erff({0})', 'log2': '__log2f({0})', 'exp2': 'f_exp2({0})',
}
_BINARY_EXPR = {
    'mul': '({0} * {1})', 'add': '({0} + {1})', 'sub': '({0} - {1})', 'div': 'f_div({0}, {1})',
    'lt': '(({0} < {1}) ? 1.0f : 0.0f)', 'gt': '(({0} > {1}) ? 1.0f : 0.0f)',
    'le': '(({0} <= {1}) ? 1.0f : 0.0f)', 'ge': '(({0} >= {1}) ? 1.0f : 0.0f)',
    'eq': '(({0} == {1}) ? 1.0f : 0.0f)', 'ne': '(({0} != {1}) ? 1.0f : 0.0f)',
    'maximum': 'fmaxf({0}, {1})', 'minimum': 'fminf({0}, {1})',
}


def _dims(ext, R, C):
    return (R if ext[0] else 1, C if ext[1] else 1)


def _ref(name, ext, R, C, const):
    rr, cc = _dims(ext, R, C)
    return f"{'const ' if const else ''}float (&{name})[{rr}][{cc}]"


def _at(name, ext):
    return f"{name}[{'r' if ext[0] else '0'}][{'c' if ext[1] else '0'}]"


def _loops(rr, cc):
    return (f'#pragma unroll\n  for (int r = 0; r < {rr}; r++)\n'
            f'#pragma unroll\n  for (int c = 0; c < {cc}; c++)\n    ')


def emit_graph_fn(g: Graph, fname: str, R: int, C: int, out_exts: Sequence[Tuple[bool, bool]],
                  reduce_fn: str, invariant: Sequence[str] = (), colmask: str = '',
                  prolog: str = '') -> Tuple[str, List[str]]:
    """Device function evaluating `g` on register tiles.  Every value is a `float[RR][CC]`
    array with RR = R if it varies along rows else 1, CC likewise for columns.  Returns the
    source and the list of graph inputs that appear in the signature (the used ones).

    `invariant` names graph inputs that do not change from one timestep to the next.
    `exp(u * v)` with such a `v` is evaluated as `exp2(u * (v * log2 e))`: the hardware
    exponential is base 2, and the rescaled `v` is loop-invariant for the compiler to hoist,
    which saves the multiply by log2 e on every step.

    `colmask` (an expression in `c`, or empty) is true for real state columns; with a state width
    that is not a power of two the padding columns are kept out of every sum by it."""
    ext = g.ext_table()
    nm = g.node_map()
    invariant = set(invariant)
    used = [i for i, u in zip(g.inputs, g.used_inputs()) if u]
    params = [_ref(i, g.input_ext[i], R, C, True) for i in used]
    params += [_ref(f'o{k}_', e, R, C, False) for k, e in enumerate(out_exts)]
    out = [f'__device__ __forceinline__ void {fname}(' + ', '.join(params) + ') {']
    if prolog:
        out.append('  ' + prolog)
    for n in g.nodes:
        rr, cc = _dims(n.ext, R, C)
        out.append(f'  float {n.name}[{rr}][{cc}];')

        def opnd(a):
            return _at(a, ext[a]) if isinstance(a, str) else _lit(a)

        if n.op == 'sum':
            assert n.dims == (1,), n
            src = n.args[0]
            sext = ext[src]
            assert sext[1]
            srr = R if sext[0] else 1
            s_at = f"{src}[{'r' if sext[0] else '0'}]"
            term = (lambda c: f'(({colmask.replace("(c)", f"({c})")}) ? {s_at}[{c}] : 0.0f)') if colmask else (lambda c: f'{s_at}[{c}]')
            out.append(f'#pragma unroll\n  for (int r = 0; r < {srr}; r++) {{\n'
                       f'    float s_ = {term("0")};\n'
                       f'#pragma unroll\n    for (int c = 1; c < {C}; c++) s_ += {term("c")};\n'
                       f'    {n.name}[r][0] = {reduce_fn}(s_);\n  }}')
        elif n.op == 'const':
            out.append(f'  {n.name}[0][0] = {_lit(n.args[0])};')
        elif n.op == 'exp' and isinstance(n.args[0], str) and n.args[0] in nm and nm[n.args[0]].op == 'mul' \
                and any(a in invariant for a in nm[n.args[0]].value_args()) and len(nm[n.args[0]].value_args()) == 2:
            u, v = nm[n.args[0]].args
            if u in invariant:
                u, v = v, u
            out.append('  ' + _loops(rr, cc) + f'{n.name}[r][c] = f_exp2({opnd(u)} * ({opnd(v)} * 1.4426950408889634f));')
        elif n.op in _UNARY_EXPR:
            out.append('  ' + _loops(rr, cc) + f'{n.name}[r][c] = ' + _UNARY_EXPR[n.op].format(opnd(n.args[0])) + ';')
        elif n.op in _BINARY_EXPR:
            out.append('  ' + _loops(rr, cc) + f'{n.name}[r][c] = '
                       + _BINARY_EXPR[n.op].format(opnd(n.args[0]), opnd(n.args[1])) + ';')
        elif n.op == 'where':
            out.append('  ' + _loops(rr, cc) + f'{n.name}[r][c] = (({opnd(n.args[0])} != 0.0f) ? '
                       f'{opnd(n.args[1])} : {opnd(n.args[2])});')
        else:
            raise NotImplementedError(n.op)
    for k, (o, e) in enumerate(zip(g.outputs, out_exts)):
        oe = ext[o]
        assert (not oe[0] or e[0]) and (not oe[1] or e[1]), (fname, o, oe, e)
        rr, cc = _dims(e, R, C)
        out.append('  ' + _loops(rr, cc) + f'o{k}_[r][c] = {_at(o, oe)};')
    out.append('}')
    return '\n'.join(out), used


# ------------------------------------------------------------------------------------ kernels

@dataclass
class KernelSpec:
    name: str
    source: str
    tensors: List[str]          # logical tensor names, in Args order
    block: int
    grid: Tuple[str, str, str]  # python expressions over B, T, H, M, nch
    geom: dict = field(default_factory=dict)    # what the grid is meant to cover (rows per workgroup, chunks per workgroup, row slices):
                                # the host checks the evaluated grid against it before a launch when asked to


class _Args:
    """Allocates TArg slots and renders `A.t[k]` accessors."""

    def __init__(self):
        self.names: List[str] = []

    def slot(self, name: str) -> int:
        if name not in self.names:
            self.names.append(name)
        return self.names.index(name)

    def p(self, name: str) -> str:
        return f'A.t[{self.slot(name)}].p'

    def s(self, name: str, d: int) -> str:
        return f'A.t[{self.slot(name)}].s[{d}]'

    def struct(self) -> str:
        return f'struct Args {{ TArg t[{max(len(self.names), 1)}]; i64 B, T, H, M, nch; }};\n'


class _Stager:
    """Global -> LDS staging of per-timestep operands for TS timesteps, split in two phases so
    that the loads of the next chunk are in flight while the current one is computed:
    `load(t0)` issues every load of the chunk back to back into registers (raw bits),
    `write()` converts them to fp32 and stores them to LDS.  Element e = tid + it*NT of the
    [TS][ln] tile is (timestep e / ln, position e % ln); when NT is a multiple of ln the position
    is the same for every `it`, so one 64-bit base index per operand is computed up front
    (`bases()`) and each load adds a multiple of the operand's time stride.  With `tail` the
    timestep is clamped to T-1 (the last chunk may be partial; the surplus values are unused)."""

    def __init__(self, TS: int, NT: int, tail: bool = False):
        self.TS, self.NT, self.tail = TS, NT, tail
        self.items = []      # (lds name, row length, dtype code, pointer, index fn(t, x_), time stride)
        self.no_lds = set()  # items that only feed derived operands: prefetched, never written to LDS
        self.width = {}      # LDS row width per item (>= its row length)
        self.derived = None  # (function name, [source item names], [derived lds names], row length)

    def add(self, name, ln, dt, ptr, idx_fn, tstride, lds=True, width=None):
        """`width` > `ln`: the LDS rows are that wide and the surplus (padding columns of a state
        width that is not a power of two) is zeroed once, by `zero_pads()`."""
        self.items.append((name, ln, dt, ptr, idx_fn, tstride))
        self.width[name] = width or ln
        if not lds:
            self.no_lds.add(name)

    def derive(self, fn_name, sources, outputs, ln, width=None):
        """Operands computed while staging: `fn_name(src..., out...)` is evaluated once per
        (timestep, position) from the converted prefetch registers of `sources` (items of row
        length `ln`) and its results are written to the LDS arrays `outputs`."""
        self.derived = (fn_name, list(sources), list(outputs), ln)
        for o in outputs:
            self.width[o] = width or ln

    def _iters(self, ln):
        return (self.TS * ln + self.NT - 1) // self.NT

    def _linear(self, ln):
        return self.NT % ln == 0

    def decls(self) -> str:
        out = ''
        for name, ln, dt, ptr, fn, ts in self.items:
            if name not in self.no_lds:
                out += f'  __shared__ float {name}[{self.TS}][{self.width[name]}];\n'
            out += f'  unsigned pf_{name}[{self._iters(ln)}];\n'
        if self.derived:
            for o in self.derived[2]:
                out += f'  __shared__ float {o}[{self.TS}][{self.width[o]}];\n'
        return out

    def zero_pads(self) -> str:
        """Clears the padding columns of every LDS array wider than its operand (nothing else ever
        writes them); a barrier must follow before the arrays are read."""
        out = ''
        arrays = [(name, ln) for name, ln, *_ in self.items if name not in self.no_lds]
        if self.derived:
            arrays += [(o, self.derived[3]) for o in self.derived[2]]
        for name, ln in arrays:
            pad = self.width[name] - ln
            if pad > 0:
                out += (f'  for (int e_ = tid; e_ < {self.TS * pad}; e_ += {self.NT}) '
                        f'{name}[e_ / {pad}][{ln} + e_ % {pad}] = 0.0f;\n')
        return out

    def bases(self) -> str:
        out = ''
        for name, ln, dt, ptr, fn, ts in self.items:
            if self._linear(ln):
                if self.tail:       # the timestep is clamped per thread, keep it out of the base
                    out += f'  const i64 pb_{name} = {fn("0", f"(tid % {ln})")};\n  const int tb_{name} = tid / {ln};\n'
                else:               # base holds the thread's own timestep; loads add a wave-uniform offset
                    out += f'  const i64 pb_{name} = {fn(f"(tid / {ln})", f"(tid % {ln})")};\n'
        return out

    def _loop(self, ln, body, ind):
        tot = self.TS * ln
        guard = '' if tot % self.NT == 0 else f'if (e_ < {tot}) '
        return (f'#pragma unroll\n{ind}for (int it_ = 0; it_ < {self._iters(ln)}; it_++) {{ const int e_ = tid + it_ * {self.NT}; '
                f'const int tt_ = e_ / {ln}, x_ = e_ % {ln}; (void)tt_; (void)x_; {guard}{body} }}\n')

    def _clamp(self, t):
        return f'min({t}, T - 1)' if self.tail else t

    def load(self, t0: str, ind: str) -> str:
        out = ''
        for name, ln, dt, ptr, fn, ts in self.items:
            if self._linear(ln) and self.tail:
                t = self._clamp(f'({t0}) + tb_{name} + it_ * {self.NT // ln}')
                idx = f'pb_{name} + (i64)({t}) * {ts}'
            elif self._linear(ln):
                idx = f'pb_{name} + (i64)(({t0}) + it_ * {self.NT // ln}) * {ts}'
            else:
                idx = fn(self._clamp(f'({t0}) + tt_'), 'x_')
            out += self._loop(ln, f'pf_{name}[it_] = ldr<{dt}>({ptr}, {idx});', ind)
        return out

    def write(self, ind: str) -> str:
        out = ''
        for name, ln, dt, ptr, fn, ts in self.items:
            if name not in self.no_lds:
                out += self._loop(ln, f'{name}[tt_][x_] = cvr<{dt}>(pf_{name}[it_]);', ind)
        if self.derived:
            fn_name, sources, outputs, ln = self.derived
            dts = {name: dt for name, _, dt, _, _, _ in self.items}
            body = '{ ' + ' '.join(f'float a{k}_[1][1]; a{k}_[0][0] = cvr<{dts[s_]}>(pf_{s_}[it_]);' for k, s_ in enumerate(sources))
            body += ' ' + ' '.join(f'float d{k}_[1][1];' for k in range(len(outputs)))
            body += f' {fn_name}(' + ', '.join([f'a{k}_' for k in range(len(sources))] + [f'd{k}_' for k in range(len(outputs))]) + ');'
            body += ' ' + ' '.join(f'{o}[tt_][x_] = d{k}_[0][0];' for k, o in enumerate(outputs)) + ' }'
            out += self._loop(ln, body, ind)
        return out


class _Prologue:
    """Values of a step that do not vary along the state's rows and are not plain inputs - a gate's sigmoid, a
    softplus step size, an L2-normalised key, anything a traced layer moved into the step - evaluated by the
    workgroup once per (timestep, column) right after a block of timesteps was staged, instead of by every row group
    of every wave inside the step.  `front` are the outermost such values (those a value with a row extent, or a
    result, reads); the step takes them from LDS like staged operands.

    On the way to them the graph is cut at every value that is one number per timestep: sums over the columns (the
    squared norm of a key) and the outermost values computed from scalars alone (a gate).  Cuts are grouped into
    levels by what they depend on; a level's sums are formed by groups of 16 lanes, one timestep per group, its
    scalar values by one lane per timestep, then a barrier.  A last pass evaluates the front values per
    (timestep, column) from the raw LDS rows and the cuts.  Inputs without a time axis are put into LDS once, before
    the time loop."""

    def __init__(self, em: 'Emitter', front, tag: str, TS: int, NT: int, A: '_Args'):
        p, joint = em.p, em.p.joint
        self.em, self.front, self.tag, self.TS, self.NT, self.A = em, list(front), tag, TS, NT, A
        self.jext = em.jext
        nm = joint.node_map()
        need, stack = set(), list(front)
        while stack:
            v = stack.pop()
            if v in need:
                continue
            need.add(v)
            if v in nm:
                stack.extend(nm[v].value_args())
        nodes = [n for n in joint.nodes if n.name in need]
        self.inputs = [i for i in range(p.ninputs) if p.in_names[i] in need]
        for i in self.inputs:
            assert not em.in_ext(i)[0], p.in_names[i]
        # cuts: sums, and scalar values that a per-column value (or the step) reads
        cuts = []
        for n in nodes:
            if n.op == 'sum':
                cuts.append(n.name)
            elif n.ext == (False, False) and n.op != 'const' and (
                    n.name in front or any(n.name in m.value_args() and m.ext[1] for m in nodes)):
                cuts.append(n.name)
        # level of a cut: one more than the highest level among the cuts it is computed from
        dep, level = {}, {}
        for n in nodes:
            d = set()
            for a in n.value_args():
                d |= ({a} if a in cuts else set()) | dep.get(a, set())
            dep[n.name] = d
        for c in cuts:
            level[c] = 1 + max((level[d] for d in dep[c]), default=-1)
        self.cuts = cuts
        self.fns, self.levels = [], []          # device functions; per level: (sum pass or None, scalar pass or None)
        for lv in range(1 + max(level.values(), default=-1)):
            done = [c for c in cuts if level[c] < lv]
            passes = []
            for kind in ('sum', 'scalar'):
                mine = [c for c in cuts if level[c] == lv and (nm[c].op == 'sum') == (kind == 'sum')]
                if not mine:
                    passes.append(None)
                    continue
                outs = [nm[c].args[0] for c in mine] if kind == 'sum' else mine
                fname = f'{tag}_p{kind}{lv}'
                g = joint.extract(fname, outs, cut=done)
                src, used = emit_graph_fn(g, fname, 1, 1, [(False, kind == 'sum')] * len(outs), 'grp_allreduce<1>', em.invariant)
                self.fns.append(src)
                passes.append((fname, used, mine))
            self.levels.append(passes)
        g = joint.extract(f'{tag}_pfront', self.front, cut=cuts)
        src, used = emit_graph_fn(g, f'{tag}_pfront', 1, 1, [self.jext[f] for f in self.front], 'grp_allreduce<1>', em.invariant)
        self.fns.append(src)
        self.final = (f'{tag}_pfront', used)

    def source(self) -> str:
        return '\n'.join(self.fns)

    def decls(self) -> str:
        em = self.em
        out = ''
        for j in range(len(self.cuts)):
            out += f'  __shared__ float s_pc{j}[{self.TS}];\n'
        for q, f in enumerate(self.front):
            out += f'  __shared__ float s_d{q}[{self.TS}][{em.NP if self.jext[f][1] else 1}];\n'
        for i in self.inputs:
            if not em.tdep[i]:
                out += f'  __shared__ float s_k{i}[{em.NP if em.in_ext(i)[1] else 1}];\n'
        return out

    def init(self) -> str:
        """Inputs without a time axis into LDS, and the padding columns of the front arrays cleared (once; a barrier
        follows before anything reads them)."""
        em, A = self.em, self.A
        out = ''
        for i in self.inputs:
            if em.tdep[i]:
                continue
            dt = DT_CODE[em.plan.in_dtypes[i]]
            if em.in_ext(i)[1]:
                out += (f'  for (int x_ = tid; x_ < {em.N}; x_ += {self.NT}) s_k{i}[x_] = '
                        f'ldf<{dt}>({A.p(f"in{i}")}, {em._in_index(A, i, t="0", n="x_")});\n')
            else:
                out += f'  if (tid == 0) s_k{i}[0] = ldf<{dt}>({A.p(f"in{i}")}, {em._in_index(A, i, t="0")});\n'
        if em.pad:
            pad = em.NP - em.N
            for q, f in enumerate(self.front):
                if self.jext[f][1]:
                    out += (f'  for (int e_ = tid; e_ < {self.TS * pad}; e_ += {self.NT}) '
                            f's_d{q}[e_ / {pad}][{em.N} + e_ % {pad}] = 0.0f;\n')
        return out

    def _value(self, v: str) -> str:
        """Expression for graph value `v` at (timestep tt_, column x_)."""
        em, p = self.em, self.em.p
        if v in self.cuts:
            return f's_pc{self.cuts.index(v)}[tt_]'
        i = p.in_names.index(v)
        col = 'x_' if em.in_ext(i)[1] else '0'
        return f's_in{i}[tt_][{col}]' if em.tdep[i] else f's_k{i}[{col}]'

    def _call(self, fname, used, outs) -> str:
        args = ' '.join(f'float a{k}_[1][1]; a{k}_[0][0] = {self._value(v)};' for k, v in enumerate(used))
        decl = ' '.join(f'float {o}[1][1];' for o in outs)
        return f'{args} {decl} {fname}(' + ', '.join([f'a{k}_' for k in range(len(used))] + list(outs)) + ');'

    def run(self, ind: str) -> str:
        """The passes of one staged block; ends with a barrier."""
        em, TS, NT = self.em, self.TS, self.NT
        out = ''
        for sums, scalars in self.levels:
            if sums:
                fname, used, mine = sums
                outs = [f'o{k}_' for k in range(len(mine))]
                # (every group of 16 lanes makes the same number of rounds, so that the cross-lane adds sit in uniform
                # control flow; a group without a timestep left works on the last one again and stores nothing)
                groups = NT // 16
                out += (f'{ind}for (int r_ = 0; r_ < {-(-TS // groups)}; r_++) {{ const int tq_ = tid / 16 + r_ * {groups}, tt_ = min(tq_, {TS - 1}); '
                        + ' '.join(f'float s{k}_ = 0.0f;' for k in range(len(mine))) + '\n'
                        f'{ind}  for (int x_ = tid % 16; x_ < {em.N}; x_ += 16) {{ {self._call(fname, used, outs)} '
                        + ' '.join(f's{k}_ += o{k}_[0][0];' for k in range(len(mine))) + ' }\n'
                        + ''.join(f'{ind}  s{k}_ = grp_allreduce<16>(s{k}_);\n' for k in range(len(mine)))
                        + f'{ind}  if ((tid & 15) == 0 && tq_ < {TS}) {{ ' + ' '.join(f's_pc{self.cuts.index(c)}[tt_] = s{k}_;' for k, c in enumerate(mine))
                        + ' } }\n')
            if scalars:
                fname, used, mine = scalars
                outs = [f'o{k}_' for k in range(len(mine))]
                out += (f'{ind}for (int tt_ = tid; tt_ < {TS}; tt_ += {NT}) {{ const int x_ = 0; (void)x_; {self._call(fname, used, outs)} '
                        + ' '.join(f's_pc{self.cuts.index(c)}[tt_] = o{k}_[0][0];' for k, c in enumerate(mine)) + ' }\n')
            out += f'{ind}__syncthreads();\n'
        fname, used = self.final
        outs = [f'o{q}_' for q in range(len(self.front))]
        vec = [(q, f) for q, f in enumerate(self.front) if self.jext[f][1]]
        sca = [(q, f) for q, f in enumerate(self.front) if not self.jext[f][1]]
        stores = ' '.join(f's_d{q}[tt_][x_] = o{q}_[0][0];' for q, f in vec)
        if sca:
            stores += ' if (x_ == 0) { ' + ' '.join(f's_d{q}[tt_][0] = o{q}_[0][0];' for q, f in sca) + ' }'
        total = TS * em.N if vec else TS
        step = em.N if vec else 1
        out += (f'{ind}for (int e_ = tid; e_ < {total}; e_ += {NT}) {{ const int tt_ = e_ / {step}, x_ = e_ % {step}; (void)x_;\n'
                f'{ind}  {self._call(fname, used, outs)} {stores} }}\n'
                f'{ind}__syncthreads();\n')
        return out


def _col_expr(C: int, L: int) -> str:
    """Column owned by (lane-in-group l, element c).  With C >= 4 a lane owns float4
    pieces, interleaved across the group so that 16 lanes x 16 B is one contiguous row
    segment (conflict-free ds_read_b128, full-line global access)."""
    if C >= 4:
        return f'(((c) >> 2) * {4 * L} + l * 4 + ((c) & 3))'
    return f'(l * {C} + (c))'


def needs_gradient_kernel(part) -> bool:
    """The per-chunk gradient kernel produces the row- and scalar-input gradients and, unless the
    reverse scan already does, the matrix-input gradients.  A recurrence with none of these
    (all inputs per-row, e.g. a vector state) is finished after the reverse scan."""
    return bool(part.row_idx or part.scalar_idx or (part.mat_idx and not part.mat_in_dstep))


class Emitter:
    def __init__(self, plan):
        self.plan = plan
        self.p = plan.part
        self.tile = plan.tile
        p = self.p
        self.cls = plan.in_cls
        # staged per timestep: everything but matrix inputs and inputs with a size-1 time axis
        # (when T == 1 every non-matrix input counts as time-dependent, with a single step)
        self.tdep = [(plan.T == 1 or not b[1]) and c != 'mat' for b, c in zip(plan.in_bcast, self.cls)]
        self.atomic = set(plan.atomic)
        # state width: N as given, NP as laid out (next power of two); `pad` when they differ
        self.N, self.NP = plan.N, plan.NP
        self.pad = plan.NP != plan.N
        self.colmask = f'COL(c) < {plan.N}' if self.pad else ''
        self.invariant = {nm for nm, td in zip(p.in_names, self.tdep) if not td}
        self.jext = p.joint.ext_table()
        # the last chunk is partial when T is not a multiple of the chunk sizes; the guards that
        # handles it are only emitted then, so aligned lengths keep the unguarded code
        self.tail_dt = plan.T % plan.tile.DT != 0

    # ------------------------------------------------------------------ helpers
    def in_ext(self, i: int):
        return {'scalar': (False, False), 'col': (True, False), 'row': (False, True), 'mat': (True, True)}[self.cls[i]]

    def _in_index(self, A: _Args, i: int, b='b', t='t', h='h', m=None, n=None) -> str:
        """Element offset into input i (strides of broadcast dims are 0 at launch)."""
        nm = f'in{i}'
        terms = [f'(i64){b} * {A.s(nm, 0)}', f'(i64)({t}) * {A.s(nm, 1)}', f'(i64){h} * {A.s(nm, 2)}']
        if m is not None:
            terms.append(f'(i64)({m}) * {A.s(nm, 3)}')
        if n is not None:
            terms.append(f'(i64)({n}) * {A.s(nm, 4)}')
        return ' + '.join(terms)

    def _kept_sums(self, TS: int, reverse: bool):
        """(Lk, J) when a block's row sums stay in registers until the block is done - after the all-reduce every lane of
        a group holds them, so lane l keeps those of the steps l, l + Lk, ... (J of them) and stores them once, to
        distinct addresses - or None for a store per step (by every lane of the group to one address, or by lane 0 under
        a branch).  Four LDS stores per step and wave become eight per block at the price of a select per row sum and
        step: RWKV-7's forward kernel 0.81 -> 0.78 ms, its reverse scan (short of issue slots, not of LDS) 0.75 -> 0.76 ms."""
        t = self.tile
        if not getattr(t, 'KS', 0) & (2 if reverse else 1) or t.L < 2:
            return None
        Lk = min(t.L, TS)
        J = TS // Lk
        return (Lk, J) if TS % Lk == 0 and J <= 2 else None

    KEPT_PAD = 4         # floats between the rows of a result array in LDS when lanes of a group store different timesteps

    # ------------------------------------------------------------------ row kernels
    def _row_front(self, graphs):
        """Row operands that can be computed while staging.  In the row kernels a value with a
        column but no row extent (a function of a timestep's row inputs: the exponential of a
        log-decay, a gate's sigmoid, a normalised key) would be recomputed by every row group of
        every wave.  Returns the outermost such values that depend on nothing but staged row
        inputs and constants; the staging threads evaluate them once per (timestep, column)."""
        p = self.p
        ok = {p.in_names[i] for i in range(p.ninputs) if self.tdep[i] and self.in_ext(i) == (False, True)}
        front = []
        for g in graphs:
            consts, pure = set(), set()
            for n in g.nodes:
                args = n.value_args()
                if n.op == 'const' or (n.op != 'sum' and n.ext == (False, False) and args and all(a in consts for a in args)):
                    consts.add(n.name)
                elif n.op != 'sum' and n.ext == (False, True) and all(a in ok or a in pure or a in consts for a in args) \
                        and any(a in ok or a in pure for a in args):
                    pure.add(n.name)
            for n in g.nodes:
                if n.name in pure and n.name not in front and (
                        n.name in g.outputs or any(n.name in m.value_args() and m.name not in pure for m in g.nodes)):
                    front.append(n.name)
        return front

    def _prologue_front(self, graphs):
        """`partition.prologue_front`; what `_row_front` finds is the special case that needs no pass of its own
        (values of one column of staged row inputs, no sums)."""
        from .partition import prologue_front
        return prologue_front(graphs)

    def _levelled(self, g: Graph, fname: str, out_exts, colmask: str = '', prolog: str = ''):
        """`g` cut at its sums, for kernels in which a sum over the columns crosses waves (two barriers each): a
        function per level that returns the operands of that level's sums (levels by dependence among the sums), and
        a last one that returns the results, each taking the sums below it as inputs.  The caller evaluates a level for
        all timesteps of a chunk, reduces everything in one exchange, and goes on.  None when `g` has no sums."""
        sums = [n for n in g.nodes if n.op == 'sum']
        if not sums:
            return None
        names = [n.name for n in sums]
        dep = {}
        for n in g.nodes:
            d = set()
            for a in n.value_args():
                d |= ({a} if a in names else set()) | dep.get(a, set())
            dep[n.name] = d
        level = {}
        for n in sums:
            level[n.name] = 1 + max((level[d] for d in dep[n.name]), default=-1)
        nm = g.node_map()
        out = {'levels': [], 'sums': names, 'src': []}
        for lv in range(1 + max(level.values())):
            mine = [c for c in names if level[c] == lv]
            done = [c for c in names if level[c] < lv]
            sub = g.extract(f'{fname}_s{lv}', [nm[c].args[0] for c in mine], cut=done)
            src, used = emit_graph_fn(sub, f'{fname}_s{lv}', 1, 1, [(False, True)] * len(mine), 'grp_allreduce<1>', self.invariant, colmask, prolog)
            out['levels'].append((f'{fname}_s{lv}', used, mine))
            out['src'].append(src)
        sub = g.extract(f'{fname}_f', g.outputs, cut=names)
        src, used = emit_graph_fn(sub, f'{fname}_f', 1, 1, out_exts, 'grp_allreduce<1>', self.invariant, colmask, prolog)
        out['final'] = (f'{fname}_f', used)
        out['src'].append(src)
        out['used'] = sorted({v for _, u, _ in out['levels'] for v in u if v not in names} | {v for v in used if v not in names})
        return out

    def _stage_row_front(self, stg: '_Stager', A: _Args, front, direct_used, MT: int, fn_name: str):
        """Registers the raw inputs the derived operands need (without an LDS array of their own
        unless the step function also reads them directly) and the derivation itself; returns the
        source of the device function."""
        p = self.p
        pre_g = p.joint.extract(fn_name, front, cut=())
        src, used = emit_graph_fn(pre_g, fn_name, 1, 1, [(False, True)] * len(front), 'grp_allreduce<1>')
        have = {it[0] for it in stg.items}
        for v in used:
            i = p.in_names.index(v)
            if f's_in{i}' not in have:
                ext = self.in_ext(i)
                assert ext == (False, True)
                dt = DT_CODE[self.plan.in_dtypes[i]]
                stg.add(f's_in{i}', self.N, dt, A.p(f'in{i}'), lambda tt, x, i=i: self._in_index(A, i, t=tt, n=x),
                        A.s(f'in{i}', 1), lds=p.in_names[i] in direct_used, width=self.NP)
        stg.derive(fn_name, [f's_in{p.in_names.index(v)}' for v in used], [f's_d{q}' for q in range(len(front))],
                   self.N, width=self.NP)
        return src

    def _row_kernel_common(self, R: int, W: int):
        """Declarations shared by fw and bw1: thread mapping and staging buffers."""
        t = self.tile
        L, C, G = t.L, t.C, t.G
        MT = W * G * R
        src = []
        src.append(f'''  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l = lane % {L}, grp = lane / {L};
  const int mt = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int rloc = (wave * {G} + grp) * {R};
  const int row0 = mt * {MT} + rloc;
  const int T = (int)A.T, H = (int)A.H, M = (int)A.M, nch = (int)A.nch;
  (void)T; (void)H; (void)nch;
''')
        return src, MT

    def _row_macros(self) -> str:
        """File-scope macros of the row kernels: column of (lane-in-group `l`, element c), the same
        clamped to the real width, and the clamped row."""
        t = self.tile
        return (f'#define COL(c) {_col_expr(t.C, t.L)}\n'
                f'#define COLC(c) {f"(min(COL(c), {self.N - 1}))" if self.pad else "COL(c)"}\n'
                '#define ROWC(r) (min(row0 + (r), M - 1))\n')

    def _row_attr(self) -> str:
        """Occupancy request of the row kernels (`TileConfig.WPE` waves per SIMD): the compiler then fits the
        kernel into 512 / WPE registers instead of using all a workgroup of its size may have."""
        wpe = int(getattr(self.tile, 'WPE', 0) or 0)
        wn = int(getattr(self.tile, 'WN', 0) or 0)
        if not wpe and wn:          # a lower bound only: 512 / WN registers as budget, more waves if fewer are used
            return f' __attribute__((amdgpu_waves_per_eu({wn})))'
        return f' __attribute__((amdgpu_waves_per_eu({wpe},{wpe})))' if wpe else ''

    def _lane_prolog(self) -> str:
        """What a device function needs to evaluate COL(c) on its own (only emitted with padding)."""
        return f'const int l = (threadIdx.x & 63) % {self.tile.L};' if self.pad else ''

    def _stage_input(self, st: '_Stager', A: _Args, i: int, MT: int):
        ext = self.in_ext(i)
        N = self.N
        dt = DT_CODE[self.plan.in_dtypes[i]]
        ts = A.s(f'in{i}', 1)
        if ext == (False, True):
            st.add(f's_in{i}', N, dt, A.p(f'in{i}'), lambda tt, x, i=i: self._in_index(A, i, t=tt, n=x), ts, width=self.NP)
        elif ext == (True, False):
            st.add(f's_in{i}', MT, dt, A.p(f'in{i}'),
                   lambda tt, x, i=i: self._in_index(A, i, t=tt, m=f'min(mt * {MT} + {x}, M - 1)'), ts)
        else:
            st.add(f's_in{i}', 1, dt, A.p(f'in{i}'), lambda tt, x, i=i: self._in_index(A, i, t=tt), ts)

    @staticmethod
    def _operand_order(g: Graph, names, skip=()):
        """The graph inputs `names` in the order a step of `g` needs them: first those that its first row sum
        depends on (a step cannot start before it has them), then the rest by first use.  States (`skip`) are
        registers, not LDS operands."""
        nm = g.node_map()
        first = next((n for n in g.nodes if n.op == 'sum'), None)
        seen = set()
        if first is not None:
            stack = [first.name]
            while stack:
                v = stack.pop()
                if v not in seen:
                    seen.add(v)
                    if v in nm:
                        stack.extend(nm[v].value_args())
        early = [v for v in names if v in seen and v not in skip]
        pos = {}
        for k, n in enumerate(g.nodes):
            for a in n.value_args():
                pos.setdefault(a, k)
        rest = sorted((v for v in names if v not in early), key=lambda v: pos.get(v, len(g.nodes)))
        return early + rest

    def _load_operand(self, var: str, sname: str, ext, R: int, C: int, tt: str) -> str:
        """Registers <- staged LDS operand for timestep tt."""
        if ext == (False, True):
            return (f'      float {var}[1][{C}];\n#pragma unroll\n      for (int c = 0; c < {C}; c++) '
                    f'{var}[0][c] = {sname}[{tt}][COL(c)];\n')
        if ext == (True, False):
            return (f'      float {var}[{R}][1];\n#pragma unroll\n      for (int r = 0; r < {R}; r++) '
                    f'{var}[r][0] = {sname}[{tt}][rloc + r];\n')
        if ext == (False, False):
            return f'      float {var}[1][1]; {var}[0][0] = {sname}[{tt}][0];\n'
        raise AssertionError

    def _load_const_input(self, A: _Args, i: int, R: int, C: int) -> str:
        """Time-independent input -> registers, once."""
        ext = self.in_ext(i)
        rr, cc = _dims(ext, R, C)
        dt = DT_CODE[self.plan.in_dtypes[i]]
        idx = self._in_index(A, i, t='0', m='ROWC(r)' if ext[0] else None, n='COLC(c)' if ext[1] else None)
        val = self._col_guard(f'ldf<{dt}>({A.p(f"in{i}")}, {idx})') if ext[1] else f'ldf<{dt}>({A.p(f"in{i}")}, {idx})'
        return (f'  float x{i}[{rr}][{cc}];\n#pragma unroll\n  for (int r = 0; r < {rr}; r++)\n'
                f'#pragma unroll\n  for (int c = 0; c < {cc}; c++) x{i}[r][c] = {val};\n')

    def _col_guard(self, expr: str) -> str:
        """`expr` for real columns, 0 for padding columns (its address uses COLC, the clamped column)."""
        return f'((COL(c) < {self.N}) ? {expr} : 0.0f)' if self.pad else expr

    def _col_if(self) -> str:
        """Statement prefix that skips padding columns."""
        return f'if (COL(c) < {self.N}) ' if self.pad else ''

    def _ck_index(self, chunk: str) -> str:
        return f'(((i64)(b * H + h) * nch + ({chunk})) * M + (row0 + r)) * {self.NP} + COL(c)'

    # ------------------------------------------------------------------ fw
    def fw(self, save: bool = True) -> KernelSpec:
        """Forward recurrence.  With `save=False` (inference: no backward pass will follow) the state
        checkpoints and the per-step row sums are not written; the kernel is then named `frnn_fwi`."""
        p, plan, t = self.p, self.plan, self.tile
        L, C, G, R, W, DT, TS = t.L, t.C, t.G, t.R, t.W, t.DT, t.TS
        N = plan.N
        NT = W * 64
        A = _Args()
        g = p.fw
        nin, nst, nout, naux = p.ninputs, p.nstates, p.noutputs, len(p.aux)
        kname = 'frnn_fw' if save else 'frnn_fwi'
        if not save:
            g = g.extract('fw', g.outputs[:nout + nst], cut=())
            naux = 0
        out_exts = [(True, False)] * nout + [(True, True)] * nst + [(True, False)] * naux
        # a state of a problem with M == 1 or N == 1 has a smaller extent; follow the joint graph
        st_ext = [self.jext[s] for s in p.st_names]
        out_exts = [(st_ext[0][0], False)] * nout + st_ext + [(st_ext[0][0], False)] * naux
        rfront = self._row_front([g])
        pro = None
        if sorted(rfront) != sorted(self._prologue_front([g])):        # sums or scalars on the way: a pass of its own
            pro = _Prologue(self, self._prologue_front([g]), 'fw', TS, NT, A)
            rfront = pro.front
        if rfront:
            g = g.extract('fw', g.outputs, cut=rfront)
        fn_src, used = emit_graph_fn(g, 'fw_step', R, C, out_exts, f'grp_allreduce<{L}>', self.invariant, self.colmask, self._lane_prolog())
        used_in = [i for i in range(nin) if p.in_names[i] in used]
        src, MT = self._row_kernel_common(R, W)
        body = []
        # staging buffers
        tail = plan.T % TS != 0
        stg = _Stager(TS, NT, tail)
        for i in sorted(set(used_in) | set(pro.inputs if pro else ())):
            if self.tdep[i]:
                self._stage_input(stg, A, i, MT)
        if pro:
            fn_src = pro.source() + '\n' + fn_src
            body.append(pro.decls())
        elif rfront:
            fn_src = self._stage_row_front(stg, A, rfront, set(used), MT, 'fw_rowpre') + '\n' + fn_src
        body.append(stg.decls() + stg.bases() + stg.zero_pads() + (pro.init() if pro else ''))
        # Results of a chunk (outputs, saved row sums) go to LDS per step and from there to memory.  With `df` they leave during
        # the next chunk, from the other half of a double buffer, and the checkpoint is stored after the staged operands were
        # written to LDS: a wave that waits for its prefetched loads also waits for every store it has issued, so stores
        # issued just before that wait put their latency into every chunk.  Measured: forward kernel and reverse scan of the
        # gated delta rule 3.60 / 3.43 -> 3.34 / 3.13 ms, Mamba-2's forward kernel 0.49 -> 0.46 ms; RWKV-7 0.81 / 0.73 -> 0.86 /
        # 0.82 ms (its stores then compete with the LDS reads of the steps), so both forms are timed candidates.
        df = bool(getattr(t, 'DF', 0))
        nb_ = 2 if df else 1
        kept = self._kept_sums(TS, False) if (nout or naux) else None
        kp = self.KEPT_PAD if kept else 0
        for k in range(nout):
            body.append(f'  __shared__ float s_out{k}[{nb_}][{TS}][{MT + kp}];\n')
        for k in range(naux):
            body.append(f'  __shared__ float s_aux{k}[{nb_}][{TS}][{MT + kp}];\n')
        # state
        for k in range(nst):
            rr, cc = _dims(st_ext[k], R, C)
            dt = DT_CODE[plan.st_dtypes[k]]
            nm = f'st{k}'
            ld = self._col_guard(f'ldf<{dt}>({A.p(nm)}, (i64)b * {A.s(nm, 0)} + (i64)h * {A.s(nm, 1)} + '
                                 f'(i64)ROWC(r) * {A.s(nm, 2)} + (i64)COLC(c) * {A.s(nm, 3)})')
            body.append(f'  float S{k}[{rr}][{cc}];\n#pragma unroll\n  for (int r = 0; r < {rr}; r++)\n'
                        f'#pragma unroll\n  for (int c = 0; c < {cc}; c++) S{k}[r][c] = {ld};\n')
        for i in used_in:
            if not self.tdep[i]:
                body.append(self._load_const_input(A, i, R, C))
        body.append(stg.load('0', '  '))
        body.append(f'  for (int t0 = 0; t0 < T; t0 += {TS}) {{\n')
        def checkpoint():
            out = [f'    if (t0 % {DT} == 0) {{\n']
            for k in range(nst if save else 0):
                rr, cc = _dims(st_ext[k], R, C)
                out.append(f'#pragma unroll\n      for (int r = 0; r < {rr}; r++) if (row0 + r < M) {{\n'
                           f'#pragma unroll\n        for (int c = 0; c < {cc}; c++) '
                           f'((float*){A.p(f"sck{k}")})[{self._ck_index(f"t0 / {DT}")}] = S{k}[r][c]; }}\n')
            out.append('    }\n')
            return out

        def flush(tbase, ntv, buf, ind):
            """The staged results of the chunk starting at `tbase` (`ntv` timesteps, LDS buffer `buf`) to memory."""
            out = [f'{ind}for (int e_ = tid; e_ < {TS * MT}; e_ += {NT}) {{ int tt_ = e_ / {MT}, x_ = e_ % {MT}; int m_ = mt * {MT} + x_;\n'
                   f'{ind}  if (m_ < M && tt_ < {ntv}) {{\n']
            for k in range(nout):
                dt = DT_CODE[plan.out_dtypes[k]]
                nm = f'out{k}'
                out.append(f'{ind}    stf<{dt}>({A.p(nm)}, (i64)b * {A.s(nm, 0)} + (i64)({tbase} + tt_) * {A.s(nm, 1)} + (i64)h * {A.s(nm, 2)} + (i64)m_ * {A.s(nm, 3)}, s_out{k}[{buf}][tt_][x_]);\n')
            for k in range(naux):
                out.append(f'{ind}    ((float*){A.p("aux")})[((((i64){k} * A.B + b) * H + h) * T + ({tbase} + tt_)) * M + m_] = s_aux{k}[{buf}][tt_][x_];\n')
            out.append(f'{ind}  }} }}\n')
            return out

        ck_late = df
        if not ck_late:
            body += checkpoint()
        body.append('    __syncthreads();\n')
        body.append(stg.write('    '))
        body.append('    __syncthreads();\n')
        if pro:
            body.append(pro.run('    '))
        body.append(f'    if (t0 + {TS} < T) {{\n' + stg.load(f't0 + {TS}', '      ') + '    }\n')
        if ck_late:
            body += checkpoint()
        if df:
            if nout or naux:        # the chunk before this one (always a whole one)
                body.append(f'    if (t0 > 0) {{\n')
                body += flush(f't0 - {TS}', str(TS), f'((t0 / {TS}) & 1) ^ 1', '      ')
                body.append('    }\n')
            body.append(f'    const int ob_ = (t0 / {TS}) & 1;\n')
        else:
            body.append('    const int ob_ = 0;\n')
        body.append(f'    const int nt = {f"min({TS}, T - t0)" if tail else TS};\n')
        # LDS operands of a step, in the order the step needs them (those its first row sum depends on first)
        operands = {}                       # graph input -> (register array, LDS array, extent)
        for nm_ in used:
            if nm_ in p.in_names and self.tdep[p.in_names.index(nm_)]:
                i = p.in_names.index(nm_)
                operands[nm_] = (f'x{i}', f's_in{i}', self.in_ext(i))
            elif nm_ in rfront:
                operands[nm_] = (f'd{rfront.index(nm_)}', f's_d{rfront.index(nm_)}', self.jext[nm_])
        order = self._operand_order(g, list(operands), skip=p.st_names)
        step = [self._load_operand(*operands[nm_], R, C, 'tt') for nm_ in order]
        call = []
        for nm_ in used:
            if nm_ in p.in_names:
                call.append(f'x{p.in_names.index(nm_)}')
            elif nm_ in p.st_names:
                call.append(f'S{p.st_names.index(nm_)}')
            elif nm_ in rfront:
                call.append(f'd{rfront.index(nm_)}')
            else:
                raise AssertionError(nm_)
        rrs = R if st_ext[0][0] else 1
        for k in range(nout):
            step.append(f'      float y{k}[{rrs}][1];\n')
            call.append(f'y{k}')
        for k in range(nst):
            rr, cc = _dims(st_ext[k], R, C)
            step.append(f'      float nS{k}[{rr}][{cc}];\n')
            call.append(f'nS{k}')
        for k in range(naux):
            step.append(f'      float a{k}[{rrs}][1];\n')
            call.append(f'a{k}')
        step.append('      fw_step(' + ', '.join(call) + ');\n')
        for k in range(nst):
            rr, cc = _dims(st_ext[k], R, C)
            step.append(f'#pragma unroll\n      for (int r = 0; r < {rr}; r++)\n#pragma unroll\n      for (int c = 0; c < {cc}; c++) S{k}[r][c] = nS{k}[r][c];\n')
        sums = [(f's_out{k}', f'y{k}') for k in range(nout)] + [(f's_aux{k}', f'a{k}') for k in range(naux)]
        ridx = 'r' if rrs > 1 else '0'
        unroll = f'#pragma unroll {max(1, getattr(t, "UR", 2))}\n'
        if kept:
            Lk, J = kept
            for _, v in sums:
                body.append(f'    float k_{v}[{J}][{R}] = {{}};\n')
            for j in range(J):
                cond = f'tl < {Lk}' + (f' && {j * Lk} + tl < nt' if tail else '')
                body.append(unroll + f'    for (int tl = 0; {cond}; tl++) {{ const int tt = {j * Lk} + tl;\n')
                body += step
                body.append('      { const bool mine_ = (l == tl);\n')
                for _, v in sums:
                    body.append(f'#pragma unroll\n        for (int r = 0; r < {R}; r++) k_{v}[{j}][r] = mine_ ? {v}[{ridx}][0] : k_{v}[{j}][r];\n')
                body.append('      }\n    }\n')
            body.append(f'    if (l < {Lk}) {{\n' if t.L > Lk else '    {\n')
            for j in range(J):
                for lds, v in sums:
                    body.append(f'#pragma unroll\n      for (int r = 0; r < {R}; r++) {lds}[ob_][{j * Lk} + l][rloc + r] = k_{v}[{j}][r];\n')
            body.append('    }\n')
        else:
            body.append(unroll + '    for (int tt = 0; tt < nt; tt++) {\n')
            body += step
            # every lane of a group holds the row sums after the all-reduce and stores them (same address, same value):
            # a store by one lane only would put a branch into every timestep and keep the compiler from overlapping
            # the next step's LDS reads and state-independent arithmetic with this step
            body.append('      {\n' if getattr(t, 'NB', 1) & 1 else '      if (l == 0) {\n')
            for lds, v in sums:
                body.append(f'#pragma unroll\n        for (int r = 0; r < {R}; r++) {lds}[ob_][tt][rloc + r] = {v}[{ridx}][0];\n')
            body.append('      }\n    }\n')
        if df:
            body.append('  }\n')
            if nout or naux:        # the last chunk (possibly a partial one)
                body.append(f'  if (T > 0) {{ const int tl_ = ((T - 1) / {TS}) * {TS};\n    __syncthreads();\n')
                body += flush('tl_', 'T - tl_', f'(tl_ / {TS}) & 1', '    ')
                body.append('  }\n')
        else:
            body.append('    __syncthreads();\n')
            body += flush('t0', 'nt', '0', '    ')
            body.append('  }\n')
        # final state
        for k in range(nst):
            rr, cc = _dims(st_ext[k], R, C)
            dt = DT_CODE[plan.st_dtypes[k]]
            nm = f'stT{k}'
            body.append(f'#pragma unroll\n  for (int r = 0; r < {rr}; r++) if (row0 + r < M) {{\n'
                        f'#pragma unroll\n    for (int c = 0; c < {cc}; c++) {self._col_if()}stf<{dt}>({A.p(nm)}, '
                        f'(i64)b * {A.s(nm, 0)} + (i64)h * {A.s(nm, 1)} + (i64)(row0 + r) * {A.s(nm, 2)} + (i64)COL(c) * {A.s(nm, 3)}, S{k}[r][c]); }}\n')
        kernel = (f'extern "C" __global__ void __launch_bounds__({NT}){self._row_attr()} {kname}(Args A) {{\n'
                  + ''.join(src) + ''.join(body) + '}\n')
        source = PRELUDE + A.struct() + self._row_macros() + fn_src + '\n' + kernel
        return KernelSpec(kname, source, list(A.names), NT, (f'(M + {MT - 1}) // {MT}', 'H', 'B'), {'kind': 'row', 'MT': MT})

    # ------------------------------------------------------------------ bw1
    def bw1(self) -> KernelSpec:
        p, plan, t = self.p, self.plan, self.tile
        L, C, G, DT = t.L, t.C, t.G, t.DT
        R, W = (t.R1 or t.R), (t.W1 or t.W)
        needs_state = p.dstep_needs_state
        TS = DT if needs_state else t.TS
        N = plan.N
        NT = W * 64
        A = _Args()
        nin, nst, nout = p.ninputs, p.nstates, p.noutputs
        naux, ndaux = len(p.aux), len(p.daux)
        st_ext = [self.jext[s] for s in p.st_names]
        colx = (st_ext[0][0], False)
        rrs = R if colx[0] else 1
        g = p.dstep
        mats = list(p.mat_idx) if p.mat_in_dstep else []
        out_exts = st_ext + [colx] * len(p.col_idx) + [colx] * ndaux + [(True, True)] * len(mats)
        restep_g = p.restep
        rfront = self._row_front([g, restep_g] if needs_state else [g])
        pro = None
        pfront = self._prologue_front([g, restep_g] if needs_state else [g])
        if sorted(rfront) != sorted(pfront):        # sums or scalars on the way: a pass of its own (as in the forward kernel)
            pro = _Prologue(self, pfront, 'bw', TS, NT, A)
            rfront = pro.front
        if rfront:
            g = g.extract('dstep', g.outputs, cut=rfront)
            restep_g = restep_g.extract('restep', restep_g.outputs, cut=rfront)
        fn_src, used = emit_graph_fn(g, 'bw_dstep', R, C, out_exts, f'grp_allreduce<{L}>', self.invariant, self.colmask, self._lane_prolog())
        fns = [fn_src]
        used_all = set(used)
        re_used = []
        if needs_state:
            re_src, re_used = emit_graph_fn(restep_g, 'bw_restep', R, C, st_ext, f'grp_allreduce<{L}>', self.invariant, self.colmask, self._lane_prolog())
            fns.append(re_src)
            used_all |= set(re_used)
        used_in = [i for i in range(nin) if p.in_names[i] in used_all]
        used_aux = [k for k in range(naux) if p.aux[k] in used_all]
        used_dout = [k for k in range(nout) if p.dout_names[k] in used_all]
        src, MT = self._row_kernel_common(R, W)
        body = []
        tail = plan.T % TS != 0
        stg = _Stager(TS, NT, tail)
        for i in sorted(set(used_in) | set(pro.inputs if pro else ())):
            if self.tdep[i]:
                self._stage_input(stg, A, i, MT)
        for k in used_aux:
            stg.add(f's_aux{k}', MT, 0, A.p('aux'),
                    lambda tt, x, k=k: f'((((i64){k} * A.B + b) * H + h) * T + {tt}) * M + min(mt * {MT} + {x}, M - 1)', 'M')
        for k in used_dout:
            nm = f'dout{k}'
            stg.add(f's_dy{k}', MT, DT_CODE[plan.out_dtypes[k]], A.p(nm),
                    lambda tt, x, nm=nm: (f'(i64)b * {A.s(nm, 0)} + (i64)({tt}) * {A.s(nm, 1)} + (i64)h * {A.s(nm, 2)} + '
                                           f'(i64)min(mt * {MT} + {x}, M - 1) * {A.s(nm, 3)}'), A.s(nm, 1))
        if pro:
            fns.insert(0, pro.source())
            body.append(pro.decls())
        elif rfront:
            fns.insert(0, self._stage_row_front(stg, A, rfront, used_all, MT, 'bw_rowpre'))
        body.append(stg.decls() + stg.bases() + stg.zero_pads() + (pro.init() if pro else ''))
        tdep_col = [i for i in p.col_idx if self.tdep[i]]
        const_col = [i for i in p.col_idx if not self.tdep[i]]
        # (as in the forward kernel: with `df` a chunk's column gradients and saved sums leave LDS during the next chunk,
        # and the d-state checkpoint is stored after the wait for the staged operands)
        df = bool(getattr(t, 'DF', 0))
        nb_ = 2 if df else 1
        kept = self._kept_sums(TS, True) if (tdep_col or ndaux) else None      # (as in the forward kernel)
        kp = self.KEPT_PAD if kept else 0
        for i in tdep_col:
            body.append(f'  __shared__ float s_dc{i}[{nb_}][{TS}][{MT + kp}];\n')
        for k in range(ndaux):
            body.append(f'  __shared__ float s_da{k}[{nb_}][{TS}][{MT + kp}];\n')
        # incoming cotangent of the final state
        for k in range(nst):
            rr, cc = _dims(st_ext[k], R, C)
            dt = DT_CODE[plan.st_dtypes[k]]
            nm = f'dstT{k}'
            ld = self._col_guard(f'ldf<{dt}>({A.p(nm)}, (i64)b * {A.s(nm, 0)} + (i64)h * {A.s(nm, 1)} + '
                                 f'(i64)ROWC(r) * {A.s(nm, 2)} + (i64)COLC(c) * {A.s(nm, 3)})')
            body.append(f'  float D{k}[{rr}][{cc}];\n#pragma unroll\n  for (int r = 0; r < {rr}; r++)\n'
                        f'#pragma unroll\n  for (int c = 0; c < {cc}; c++) D{k}[r][c] = {ld};\n')
        for i in used_in:
            if not self.tdep[i]:
                body.append(self._load_const_input(A, i, R, C))
        for i in const_col:
            body.append(f'  float gacc{i}[{rrs}][1];\n#pragma unroll\n  for (int r = 0; r < {rrs}; r++) gacc{i}[r][0] = 0.0f;\n')
        for i in mats:
            body.append(f'  float gmacc{i}[{R}][{C}];\n#pragma unroll\n  for (int r = 0; r < {R}; r++)\n#pragma unroll\n'
                        f'  for (int c = 0; c < {C}; c++) gmacc{i}[r][c] = 0.0f;\n')
        body.append(f'  const int tlast = ((T - 1) / {TS}) * {TS};\n')
        body.append(stg.load('tlast', '  '))

        def ckpt_fetch(k, chunk, indent):
            """The state checkpoint of `chunk` into the registers pS<k>: issued one chunk ahead, like the
            staged operands, so that no chunk starts by waiting for HBM."""
            rr, cc = _dims(st_ext[k], R, C)
            return (f'#pragma unroll\n{indent}for (int r = 0; r < {rr}; r++)\n#pragma unroll\n{indent}for (int c = 0; c < {cc}; c++) '
                    f'pS{k}[r][c] = ((const float*){A.p(f"sck{k}")})[(((i64)(b * H + h) * nch + ({chunk})) * M + ROWC(r)) * {self.NP} + COL(c)];\n')

        for k in range(nst if needs_state else 0):
            rr, cc = _dims(st_ext[k], R, C)
            body.append(f'  float pS{k}[{rr}][{cc}];\n' + ckpt_fetch(k, f'tlast / {DT}', '  '))
        body.append(f'  for (int t0 = tlast; t0 >= 0; t0 -= {TS}) {{\n')
        body.append(f'    const int nt = {f"min({TS}, T - t0)" if tail else TS};\n')
        def d_checkpoint():
            # d_state checkpoints are only read by the gradient kernel
            out = [f'    if ((t0 + {TS}) % {DT} == 0{f" || t0 + {TS} >= T" if self.tail_dt else ""}) {{\n']
            for k in range(nst if needs_gradient_kernel(p) else 0):
                rr, cc = _dims(st_ext[k], R, C)
                out.append(f'#pragma unroll\n      for (int r = 0; r < {rr}; r++) if (row0 + r < M) {{\n'
                           f'#pragma unroll\n        for (int c = 0; c < {cc}; c++) '
                           f'((float*){A.p(f"dck{k}")})[{self._ck_index(f"t0 / {DT}")}] = D{k}[r][c]; }}\n')
            out.append('    }\n')
            return out

        def flush(tbase, ntv, buf, ind):
            """Column gradients and saved sums of the chunk starting at `tbase` (`ntv` timesteps, LDS buffer `buf`) to memory."""
            if not (tdep_col or ndaux):
                return []
            out = [f'{ind}for (int e_ = tid; e_ < {TS * MT}; e_ += {NT}) {{ int tt_ = e_ / {MT}, x_ = e_ % {MT}; int m_ = mt * {MT} + x_;\n'
                   f'{ind}  if (m_ < M && tt_ < {ntv}) {{\n']
            for i in tdep_col:
                nm = f'din{i}'
                idx = f'(i64)b * {A.s(nm, 0)} + (i64)({tbase} + tt_) * {A.s(nm, 1)} + (i64)h * {A.s(nm, 2)} + (i64)m_ * {A.s(nm, 3)}'
                if i in self.atomic:
                    out.append(f'{ind}    atomic_addf({A.p(nm)}, {idx}, s_dc{i}[{buf}][tt_][x_]);\n')
                else:
                    dt = DT_CODE[plan.in_dtypes[i]]
                    out.append(f'{ind}    stf<{dt}>({A.p(nm)}, {idx}, s_dc{i}[{buf}][tt_][x_]);\n')
            for k in range(ndaux):
                out.append(f'{ind}    ((float*){A.p("daux")})[((((i64){k} * A.B + b) * H + h) * T + ({tbase} + tt_)) * M + m_] = s_da{k}[{buf}][tt_][x_];\n')
            out.append(f'{ind}  }} }}\n')
            return out

        ck_late = df
        if not ck_late:
            body += d_checkpoint()
        body.append('    __syncthreads();\n')
        body.append(stg.write('    '))
        body.append('    __syncthreads();\n')
        if pro:
            body.append(pro.run('    '))
        for k in range(nst if needs_state else 0):
            rr, cc = _dims(st_ext[k], R, C)
            body.append(f'    float Sh{k}_0[{rr}][{cc}];\n#pragma unroll\n    for (int r = 0; r < {rr}; r++)\n'
                        f'#pragma unroll\n    for (int c = 0; c < {cc}; c++) Sh{k}_0[r][c] = pS{k}[r][c];\n')
        body.append(f'    if (t0 >= {TS}) {{\n' + stg.load(f't0 - {TS}', '      ')
                    + ''.join(ckpt_fetch(k, f't0 / {DT} - 1', '      ') for k in range(nst if needs_state else 0)) + '    }\n')
        if ck_late:
            body += d_checkpoint()
        if df:
            pre = flush(f't0 + {TS}', f'min({TS}, T - (t0 + {TS}))' if tail else str(TS), f'((t0 / {TS}) & 1) ^ 1', '      ')
            if pre:                 # the chunk walked before this one (the later timesteps; only that one can be partial)
                body.append('    if (t0 < tlast) {\n')
                body += pre
                body.append('    }\n')
            body.append(f'    const int ob_ = (t0 / {TS}) & 1;\n')
        else:
            body.append('    const int ob_ = 0;\n')

        # With state recompute a timestep's operands are read by `bw_restep` and again by
        # `bw_dstep`.  Those without a column extent (one register per row) are loaded once for
        # both, so that the compiler sees common subexpressions of the two calls - typically
        # the exponential of a per-row decay - as such.
        shared_in = [i for i in used_in if needs_state and getattr(t, 'SH', 1) and self.tdep[i] and not self.in_ext(i)[1]
                     and p.in_names[i] in used and p.in_names[i] in re_used]

        def operand_loads(tt, names, state_var, order=None):
            """Loads of the LDS operands among `names` for timestep `tt` and the argument list.  With `order` the
            loads come in that order."""
            code, call, loads = [], [], {}
            for nm_ in names:
                if nm_ in p.in_names:
                    i = p.in_names.index(nm_)
                    if i in shared_in:
                        call.append(f'x{i}_{tt}')
                    elif self.tdep[i]:
                        v = f'x{i}_{tt}' if needs_state else f'x{i}'
                        loads[nm_] = (v, f's_in{i}', self.in_ext(i))
                        call.append(v)
                    else:
                        call.append(f'x{i}')
                elif nm_ in p.st_names:
                    call.append(state_var(p.st_names.index(nm_)))
                elif nm_ in p.aux:
                    k = p.aux.index(nm_)
                    e = self.jext[nm_]
                    v = f'ax{k}_{tt}' if needs_state else f'ax{k}'
                    loads[nm_] = (v, f's_aux{k}', (e[0], False))
                    call.append(v)
                elif nm_ in p.dout_names:
                    k = p.dout_names.index(nm_)
                    v = f'dy{k}_{tt}' if needs_state else f'dy{k}'
                    loads[nm_] = (v, f's_dy{k}', colx)
                    call.append(v)
                elif nm_ in p.dnst_names:
                    call.append(f'D{p.dnst_names.index(nm_)}')
                elif nm_ in rfront:
                    q = rfront.index(nm_)
                    v = f'd{q}_{tt}' if needs_state else f'd{q}'
                    loads[nm_] = (v, f's_d{q}', self.jext[nm_])
                    call.append(v)
                else:
                    raise AssertionError(nm_)
            for nm_ in (order if order is not None else list(loads)):
                if nm_ in loads:
                    code.append(self._load_operand(*loads[nm_], R, C, tt))
            return code, call, loads

        sums = [(f's_dc{i}', f'gc{i}') for i in tdep_col] + [(f's_da{k}', f'da{k}') for k in range(ndaux)]

        def dstep_block(tt, state_var, indent='      ', order=None, keep=None):
            """One timestep of the scan.  `keep` = (j, tl): the step is number tl of the j-th group of kept row sums."""
            code, call, _ = operand_loads(tt, used, state_var, order)
            for k in range(nst):
                rr, cc = _dims(st_ext[k], R, C)
                code.append(f'{indent}float nD{k}[{rr}][{cc}];\n')
                call.append(f'nD{k}')
            for i in p.col_idx:
                code.append(f'{indent}float gc{i}[{rrs}][1];\n')
                call.append(f'gc{i}')
            for k in range(ndaux):
                code.append(f'{indent}float da{k}[{rrs}][1];\n')
                call.append(f'da{k}')
            for i in mats:
                code.append(f'{indent}float gm{i}[{R}][{C}];\n')
                call.append(f'gm{i}')
            code.append(f'{indent}bw_dstep(' + ', '.join(call) + ');\n')
            for i in mats:
                code.append(f'#pragma unroll\n{indent}for (int r = 0; r < {R}; r++)\n#pragma unroll\n{indent}for (int c = 0; c < {C}; c++) gmacc{i}[r][c] += gm{i}[r][c];\n')
            for k in range(nst):
                rr, cc = _dims(st_ext[k], R, C)
                code.append(f'#pragma unroll\n{indent}for (int r = 0; r < {rr}; r++)\n#pragma unroll\n{indent}for (int c = 0; c < {cc}; c++) D{k}[r][c] = nD{k}[r][c];\n')
            for i in const_col:
                code.append(f'#pragma unroll\n{indent}for (int r = 0; r < {rrs}; r++) gacc{i}[r][0] += gc{i}[r][0];\n')
            ridx = 'r' if rrs > 1 else '0'
            if keep is not None:
                j, tl = keep
                code.append(f'{indent}{{ const bool mine_ = (l == {tl});\n')
                for _, v in sums:
                    code.append(f'#pragma unroll\n{indent}  for (int r = 0; r < {R}; r++) k_{v}[{j}][r] = mine_ ? {v}[{ridx}][0] : k_{v}[{j}][r];\n')
                code.append(f'{indent}}}\n')
                return code
            # (as in the forward kernel: with bit 1 of NB all lanes of a group store the same sums, no branch inside the time loop)
            code.append(f'{indent}{{\n' if getattr(t, 'NB', 1) & 2 else f'{indent}if (l == 0) {{\n')
            for lds, v in sums:
                code.append(f'#pragma unroll\n{indent}  for (int r = 0; r < {R}; r++) {lds}[ob_][{tt}][rloc + r] = {v}[{ridx}][0];\n')
            code.append(f'{indent}}}\n')
            return code

        def kept_store():
            Lk, J = kept
            code = [f'    if (l < {Lk}) {{\n' if t.L > Lk else '    {\n']
            for j in range(J):
                for lds, v in sums:
                    code.append(f'#pragma unroll\n      for (int r = 0; r < {R}; r++) {lds}[ob_][{j * Lk} + l][rloc + r] = k_{v}[{j}][r];\n')
            return code + ['    }\n']

        if kept:
            for _, v in sums:
                body.append(f'    float k_{v}[{kept[1]}][{R}] = {{}};\n')

        if not needs_state:
            # operands in the order the step needs them
            no_state = lambda k: (_ for _ in ()).throw(AssertionError())
            _, _, loads = operand_loads('tt', used, no_state)
            order = self._operand_order(g, list(loads), skip=p.dnst_names)
            unroll = f'#pragma unroll {max(1, getattr(t, "UR", 2))}\n'
            if kept:
                Lk, J = kept
                for j in range(J - 1, -1, -1):
                    first = f'min({Lk}, nt - {j * Lk})' if tail else str(Lk)
                    body.append(unroll + f'    for (int tl = {first} - 1; tl >= 0; tl--) {{ const int tt = {j * Lk} + tl;\n')
                    body += dstep_block('tt', no_state, order=order, keep=(j, 'tl'))
                    body.append('    }\n')
                body += kept_store()
            else:
                body.append(unroll + '    for (int tt = nt - 1; tt >= 0; tt--) {\n')
                body += dstep_block('tt', no_state, order=order)
                body.append('    }\n')
        else:
            # recompute the DT states of this chunk from its checkpoint, then walk back
            for tt in range(1, DT):
                for k in range(nst):
                    rr, cc = _dims(st_ext[k], R, C)
                    body.append(f'    float Sh{k}_{tt}[{rr}][{cc}];\n')
            for tt in range(DT):
                for i in shared_in:
                    body.append(self._load_operand(f'x{i}_{tt}', f's_in{i}', self.in_ext(i), R, C, str(tt)))
            for tt in range(DT - 1):
                body.append(f'    if ({tt + 1} < nt) {{\n' if tail else '    {\n')
                code, call, _ = operand_loads(str(tt), re_used, lambda k, tt=tt: f'Sh{k}_{tt}')
                body += code
                for k in range(nst):
                    call.append(f'Sh{k}_{tt + 1}')
                body.append('      bw_restep(' + ', '.join(call) + ');\n    }\n')
            for tt in range(DT - 1, -1, -1):
                body.append(f'    if ({tt} < nt) {{\n' if tail else '    {\n')
                body += dstep_block(str(tt), lambda k, tt=tt: f'Sh{k}_{tt}', keep=(tt // kept[0], tt % kept[0]) if kept else None)
                body.append('    }\n')
            if kept:
                body += kept_store()
        if df:
            body.append('  }\n')
            last = flush('0', f'min({TS}, T)' if tail else str(TS), '0', '    ')
            if last:                # the chunk walked last: timesteps 0 .. TS-1
                body.append('  if (T > 0) {\n    __syncthreads();\n')
                body += last
                body.append('  }\n')
        else:
            body.append('    __syncthreads();\n')
            body += flush('t0', 'nt', '0', '    ')
            body.append('  }\n')
        for i in const_col:
            nm = f'din{i}'
            body.append(f'  if (l == 0) {{\n#pragma unroll\n    for (int r = 0; r < {R}; r++) if (row0 + r < M) '
                        f'atomic_addf({A.p(nm)}, (i64)b * {A.s(nm, 0)} + (i64)h * {A.s(nm, 2)} + (i64)(row0 + r) * {A.s(nm, 3)}, gacc{i}[{"r" if rrs > 1 else "0"}][0]);\n  }}\n')
        for i in mats:
            nm = f'din{i}'
            bB, _, bH = plan.in_bcast[i]
            idx = (f'(i64)b * {A.s(nm, 0)} + (i64)h * {A.s(nm, 2)} + (i64)(row0 + r) * {A.s(nm, 3)} + (i64)COL(c) * {A.s(nm, 4)}')
            put = (f'atomic_addf({A.p(nm)}, {idx}, gmacc{i}[r][c])' if (bB or bH)
                   else f'stf<0>({A.p(nm)}, {idx}, gmacc{i}[r][c])')
            body.append(f'#pragma unroll\n  for (int r = 0; r < {R}; r++) if (row0 + r < M) {{\n#pragma unroll\n'
                        f'    for (int c = 0; c < {C}; c++) {self._col_if()}{put}; }}\n')
        for k in range(nst):
            rr, cc = _dims(st_ext[k], R, C)
            dt = DT_CODE[plan.st_dtypes[k]]
            nm = f'dst{k}'
            body.append(f'#pragma unroll\n  for (int r = 0; r < {rr}; r++) if (row0 + r < M) {{\n'
                        f'#pragma unroll\n    for (int c = 0; c < {cc}; c++) {self._col_if()}stf<{dt}>({A.p(nm)}, '
                        f'(i64)b * {A.s(nm, 0)} + (i64)h * {A.s(nm, 1)} + (i64)(row0 + r) * {A.s(nm, 2)} + (i64)COL(c) * {A.s(nm, 3)}, D{k}[r][c]); }}\n')
        kernel = (f'extern "C" __global__ void __launch_bounds__({NT}){self._row_attr()} frnn_bw1(Args A) {{\n'
                  + ''.join(src) + ''.join(body) + '}\n')
        source = PRELUDE + A.struct() + self._row_macros() + '\n'.join(fns) + '\n' + kernel
        return KernelSpec('frnn_bw1', source, list(A.names), NT, (f'(M + {MT - 1}) // {MT}', 'H', 'B'), {'kind': 'row', 'MT': MT})

    # ------------------------------------------------------------------ bw2
    def bw2(self, waves_per_simd: int = 0, prefetch: int = 4, reread_scalars: bool = False) -> KernelSpec:
        """`waves_per_simd` > 0 asks the compiler to fit that many waves on a SIMD (fewer registers,
        possibly spills); the caller compares the outcomes.  `reread_scalars`: per-timestep scalar inputs that the
        preparation and the epilogue read but the row loop does not are read twice instead of kept (DT registers
        each; worth it only where that lifts the occupancy: Mamba-2 at 128 rows 178 -> 162 registers and
        1.13 -> 0.97 ms, the gated delta rule 252 -> 236 and 2 % slower)."""
        p, plan, t = self.p, self.plan, self.tile
        N, DT = plan.NP, t.DT              # lanes cover the padded width; `nok` marks real columns
        IPB = max(1, 64 // N)
        NT = max(64, N)
        nok = 'nok' if self.pad else ''
        nok_prolog = f'const bool nok = (int)(threadIdx.x % {N}) < {plan.N};' if self.pad else ''
        HB = max(1, getattr(t, 'HB', 1))
        MS = max(1, getattr(t, 'MS', 1))
        MR = -(-plan.M // MS)               # rows per instance
        PD = max(1, prefetch)               # checkpoint rows in flight ahead of the row loop
        assert plan.H % HB == 0
        A = _Args()
        nin, nst, nout = p.ninputs, p.nstates, p.noutputs
        naux, ndaux = len(p.aux), len(p.daux)
        st_ext = [self.jext[s] for s in p.st_names]
        nm_ = p.joint.node_map()
        rs = p.row_idx + p.scalar_idx
        red = f'inst_allreduce<{N}>'
        op_names = [nm_[m].args[0] for m in p.msums]
        mats2 = [] if p.mat_in_dstep else list(p.mat_idx)
        # Per-row scalars.  A value with a row extent but no column extent is the same on every
        # lane of an instance; the row loop would recompute it on each of them for every
        # (row, timestep).  The outermost such values (`front`: those feeding a full-tile value or
        # a row sum) are instead evaluated where the chunk's per-row operands are staged, one
        # (row, timestep) per lane, and reach the row loop through LDS like a raw operand.  A row
        # sum of such a value (`colsum`) never enters the row loop: it is summed from LDS.
        front = []
        # (a vector state, N == 1, has no column extent itself: nothing to tell apart there)
        for g_ in ((p.restep, p.drow) if all(e[1] for e in st_ext) else ()):
            for n_ in g_.nodes:
                if n_.ext == (True, False) and n_.name not in front and (
                        n_.name in g_.outputs or any(n_.name in m_.value_args() and m_.ext[1] for m_ in g_.nodes)):
                    front.append(n_.name)
        colsum = [j for j, o in enumerate(op_names) if o in front]
        loop_ops = [j for j in range(len(op_names)) if j not in colsum]
        # Row-invariant values (no row extent: functions of the row / scalar inputs of a timestep,
        # e.g. the exponential of a log-decay) are the same for every row of the chunk.  The
        # outermost ones (`rfront`) are evaluated once per chunk, before the row loop, which then
        # takes them like inputs; the epilogue reuses them.
        rfront = []
        for g_ in (p.restep, p.drow):
            for n_ in g_.nodes:
                if not n_.ext[0] and n_.op != 'const' and n_.name not in rfront and \
                        any(n_.name in m_.value_args() and m_.ext[0] for m_ in g_.nodes):
                    rfront.append(n_.name)
        cut_all = front + rfront
        restep_g = p.restep.extract('restep', p.restep.outputs, cut=cut_all) if cut_all else p.restep
        drow_outs = list(p.drow.outputs[:nst + len(mats2)]) + [op_names[j] for j in loop_ops]
        drow_g = p.drow.extract('drow', drow_outs, cut=cut_all) if cut_all else p.drow
        drow_exts = st_ext + [(True, True)] * len(mats2) + [self.jext[op_names[j]] for j in loop_ops]
        drow_src, drow_used = emit_graph_fn(drow_g, 'bw_drow', 1, 1, drow_exts, red, self.invariant)
        re_src, re_used = emit_graph_fn(restep_g, 'bw_restep', 1, 1, st_ext, red, self.invariant)
        epi_exts = [self.in_ext(i) for i in rs]
        epi_nodes = {n_.name for n_ in p.epi.nodes}
        epi_g = p.epi.extract('epi', p.epi.outputs, cut=[f for f in rfront if f in epi_nodes]) if rfront else p.epi
        epi_src, epi_used = emit_graph_fn(epi_g, 'bw_epi', 1, 1, epi_exts, red, (), nok, nok_prolog)
        # With more than one wave per instance every sum over the columns costs two barriers; sums inside the
        # preparation and inside the epilogue (the norm of a key a traced layer normalises, and its gradient) are
        # then formed level by level for all timesteps of the chunk at once: one exchange per level.
        epi_lev = self._levelled(epi_g, 'bw_epi', epi_exts, nok, nok_prolog) if N > 64 else None
        if epi_lev:
            epi_src, epi_used = '\n'.join(epi_lev['src']), epi_lev['used']
        loop_used = set(drow_used) | set(re_used)
        pre_src, pre_used = '', []
        cuts = [i for g_ in (p.restep, p.drow) for i in g_.inputs if i not in p.joint.input_ext]
        if front:
            # (a per-row scalar may read a value computed once per chunk - a sum over a row input, say; such values are
            # inputs here and reach the staging loop, which picks the timestep at run time, through a small LDS table)
            pre_g = p.joint.extract('colpre', front, cut=set(cuts) | set(rfront))
            pre_src, pre_used = emit_graph_fn(pre_g, 'bw_colpre', 1, 1, [(True, False)] * len(front), red, self.invariant)
            assert all(self.jext[v] == (False, False) for v in pre_used if v in rfront), 'a per-row scalar cannot read a per-column value'
        g_tables = [q for q, f in enumerate(rfront) if f in pre_used]
        rpre_used = []
        if rfront:
            rpre_g = p.joint.extract('rowpre', rfront, cut=set(cuts))
            rpre_src, rpre_used = emit_graph_fn(rpre_g, 'bw_rowpre', 1, 1, [self.jext[f] for f in rfront], red, self.invariant, nok, nok_prolog)
            rpre_lev = self._levelled(rpre_g, 'bw_rowpre', [self.jext[f] for f in rfront], nok, nok_prolog) if N > 64 else None
            if rpre_lev:
                rpre_src, rpre_used = '\n'.join(rpre_lev['src']), rpre_lev['used']
            pre_src += '\n' + rpre_src
        else:
            rpre_lev = None
        all_used = loop_used | set(epi_used) | set(rpre_used)

        def is_rowlike(nm):      # no row extent: can be loaded once per chunk
            return not self.jext[nm][0]

        helper = f'''
template <int N_> __device__ __forceinline__ float inst_allreduce(float x) {{
  if constexpr (N_ <= 64) {{ return grp_allreduce<N_>(x); }}
  else {{
    __shared__ float red_[N_ / 64];
    x = grp_allreduce<64>(x);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red_[threadIdx.x >> 6] = x;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < N_ / 64; w++) s += red_[w];
    return s;
  }}
}}
'''
        helper += '''
// x summed over the 64 / N_ instances of a wave (lanes N_ apart); every lane gets the total
template <int N_> __device__ __forceinline__ float inst_total(float x) {
  if constexpr (N_ <= 16) x = xor16_sum(x);
  if constexpr (N_ <= 32) x = xor32_sum(x);
  return x;
}
'''
        b = []
        # Narrow states pack IPB = 64 / N instances into a wave.  With split rows they are IPB consecutive row slices
        # of one chunk (`share`): the wave then reads whole 128-byte lines of every per-row operand (a slice of 16 fp32
        # rows is half a line; with the instances on different chunks every line was fetched twice), and the slices'
        # row / scalar gradients - which meet in the same addresses - are summed across the wave's instances with
        # lane swaps before one instance adds them to memory.  Otherwise the instances of a wave are IPB chunks.
        share = IPB > 1 and MS > 1 and MS % IPB == 0 and N in (16, 32) and HB == 1
        if MS == 1:
            rows_decl = '  const int mlo = 0, mhi = M;'
        elif share:
            rows_decl = (f'  const int mlo = (blockIdx.z * {IPB} + inst) * {MR}, mhi = min(M, mlo + {MR});   // rows of this instance\n'
                         '  valid = valid && mlo < M;               // (a slice beyond the last row walks no rows and adds nothing)')
        else:
            rows_decl = (f'  const int mlo = blockIdx.z * {MR}, mhi = min(M, mlo + {MR});   // rows of this instance\n'
                         '  if (mlo >= M) return;')
        cpb = 1 if share else IPB           # chunks per workgroup
        # grid y is limited to 65535 blocks: with more (batch, head group) pairs than that, both indices
        # travel in x, in the same order of dispatch
        fold = plan.B * (plan.H // HB) > MAX_GRID_Y
        block_decl = (f'  const int gx_ = (nch + {cpb - 1}) / {cpb};\n  const int bx_ = blockIdx.x % gx_, by_ = blockIdx.x / gx_;\n'
                      if fold else '')
        bx, by = ('bx_', 'by_') if fold else ('blockIdx.x', 'blockIdx.y')
        b.append(f'''  const int tid = threadIdx.x;
  const int n = tid % {N};
  const bool nok = n < {plan.N}; const int nc = min(n, {plan.N - 1});     // real column? / column clamped for addresses
  (void)nok; (void)nc;
  const int inst = {"tid / " + str(N) if IPB > 1 else "0"};
  const int T = (int)A.T, H = (int)A.H, M = (int)A.M, nch = (int)A.nch;
  (void)T;
{block_decl}  int ch = {f"{bx}" if share else f"{bx} * {IPB} + inst"};
  bool valid = ch < nch;
  if (!valid) ch = nch - 1;
  const int HG = H / {HB};                     // head groups; an instance walks {HB} heads
  const int b = {by} / HG, h0 = ({by} % HG) * {HB};
  const int t0 = ch * {DT};
{rows_decl}
  const int nt = {f"min({DT}, T - t0)" if self.tail_dt else DT};          // timesteps of this chunk
  (void)nt;
''')
        tail = self.tail_dt

        def tclamp(tt):
            return f'min(t0 + {tt}, T - 1)' if tail else f't0 + {tt}'

        # gradients of inputs broadcast over heads / time are summed in registers across the
        # head loop / the chunk before they leave the kernel
        def bflags(i):
            return plan.in_bcast[i]
        hacc = [i for i in rs if bflags(i)[2] and HB > 1]
        for i in hacc:
            if bflags(i)[1]:
                b.append(f'  float gh{i} = 0.0f;\n')
            else:
                for tt in range(DT):
                    b.append(f'  float gh{i}_{tt} = 0.0f;\n')
        b.append(f'  for (int hh = 0; hh < {HB}; hh++) {{\n  const int h = h0 + hh; const int bh = b * H + h;\n')

        def load_in(i, tt, m=None, col='nc'):
            ext = self.in_ext(i)
            dt = DT_CODE[plan.in_dtypes[i]]
            idx = self._in_index(A, i, t=(tclamp(tt) if self.tdep[i] else '0'),
                                 m=('m' if ext[0] else None), n=(col if ext[1] else None))
            ld = f'ldf<{dt}>({A.p(f"in{i}")}, {idx})'
            return f'(nok ? {ld} : 0.0f)' if (self.pad and ext[1]) else ld

        def var_in(i, tt):
            return f'x{i}_{tt}' if self.tdep[i] else f'x{i}'

        def aux_load(k, tt, mexpr):
            return f'((const float*){A.p("aux")})[((((i64){k} * A.B + b) * H + h) * T + ({tclamp(tt)})) * M + {mexpr}]'

        def raw_value(v, tt, mexpr):
            """Global-memory value of graph input `v` (an input, saved sum or output gradient without
            a column extent) at timestep offset `tt` of the chunk and row `mexpr`."""
            if v in rfront:
                return f's_g{rfront.index(v)}[inst][{tt}]'
            if v in p.in_names:
                i = p.in_names.index(v)
                ext = self.in_ext(i)
                assert not ext[1], v
                dt = DT_CODE[plan.in_dtypes[i]]
                idx = self._in_index(A, i, t=(tclamp(tt) if self.tdep[i] else '0'), m=(mexpr if ext[0] else None))
                return f'ldf<{dt}>({A.p(f"in{i}")}, {idx})'
            if v in p.aux:
                return aux_load(p.aux.index(v), tt, mexpr if self.jext[v][0] else '0')
            if v in p.daux:
                return f'((const float*){A.p("daux")})[((((i64){p.daux.index(v)} * A.B + b) * H + h) * T + ({tclamp(tt)})) * M + {mexpr}]'
            if v in p.dout_names:
                k = p.dout_names.index(v)
                dt = DT_CODE[plan.out_dtypes[k]]
                nmv = f'dout{k}'
                return (f'ldf<{dt}>({A.p(nmv)}, (i64)b * {A.s(nmv, 0)} + (i64)({tclamp(tt)}) * {A.s(nmv, 1)} + '
                        f'(i64)h * {A.s(nmv, 2)} + (i64)({mexpr}) * {A.s(nmv, 3)})')
            raise AssertionError(v)

        # ---- per-chunk loads of everything without a row extent.  Inputs that only the preparation before the row loop and
        # the epilogue read (the raw projections behind a preparation that a traced layer moved into the step) would
        # occupy registers across the row loop, which decides the kernel's occupancy: when there are more than 32 such
        # registers they are loaded in a block of their own for the preparation and again after the row loop (`late`).
        # Fewer stay where they are: the second load's latency is not hidden (Mamba-2: 1.06 -> 1.13 ms when tried).
        def chunk_loads(names, col='nc'):
            out = []
            for i in range(nin):
                if p.in_names[i] not in names or self.in_ext(i)[0]:
                    continue
                if self.tdep[i]:
                    for tt in range(DT):
                        out.append(f'  float x{i}_{tt}[1][1]; x{i}_{tt}[0][0] = {load_in(i, tt, col=col)};\n')
                else:
                    out.append(f'  float x{i}[1][1]; x{i}[0][0] = {load_in(i, 0, col=col)};\n')
            for k in range(naux):
                if p.aux[k] in names and is_rowlike(p.aux[k]):
                    for tt in range(DT):
                        out.append(f'  float ax{k}_{tt}[1][1]; ax{k}_{tt}[0][0] = {aux_load(k, tt, "0")};\n')
            return out

        prep_only = all_used - loop_used
        if DT * sum(1 for i in range(nin) if p.in_names[i] in prep_only and not self.in_ext(i)[0] and self.tdep[i]) >= 32:
            late_in = set(prep_only)
        elif reread_scalars:
            late_in = {v for v in set(rpre_used) & set(epi_used) - loop_used if v in p.in_names
                       and self.in_ext(p.in_names.index(v)) == (False, False) and self.tdep[p.in_names.index(v)]}
        else:
            late_in = set()
        late = bool(late_in)
        b += chunk_loads(all_used - late_in if late else all_used)
        for j in loop_ops:
            for tt in range(DT):
                b.append(f'  float acc{j}_{tt} = 0.0f;\n')
        n_uniform = sum(1 for f in rfront if self.jext[f] == (False, False))
        NW = max(1, N // 64)

        def exchange(tag, vals):
            """Sums of the per-lane values `vals` (expressions) over the instance's lanes, all in one exchange through
            LDS between two barriers; returns the names of the totals."""
            b.append(f'  __shared__ float red_{tag}[{len(vals)}][{NW}];\n')
            for k, v in enumerate(vals):
                b.append(f'  float {tag}p{k} = grp_allreduce<64>({f"nok ? {v} : 0.0f" if self.pad else v});\n')
            b.append('  __syncthreads();\n  if ((tid & 63) == 0) { ' + ' '.join(f'red_{tag}[{k}][tid >> 6] = {tag}p{k};' for k in range(len(vals)))
                     + ' }\n  __syncthreads();\n')
            for k in range(len(vals)):
                b.append(f'  float {tag}t{k}[1][1]; {tag}t{k}[0][0] = ' + ' + '.join(f'red_{tag}[{k}][{w}]' for w in range(NW)) + ';\n')
            return [f'{tag}t{k}' for k in range(len(vals))]

        fresh = [0]

        def total_of(tot, v, tt, ind='  '):
            """A new variable holding the total of sum `v` at timestep `tt`, read from where `levelled` left it."""
            fresh[0] += 1
            name = f'lt{fresh[0]}'
            b.append(f'{ind}float {name}[1][1]; {name}[0][0] = {tot[(v, tt)]};\n')
            return name

        def levelled(lev, tag, arg_of):
            """Evaluates the levels of `lev` for every timestep of the chunk; returns {(sum name, timestep): expression
            of the total}.  A level's totals stay in LDS and are read where they are used (`total_of`), and a
            wave's partial sums go there as they are formed: neither holds DT registers per sum."""
            tot = {}
            for li, (fn, used, mine) in enumerate(lev['levels']):
                red_ = f'red_{tag}{li}'
                b.append(f'  __shared__ float {red_}[{DT * len(mine)}][{NW}];\n  __syncthreads();\n')
                for tt in range(DT):
                    outs = [f'{tag}o{li}_{k}' for k in range(len(mine))]
                    b.append('  { ' + ' '.join(f'float {o}[1][1];' for o in outs) + '\n')
                    args = [total_of(tot, v, tt, '    ') if (v, tt) in tot else arg_of(v, tt) for v in used]
                    b.append(f'    {fn}(' + ', '.join(args + outs) + ');\n')
                    for k, o in enumerate(outs):
                        v = f'{o}[0][0]'
                        b.append(f'    {{ const float p_ = grp_allreduce<64>({f"nok ? {v} : 0.0f" if self.pad else v}); '
                                 f'if ((tid & 63) == 0) {red_}[{tt * len(mine) + k}][tid >> 6] = p_; }}\n')
                    b.append('  }\n')
                b.append('  __syncthreads();\n')
                for tt in range(DT):
                    for k, c in enumerate(mine):
                        tot[(c, tt)] = '(' + ' + '.join(f'{red_}[{tt * len(mine) + k}][{w}]' for w in range(NW)) + ')'
            return tot

        def rpre_arg(v, tt):
            if v in p.in_names:
                return var_in(p.in_names.index(v), tt)
            assert v in p.aux and is_rowlike(v), v
            return f'ax{p.aux.index(v)}_{tt}'

        def uniform(tt):
            # With one instance per wave a value without row and column extent is the same on all lanes;
            # kept in a scalar register it costs no vector register for the length of the chunk (Mamba-2's
            # per-step decay: 184 -> 150 registers, three waves per SIMD without spills).  The scalar
            # inputs themselves stay in vector registers: as scalar operands of the row loop's
            # multiply-adds they cost moves (gated delta rule: 7 % slower).
            return [f'  g{q}_{tt}[0][0] = wave_uniform(g{q}_{tt}[0][0]);\n' for q, f in enumerate(rfront)
                    if IPB == 1 and self.jext[f] == (False, False) and n_uniform * DT <= 32]      # (more would spill scalar registers)

        if rfront and late:
            for tt in range(DT):
                b.append('  ' + ' '.join(f'float g{q}_{tt}[1][1];' for q in range(len(rfront))) + '\n')
            b.append('  {\n')
            b += chunk_loads(set(rpre_used) & late_in)
        if rfront and rpre_lev:
            tot = levelled(rpre_lev, 'rp', rpre_arg)
            fn, used = rpre_lev['final']
            for tt in range(DT):
                outs = [f'g{q}_{tt}' for q in range(len(rfront))]
                args = [total_of(tot, v, tt) if (v, tt) in tot else rpre_arg(v, tt) for v in used]
                b.append('  ' + ('' if late else ' '.join(f'float {o}[1][1];' for o in outs)) + f' {fn}(' + ', '.join(args + outs) + ');\n')
                b += uniform(tt)
        if rfront and not rpre_lev:
            for tt in range(DT):
                call = [rpre_arg(v, tt) for v in rpre_used]
                for q in range(len(rfront)):
                    if not late:
                        b.append(f'  float g{q}_{tt}[1][1];\n')
                    call.append(f'g{q}_{tt}')
                b.append('  bw_rowpre(' + ', '.join(call) + ');\n')
                b += uniform(tt)
        if rfront and late:
            b.append('  }\n')
        if rfront:
            for q in g_tables:
                b.append(f'  __shared__ float s_g{q}[{IPB}][{DT}];\n')
                if HB > 1:
                    b.append('  __syncthreads();\n')
                b.append('  if (n == 0) { ' + ' '.join(f's_g{q}[inst][{tt}] = g{q}_{tt}[0][0];' for tt in range(DT)) + ' }\n')
        # ---- per-row operands of the chunk go through LDS: staged once per row block by the
        # instance's own lanes (coalesced along m), read back per row as broadcast vectors
        rowops = []          # (lds name, loader(tt, mexpr) -> expr, register prefix)
        for i in range(nin):
            if p.in_names[i] in loop_used and self.in_ext(i) == (True, False) and self.tdep[i]:
                def ld(tt, mexpr, i=i):
                    dt = DT_CODE[plan.in_dtypes[i]]
                    idx = self._in_index(A, i, t=tclamp(tt), m=mexpr)
                    return f'ldf<{dt}>({A.p(f"in{i}")}, {idx})'
                rowops.append((f's_c{i}', ld, f'x{i}'))
        for k in range(naux):
            if p.aux[k] in loop_used and not is_rowlike(p.aux[k]):
                rowops.append((f's_ax{k}', (lambda tt, mexpr, k=k: aux_load(k, tt, mexpr)), f'ax{k}'))
        for k in range(ndaux):
            if p.daux[k] in loop_used:
                def ldd(tt, mexpr, k=k):
                    return f'((const float*){A.p("daux")})[((((i64){k} * A.B + b) * H + h) * T + ({tclamp(tt)})) * M + {mexpr}]'
                rowops.append((f's_da{k}', ldd, f'da{k}'))
        for k in range(nout):
            if p.dout_names[k] in loop_used:
                def ldy(tt, mexpr, k=k):
                    dt = DT_CODE[plan.out_dtypes[k]]
                    nmv = f'dout{k}'
                    return (f'ldf<{dt}>({A.p(nmv)}, (i64)b * {A.s(nmv, 0)} + (i64)({tclamp(tt)}) * {A.s(nmv, 1)} + '
                            f'(i64)h * {A.s(nmv, 2)} + (i64)({mexpr}) * {A.s(nmv, 3)})')
                rowops.append((f's_dy{k}', ldy, f'dy{k}'))
        for q in range(len(front)):
            rowops.append((f's_f{q}', None, f'f{q}'))
        for j in colsum:
            b.append(f'  __shared__ float s_cs{j}[{IPB}][{DT}];\n')
        if colsum:
            if HB > 1:
                b.append('  __syncthreads();\n')
            b.append(f'  for (int tt_ = n; tt_ < {DT}; tt_ += {min(N, NT)}) {{ '
                     + ' '.join(f's_cs{j}[inst][tt_] = 0.0f;' for j in colsum) + ' }\n')
        MB = 1
        # (row blocks of up to three tenths of the compute unit's 160 KB of LDS: three workgroups of this kernel stay resident)
        while MB * 2 <= MR and len(rowops) * IPB * (MB * 2) * DT * 4 <= 160 * 1024 * 3 // 10:
            MB *= 2
        lanes = min(N, NT)          # lanes of one instance
        PDe = min(PD, MB)           # (a row block is a whole number of prefetch rounds)
        for nm_lds, _, _ in rowops:
            b.append(f'  __shared__ float {nm_lds}[{IPB}][{MB}][{DT}];\n')

        # element (row m, column n) of this instance's checkpoint: base pointer + m * N
        for k in range(nst):
            b.append(f'  const float* sckp{k} = (const float*){A.p(f"sck{k}")} + (((i64)bh * nch + ch) * M) * {N} + n;\n')
            b.append(f'  const float* dckp{k} = (const float*){A.p(f"dck{k}")} + (((i64)bh * nch + ch) * M) * {N} + n;\n')
            for j in range(PDe):
                b.append(f'  float Sq{k}_{j} = sckp{k}[min(mlo + {j}, M - 1) * {N}];\n  float Dq{k}_{j} = dckp{k}[min(mlo + {j}, M - 1) * {N}];\n')
        if share:       # (the same number of row blocks for every instance of the wave: there are barriers inside)
            b.append(f'  for (int mi_ = 0; mi_ < {MR}; mi_ += {MB}) {{ const int m0 = mlo + mi_;\n')
        else:
            b.append(f'  for (int m0 = mlo; m0 < mhi; m0 += {MB}) {{\n')
        if rowops:
            b.append('    __syncthreads();\n')
            # fixed trip count, fully unrolled: every load of the block is in flight before the
            # first LDS write waits for one
            trips = -(-(MB * DT) // lanes)
            guard = '' if (MB * DT) % lanes == 0 else f'if (e_ < {MB * DT}) '
            b.append(f'#pragma unroll {min(trips, 2)}\n    for (int i_ = 0; i_ < {trips}; i_++) {{ const int e_ = n + i_ * {lanes}; {guard}{{ '
                     f'const int tt_ = e_ / {MB}, mm_ = e_ % {MB}; const int mc_ = min(m0 + mm_, M - 1);\n')
            for nm_lds, ld, _ in rowops:
                if ld is not None:
                    b.append(f'      {nm_lds}[inst][mm_][tt_] = {ld("tt_", "mc_")};\n')
            if front:
                call = []
                for v in pre_used:
                    b.append(f'      float p_{v}[1][1]; p_{v}[0][0] = {raw_value(v, "tt_", "mc_")};\n')
                    call.append(f'p_{v}')
                for q in range(len(front)):
                    b.append(f'      float pf{q}[1][1];\n')
                    call.append(f'pf{q}')
                b.append('      bw_colpre(' + ', '.join(call) + ');\n')
                for q in range(len(front)):
                    b.append(f'      s_f{q}[inst][mm_][tt_] = pf{q}[0][0];\n')
            b.append('    } }\n    __syncthreads();\n')
            if colsum:
                cond = f'if (tt_ < nt) ' if tail else ''
                b.append(f'    for (int tt_ = n; tt_ < {DT}; tt_ += {lanes}) {cond}{{ const int nv_ = min({MB}, mhi - m0);\n')
                for j in colsum:
                    q = front.index(op_names[j])
                    b.append(f'      {{ float a_ = 0.0f; for (int mm_ = 0; mm_ < nv_; mm_++) a_ += s_f{q}[inst][mm_][tt_]; s_cs{j}[inst][tt_] += a_; }}\n')
                b.append('    }\n')
        # The row loop body is written out PDe times per iteration; copy j works on the row in
        # slot j of a ring of checkpoint rows and refills that slot with the row PDe further on
        # (fetched that many rows ahead of use: one row of arithmetic is shorter than a trip to HBM).
        b.append(f'  for (int mm0 = 0; mm0 < {MB}; mm0 += {PDe}) {{\n')
        body_start = len(b)
        for k in range(nst):
            b.append(f'    float Sh{k}_0[1][1]; Sh{k}_0[0][0] = Sq{k}_@J@;\n')
            b.append(f'    float D{k}[1][1]; D{k}[0][0] = Dq{k}_@J@;\n')
        b.append(f'    {{ const int mn_ = min(m + {PDe}, M - 1);\n')
        for k in range(nst):
            b.append(f'      Sq{k}_@J@ = sckp{k}[mn_ * {N}];\n')
            b.append(f'      Dq{k}_@J@ = dckp{k}[mn_ * {N}];\n')
        b.append('    }\n')
        for nm_lds, ld, pref in rowops:
            if ld is None and front[int(pref[1:])] not in loop_used:
                continue                    # only summed over rows, never read by the row loop
            for tt in range(DT):
                b.append(f'    float {pref}_{tt}[1][1]; {pref}_{tt}[0][0] = {nm_lds}[inst][mm][{tt}];\n')
        for i in range(nin):
            if p.in_names[i] not in loop_used or not self.in_ext(i)[0]:
                continue
            if not self.tdep[i]:
                b.append(f'    float x{i}[1][1]; x{i}[0][0] = {load_in(i, 0)};\n')

        def call_args(names, tt, state_var):
            call = []
            for v in names:
                if v in p.in_names:
                    call.append(var_in(p.in_names.index(v), tt))
                elif v in p.st_names:
                    call.append(state_var(p.st_names.index(v)))
                elif v in p.aux:
                    call.append(f'ax{p.aux.index(v)}_{tt}')
                elif v in p.daux:
                    call.append(f'da{p.daux.index(v)}_{tt}')
                elif v in p.dout_names:
                    call.append(f'dy{p.dout_names.index(v)}_{tt}')
                elif v in p.dnst_names:
                    call.append(f'D{p.dnst_names.index(v)}')
                elif v in p.msums:
                    call.append(f'ms{p.msums.index(v)}')
                elif v in front:
                    call.append(f'f{front.index(v)}_{tt}')
                elif v in rfront:
                    call.append(f'g{rfront.index(v)}_{tt}')
                else:
                    raise AssertionError(v)
            return call

        for tt in range(DT - 1):
            for k in range(nst):
                b.append(f'    float Sh{k}_{tt + 1}[1][1];\n')
            call = call_args(re_used, tt, lambda k, tt=tt: f'Sh{k}_{tt}') + [f'Sh{k}_{tt + 1}' for k in range(nst)]
            b.append('    bw_restep(' + ', '.join(call) + ');\n')
        for i in mats2:
            b.append(f'    float ma{i} = 0.0f;\n')
        for tt in range(DT - 1, -1, -1):
            b.append(f'    if ({tt} < nt) {{\n' if tail else '    {\n')
            call = call_args(drow_used, tt, lambda k, tt=tt: f'Sh{k}_{tt}')
            for k in range(nst):
                b.append(f'      float nD{k}[1][1];\n')
                call.append(f'nD{k}')
            for i in mats2:
                b.append(f'      float gm{i}[1][1];\n')
                call.append(f'gm{i}')
            for j in loop_ops:
                b.append(f'      float op{j}[1][1];\n')
                call.append(f'op{j}')
            b.append('      bw_drow(' + ', '.join(call) + ');\n')
            for k in range(nst):
                b.append(f'      D{k}[0][0] = nD{k}[0][0];\n')
            for i in mats2:
                b.append(f'      ma{i} += gm{i}[0][0];\n')
            for j in loop_ops:
                b.append(f'      acc{j}_{tt} += op{j}[0][0];\n')
            b.append('    }\n')
        for i in mats2:
            nmv = f'din{i}'
            idx = f'(i64)b * {A.s(nmv, 0)} + (i64)h * {A.s(nmv, 2)} + (i64)m * {A.s(nmv, 3)} + (i64)n * {A.s(nmv, 4)}'
            b.append(f'    if (valid{" && nok" if self.pad else ""}) atomic_addf({A.p(nmv)}, {idx}, ma{i});\n')
        body = ''.join(b[body_start:])
        del b[body_start:]
        for j in range(PDe):
            b.append(f'  {{\n    const int mm = mm0 + {j}; const int m = m0 + mm;\n    if (m >= mhi) break;\n'
                     + body.replace('@J@', str(j)) + '  }\n')
        b.append('  }\n  }\n')
        # ---- epilogue
        def out_index(i, tt, hexpr):
            nmv = f'din{i}'
            ext = self.in_ext(i)
            return (f'(i64)b * {A.s(nmv, 0)} + (i64)(t0 + {tt}) * {A.s(nmv, 1)} + (i64)({hexpr}) * {A.s(nmv, 2)}'
                    + (f' + (i64)n * {A.s(nmv, 4)}' if ext[1] else ''))

        def write_out(i, tt, hexpr, val, ind):
            nmv = f'din{i}'
            ext = self.in_ext(i)
            bB, bT, bH = bflags(i)
            cond = ('inst == 0' if share else 'valid') + ((' && nok' if self.pad else '') if ext[1] else ' && n == 0')
            if tail and not bT:
                cond += f' && t0 + {tt} < T'
            idx = out_index(i, tt, hexpr)
            if bB or bT or (bH and HB < plan.H) or MS > 1:
                if share:       # the wave's instances hold slices of the same sum: all lanes add them up, one instance writes
                    return f'{ind}{{ const float tot_ = inst_total<{N}>({val}); if ({cond}) atomic_addf({A.p(nmv)}, {idx}, tot_); }}\n'
                return f'{ind}if ({cond}) atomic_addf({A.p(nmv)}, {idx}, {val});\n'
            dt = 0 if i in self.atomic else DT_CODE[plan.in_dtypes[i]]      # broadcast inputs use fp32 scratch
            return f'{ind}if ({cond}) stf<{dt}>({A.p(nmv)}, {idx}, {val});\n'

        tacc = [i for i in rs if bflags(i)[1]]
        for i in tacc:
            b.append(f'  float gt{i} = 0.0f;\n')
        # sums over rows and columns: the column part is a reduction over the instance's lanes.
        # With more than one wave per instance all of them share one pair of barriers.
        nred = [j for j, mname in enumerate(p.msums)
                if 1 in nm_[mname].dims and self.jext[nm_[mname].args[0]][1]]
        batched = N > 64 and bool(nred)
        if colsum:
            b.append('  __syncthreads();\n')
        if batched:
            NW = N // 64
            b.append(f'  __shared__ float red_ms[{len(nred) * DT}][{NW}];\n')
            for q, j in enumerate(nred):
                for tt in range(DT):
                    b.append(f'  acc{j}_{tt} = grp_allreduce<64>({f"nok ? acc{j}_{tt} : 0.0f" if self.pad else f"acc{j}_{tt}"});\n')
            b.append('  __syncthreads();\n  if ((tid & 63) == 0) {\n')
            for q, j in enumerate(nred):
                for tt in range(DT):
                    b.append(f'    red_ms[{q * DT + tt}][tid >> 6] = acc{j}_{tt};\n')
            b.append('  }\n  __syncthreads();\n')
            for q, j in enumerate(nred):
                for tt in range(DT):
                    b.append(f'  acc{j}_{tt} = ' + ' + '.join(f'red_ms[{q * DT + tt}][{w}]' for w in range(NW)) + ';\n')
        if late:
            # An input the preparation has read as well is read again here through a column index the compiler cannot
            # relate to the first one: otherwise it keeps the DT 64-bit addresses of the first read in registers
            # for the length of the row loop (gated linear attention with its gate's raw projection: 195 -> 169).
            b.append('  int nc_late = nc; asm volatile("" : "+v"(nc_late));\n')
            b += chunk_loads(set(epi_used) & late_in, col='nc_late')

        def ms_value(j, tt):
            node = nm_[p.msums[j]]
            if 1 in node.dims and self.jext[node.args[0]][1] and not batched:
                return f'{red}({f"nok ? acc{j}_{tt} : 0.0f" if self.pad else f"acc{j}_{tt}"})'
            return f's_cs{j}[inst][{tt}]' if j in colsum else f'acc{j}_{tt}'

        epi_tot = {}
        if epi_lev:
            for tt in range(DT):
                for j in range(len(p.msums)):
                    b.append(f'  float ms{j}_{tt}[1][1]; ms{j}_{tt}[0][0] = {ms_value(j, tt)};\n')

            def epi_arg(v, tt):
                return f'ms{p.msums.index(v)}_{tt}' if v in p.msums else call_args([v], tt, None)[0]

            epi_tot = levelled(epi_lev, 'ep', epi_arg)
        for tt in range(DT):
            b.append('  {\n')
            if epi_lev:
                fn, used = epi_lev['final']
                call = [total_of(epi_tot, v, tt, '    ') if (v, tt) in epi_tot else epi_arg(v, tt) for v in used]
            else:
                for j in range(len(p.msums)):
                    b.append(f'    float ms{j}[1][1]; ms{j}[0][0] = {ms_value(j, tt)};\n')
                fn, call = 'bw_epi', call_args(epi_used, tt, None)
            for i in rs:
                b.append(f'    float g{i}[1][1];\n')
                call.append(f'g{i}')
            b.append(f'    {fn}(' + ', '.join(call) + ');\n')
            for i in rs:
                if i in tacc:
                    b.append(f'    gt{i} += g{i}[0][0];\n')
                elif i in hacc:
                    b.append(f'    gh{i}_{tt} += g{i}[0][0];\n')
                else:
                    b.append(write_out(i, tt, 'h', f'g{i}[0][0]', '    '))
            b.append('  }\n')
        for i in tacc:
            if i in hacc:
                b.append(f'  gh{i} += gt{i};\n')
            else:
                b.append(write_out(i, '0', 'h', f'gt{i}', '  '))
        b.append('  }\n')        # head loop
        for i in hacc:
            if i in tacc:
                b.append(write_out(i, '0', 'h0', f'gh{i}', '  '))
            else:
                for tt in range(DT):
                    b.append(write_out(i, tt, 'h0', f'gh{i}_{tt}', '  '))
        wpe = int(waves_per_simd)
        attr = f' __attribute__((amdgpu_waves_per_eu({wpe},{wpe})))' if wpe else ''
        kernel = (f'extern "C" __global__ void __launch_bounds__({NT}){attr} frnn_bw2(Args A) {{\n' + ''.join(b) + '}\n')
        source = PRELUDE + A.struct() + helper + re_src + '\n' + drow_src + '\n' + epi_src + '\n' + pre_src + '\n' + kernel
        gx, gy, gz = f'(nch + {cpb - 1}) // {cpb}', f'B * (H // {HB})', str(MS // IPB if share else MS)
        geom = {'kind': 'grad', 'cpb': cpb, 'HB': HB, 'gz': int(gz), 'fold': fold,
                'rows_per_z': plan.M if MS == 1 else (MR * IPB if share else MR)}
        return KernelSpec('frnn_bw2', source, list(A.names), NT, (f'({gx}) * {gy}', '1', gz) if fold else (gx, gy, gz), geom)
