"""Split the joint (step + VJP) graph into the sub-graphs the three kernels run.

The reference makes the equivalent split in
/root/reference/flex_rnn/twopass.py:93-151 (`step`, `restep`, `row_restep`,
`dstep`, `drow`, with `aux` = forward row-sums and `daux` = backward row-sums
saved so that state recompute and all remaining gradients become elementwise
per state element).  It rewrites every sum over the row axis into an
accumulation and leans on the linearity of whatever follows.  Here the split is
made on true broadcast extents instead:

  fw     forward kernel       outputs, new state, aux            (row sums allowed)
  restep recompute            new state from (inputs, state, aux) (no sums left)
  dstep  reverse scan kernel  d_state, col-input grads, daux      (row sums allowed)
  drow   gradient kernel, per element: d_state again, matrix-input grads and
         the operands of every sum over the row axis              (no sums left)
  epi    gradient kernel, once per timestep after the row loop: maps the
         accumulated row-axis sums to the row/scalar-input grads  (column sums allowed)

A value `v` is
  * cotangent-dependent if it depends on an upstream gradient input,
  * an "msum" if it is a sum whose reduced axes include the row axis (0).
Forward sums (`aux`) are those not depending on a cotangent; they are computed by
`fw` and saved.  Backward sums over columns only (`daux`) are computed by `dstep`
and saved when `drow` needs them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Sequence

from .ir import Graph


class PartitionError(AssertionError):
    pass


@dataclass
class Partition:
    joint: Graph
    ninputs: int
    nstates: int
    noutputs: int
    # names in the joint graph
    in_names: List[str]
    st_names: List[str]
    dout_names: List[str]
    dnst_names: List[str]
    out_names: List[str]
    nst_names: List[str]
    din_names: List[str]
    dst_names: List[str]
    aux: List[str]
    daux: List[str]
    msums: List[str]                 # msum nodes consumed by `epi` (accumulated by the row loop)
    col_idx: List[int]
    row_idx: List[int]
    scalar_idx: List[int]
    mat_idx: List[int]
    fw: Graph = None
    restep: Graph = None
    dstep: Graph = None
    drow: Graph = None
    epi: Graph = None
    dstep_needs_state: bool = False
    mat_in_dstep: bool = False       # matrix-input grads are accumulated by the reverse scan (it has the state)
    epi_linear: bool = False         # `epi` is linear and homogeneous in the msums: partial row sums may be
                                     # mapped separately and the results added

    def describe(self) -> str:
        return '\n\n'.join(g.code() for g in (self.fw, self.restep, self.dstep, self.drow, self.epi))


def prologue_front(graphs) -> List[str]:
    """The outermost values of `graphs` that do not vary along the state's rows and are not plain inputs or
    constants: those read by a value with a row extent, or returned.  The row kernels evaluate them once per
    (timestep, column) after staging instead of inside the step."""
    front = []
    for g in graphs:
        for n in g.nodes:
            if n.ext[0] or n.op == 'const' or n.name in front:
                continue
            if n.name in g.outputs or any(n.name in m.value_args() and m.ext[0] for m in g.nodes):
                front.append(n.name)
    return front


def _depends(graph: Graph, seeds: Sequence[str]) -> Dict[str, bool]:
    dep = {i: (i in seeds) for i in graph.inputs}
    for n in graph.nodes:
        dep[n.name] = any(dep[a] for a in n.value_args())
    return dep


def _linear_in(graph: Graph, seeds: Sequence[str]) -> bool:
    """True if every output of `graph` is a linear homogeneous function of the inputs named in
    `seeds` (their coefficients may depend on the other inputs in any way)."""
    IND, LIN, NON = 0, 1, 2          # independent of the seeds / linear in them / anything else
    kind = {i: (LIN if i in seeds else IND) for i in graph.inputs}

    def k(a):
        return kind[a] if isinstance(a, str) else IND

    for n in graph.nodes:
        ks = [k(a) for a in n.args]
        if all(x == IND for x in ks):
            r = IND
        elif NON in ks:
            r = NON
        elif n.op in ('neg', 'copy', 'sum'):
            r = ks[0]
        elif n.op in ('add', 'sub'):
            r = LIN if ks == [LIN, LIN] else NON
        elif n.op == 'mul':
            r = LIN if sorted(ks) == [IND, LIN] else NON
        elif n.op == 'div':
            r = LIN if ks == [LIN, IND] else NON
        elif n.op == 'where':
            r = LIN if ks == [IND, LIN, LIN] else NON
        else:
            r = NON
        kind[n.name] = r
    return all(kind[o] == LIN for o in graph.outputs)


def partition(joint: Graph, ninputs: int, nstates: int, noutputs: int,
              input_classes: Sequence[str]) -> Partition:
    """`input_classes[i]` in {'scalar','col','row','mat'} is the class of input i as
    decided from the caller's tensor shapes (twopass.py:62-72)."""
    names = joint.inputs
    if len(names) != ninputs + nstates + noutputs + nstates:
        raise PartitionError('unexpected joint signature')
    in_names = names[:ninputs]
    st_names = names[ninputs:ninputs + nstates]
    dout_names = names[ninputs + nstates:ninputs + nstates + noutputs]
    dnst_names = names[ninputs + nstates + noutputs:]
    outs = joint.outputs
    out_names = outs[:noutputs]
    nst_names = outs[noutputs:noutputs + nstates]
    din_names = outs[noutputs + nstates:noutputs + nstates + ninputs]
    dst_names = outs[noutputs + nstates + ninputs:]
    if len(dst_names) != nstates:
        raise PartitionError('unexpected joint outputs')

    cot = set(dout_names) | set(dnst_names)
    dep = _depends(joint, cot)
    nm = joint.node_map()

    # forward results must not depend on cotangents
    for v in out_names + nst_names:
        if dep.get(v, False):
            raise PartitionError('forward result depends on a gradient input')

    # classify sums
    aux_all, bsum_n, msum_all = [], [], []
    for n in joint.nodes:
        if n.op != 'sum':
            continue
        if not dep[n.name]:
            if n.dims != (1,):
                raise PartitionError('Only torch.sum(x, dim=-1, keepdim=True) is supported')
            aux_all.append(n.name)
        elif 0 in n.dims:
            msum_all.append(n.name)
        else:
            bsum_n.append(n.name)

    # A forward sum without a row extent (the squared norm of a key that the step normalises, say) depends on a
    # timestep's row / scalar inputs only - anything that reads the state varies along rows.  It is not saved per state
    # row like the others: every kernel forms it again from the inputs, once per timestep.
    jext = joint.ext_table()
    aux_all = [a for a in aux_all if jext[a][0]]

    def row_sums(g: Graph):
        """Sums in `g` over an operand that varies along rows: those a per-element pass cannot contain."""
        gm = g.ext_table()
        return [n.name for n in g.nodes if n.op == 'sum' and gm[n.args[0]][0]]

    mdep = {i: False for i in joint.inputs}
    for n in joint.nodes:
        mdep[n.name] = (n.name in msum_all) or any(mdep[a] for a in n.value_args())

    col_idx = [i for i, c in enumerate(input_classes) if c == 'col']
    row_idx = [i for i, c in enumerate(input_classes) if c == 'row']
    scalar_idx = [i for i, c in enumerate(input_classes) if c == 'scalar']
    mat_idx = [i for i, c in enumerate(input_classes) if c == 'mat']

    # --- epilogue: row/scalar input grads from accumulated row-axis sums ---------------
    epi_outs = [din_names[i] for i in row_idx + scalar_idx]
    epi = joint.extract('epi', epi_outs, cut=set(aux_all) | set(msum_all))
    for n in epi.nodes:
        if n.ext[0]:
            raise PartitionError(f'gradient of a row/scalar input needs a per-row value after the row reduction ({n.name})')
        if n.op == 'sum' and n.dims != (1,):
            raise PartitionError('unexpected reduction in gradient epilogue')
    for i, used in zip(epi.inputs, epi.used_inputs()):
        if used and epi.input_ext[i][0]:
            if i in msum_all:
                continue
            raise PartitionError(f'gradient epilogue reads a per-row value ({i})')
    msums = [m for m in msum_all if epi.uses(m)]
    for o in epi_outs:
        if o in joint.input_ext and joint.input_ext[o][0]:
            raise PartitionError('row/scalar gradient aliases a per-row input')
    msum_operands = [nm[m].args[0] for m in msums]
    for v in msum_operands:
        if mdep[v]:
            raise PartitionError('nested reductions over the row axis are not supported')

    # --- where matrix-input gradients are formed ------------------------------------------
    # If the reverse scan has to recompute the state anyway (a column gradient or a saved
    # backward sum reads it), it also accumulates the matrix-input gradients over the whole
    # sequence in registers; otherwise the gradient kernel does, chunk by chunk.
    probe = joint.extract('probe', list(dst_names) + [din_names[i] for i in col_idx], cut=set(aux_all))
    # The same holds when the gradient kernel would have nothing else to do (no row or scalar
    # input): recomputing the state in the reverse scan is cheaper than a kernel whose every
    # chunk adds a full matrix of partial gradients with atomics.
    mat_in_dstep = bool(mat_idx) and (any(probe.uses(s_) for s_ in st_names) or not (row_idx or scalar_idx))
    mats_drow = [] if mat_in_dstep else list(mat_idx)
    mats_dstep = list(mat_idx) if mat_in_dstep else []

    # --- drow: per-element part of the gradient kernel -------------------------------
    drow_outs = list(dst_names) + [din_names[i] for i in mats_drow] + msum_operands
    for v in list(dst_names) + [din_names[i] for i in mat_idx + col_idx]:
        if mdep.get(v, False):
            raise PartitionError('state / column / matrix gradient depends on a reduction over the row axis')
    drow = joint.extract('drow', drow_outs, cut=set(aux_all) | set(bsum_n))
    if row_sums(drow):
        raise PartitionError('unsupported reduction in the backward pass')
    daux = [s for s in bsum_n if drow.uses(s)]

    # --- dstep: reverse scan -----------------------------------------------------------
    dstep_outs = list(dst_names) + [din_names[i] for i in col_idx] + daux + [din_names[i] for i in mats_dstep]
    dstep = joint.extract('dstep', dstep_outs, cut=set(aux_all))
    for n in dstep.nodes:
        if n.op == 'sum' and n.dims != (1,):
            raise PartitionError('column-input gradient needs a reduction over the row axis')
    dstep_needs_state = any(dstep.uses(s) for s in st_names)

    # --- restep -------------------------------------------------------------------------
    restep = joint.extract('restep', list(nst_names), cut=set(aux_all))
    if row_sums(restep):
        raise PartitionError('unsupported reduction while recomputing the state')

    aux = [a for a in aux_all if restep.uses(a) or dstep.uses(a) or drow.uses(a) or epi.uses(a)]

    # re-extract with the final aux set only (so unused forward sums are recomputed inline
    # rather than listed as inputs); cutting at the full set is equivalent since unused cuts
    # never become inputs.
    fw = joint.extract('fw', list(out_names) + list(nst_names) + aux, cut=())
    for n in fw.nodes:
        if n.op == 'sum' and n.dims != (1,):
            raise PartitionError('Only torch.sum(x, dim=-1, keepdim=True) is supported')
    fw_used = fw.used_inputs()
    if any(fw_used[ninputs + nstates:]):
        raise PartitionError('forward pass depends on gradients')

    p = Partition(joint, ninputs, nstates, noutputs, in_names, st_names, dout_names, dnst_names,
                  out_names, nst_names, din_names, dst_names, aux, daux, msums,
                  col_idx, row_idx, scalar_idx, mat_idx,
                  fw=fw, restep=restep, dstep=dstep, drow=drow, epi=epi,
                  dstep_needs_state=dstep_needs_state, mat_in_dstep=mat_in_dstep,
                  epi_linear=_linear_in(epi, set(msums)))
    return p
