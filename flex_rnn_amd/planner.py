"""Planner: validates the call, classifies operands, traces + partitions the step,
chooses tile sizes and hidden-buffer layouts, and (unless `dryrun`) builds the
HIP kernels and returns the `forward` / `backward` closures.

Interface and behaviour follow /root/reference/flex_rnn/twopass.py:
  * `split_list`, `get_meta`, `verify_meta`                     (twopass.py:8-15, 33-42)
  * `build_twopass(step, inputs, state, dryrun=False)`           (twopass.py:44-366)
      -> (forward, backward, forward_meta, backward_meta)  or the two metas when dryrun
  * `forward(inputs, state) -> (*y, *stateT, *state_store, aux)` (twopass.py:224-237)
  * `backward(doutput, dstateT, inputs, state_store, aux)
        -> (tuple(dinputs), tuple(dstate0))`                     (twopass.py:343-363)
The kernels, their tiling and the layout of the hidden buffers (`state_store`,
`aux`) are this backend's own.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch as th

from . import tracer
from .partition import Partition, partition, prologue_front

SUPPORTED_DTYPES = (th.float32, th.bfloat16, th.float16, th.float64)
LDS_BYTES = 160 * 1024         # per compute unit on gfx950 (and the most one workgroup may use)


def split_list(args, lens):
    """Cut `args` into consecutive pieces of the given lengths (twopass.py:8-15)."""
    out, off = [], 0
    for n in lens:
        out.append(args[off:off + n])
        off += n
    assert off == len(args), f'expected {off} arguments, got {len(args)}'
    return out


def get_meta(tensors):
    return tuple((t.shape, t.stride(), t.dtype) for t in tensors)


def _eff_stride(shape, stride):
    return [s if n > 1 else 0 for s, n in zip(stride, shape)]


def verify_meta(a, b, msg=''):
    """Shapes, dtypes and strides (ignoring size-1 dims) must agree (twopass.py:36-42)."""
    for i, (x, y) in enumerate(zip(a, b)):
        ash, ast, adt, bsh, bst, bdt = x.shape, x.stride(), x.dtype, y.shape, y.stride(), y.dtype
        if ash == bsh and ast == bst and adt == bdt:
            continue
        assert ash == bsh, msg + f'#{i+1}: a_shape={ash} != b_shape={bsh}'
        a_stride, b_stride = _eff_stride(ash, ast), _eff_stride(bsh, bst)
        assert a_stride == b_stride, msg + f'#{i+1}: {a_stride=} != {b_stride=}'
        assert adt == bdt, msg + f'#{i+1}: a_dtype={adt} != b_dtype={bdt}'


def _pow2_floor(n: int) -> int:
    return 1 << (max(int(n), 1).bit_length() - 1)


def _is_pow2(n: int) -> bool:
    return n >= 1 and (n & (n - 1)) == 0


@dataclass
class TileConfig:
    """Launch geometry of the three kernels.

    Row kernels (fw, bw1): a wave holds G = 64/L row groups; each group of L lanes holds
    R consecutive state rows, each lane C = N/L columns of them.  W waves per workgroup, so a
    workgroup owns MT = W*G*R rows of one (batch, head).  Inputs are staged through LDS TS
    timesteps at a time; the state is checkpointed every DT steps.
    Gradient kernel (bw2): one lane per state column, DT timesteps per instance, a serial
    loop over the M rows."""
    L: int
    C: int
    R: int
    W: int
    DT: int
    TS: int
    R1: int = 0          # rows per lane / waves in bw1 (0 = same as fw)
    W1: int = 0
    HB: int = 1          # heads walked by one gradient-kernel instance (sums head-broadcast grads in registers)
    MS: int = 1          # instances sharing the rows of one (batch, head, chunk) in the gradient kernel;
                         # above 1 the row/scalar-input grads are summed across them with atomics
    WPE: int = 0         # waves per SIMD the row kernels are compiled for (0 = whatever the compiler arrives at)
    WN: int = 0          # row kernels: at least this many waves per SIMD (0 = no request).  A workgroup of four waves may use a
                         # SIMD's whole register file; near 256 registers the compiler then parks values in the accumulation
                         # registers or in scratch, with 2 here it allocates within 256 (Mamba-1's reverse scan: 0.33 -> 0.31 ms)
    UR: int = 2          # row kernels: unrolling of the loop over the staged timesteps
    NB: int = 1          # row sums leave a step without a branch (every lane of a group stores them): bit 0 = forward
                         # kernel, bit 1 = reverse scan.  Lets the compiler overlap consecutive steps, at the price of registers.
    DF: int = 0          # row kernels: 1 = a chunk's results leave LDS during the next chunk (double buffer) and checkpoints are
                         # stored after the wait for the staged operands, so that a wave's stores have a chunk's time to complete
                         # before it next waits for its prefetched loads.  Pays on some recurrences only; a timed candidate.
    KS: int = 0          # row kernels: a block's row sums stay in registers (lane l of a group keeps the steps l, l + L, ...) and
                         # go to LDS once per block instead of once per step, where a group has at least TS / 2 lanes: bit 0 =
                         # forward kernel, bit 1 = reverse scan.  Fewer LDS stores for a few more vector instructions; a timed candidate.
    SH: int = 1          # reverse scan with state recompute: per-row operands loaded once for recompute and d-step
                         # (measured on RWKV-7: within 2 % of 0 either way; kept as a tuning knob)

    @property
    def G(self): return 64 // self.L
    @property
    def MT(self): return self.W * self.G * self.R


@dataclass
class Plan:
    B: int
    T: int
    H: int
    M: int
    N: int
    part: Partition
    in_cls: List[str]
    in_dtypes: List[th.dtype]
    in_bcast: List[Tuple[bool, bool, bool]]     # input broadcast over (B, T, H)
    st_dtypes: List[th.dtype]
    out_dtypes: List[th.dtype]
    tile: TileConfig
    nchunks: int

    @property
    def NP(self) -> int:
        """State width the kernels are laid out for: N rounded up to a power of two.  The columns
        beyond N are padding: never loaded or stored, masked out of every sum."""
        return 1 << (self.N - 1).bit_length()

    @property
    def atomic(self) -> List[int]:
        """Inputs whose gradient is accumulated in fp32 (zero-filled, cast back afterwards): those
        broadcast over batch, time or heads, the row / scalar inputs of a row-split gradient kernel,
        and every matrix input.  A matrix input has no time axis, so its gradient is a sum over the
        timesteps and the kernels always form it in fp32 - also at T == 1, where its size-1 time axis
        does not count as a broadcast."""
        split = set(self.part.row_idx + self.part.scalar_idx) if self.tile.MS > 1 else set()
        mats = set(self.part.mat_idx)
        return [i for i, b in enumerate(self.in_bcast) if any(b) or i in split or i in mats]


def classify(inputs, state):
    """Shape validation and operand classes (twopass.py:45-72)."""
    B, T, H = [max(i.shape[j] for i in inputs) for j in range(3)]
    if state and state[0].ndim == 4 and 0 in (state[0].shape[0], min(i.shape[1] for i in inputs)):
        # an empty batch or no timesteps: a size of 1 is a broadcast input there, not the extent
        B = state[0].shape[0]
        T = 0 if min(i.shape[1] for i in inputs) == 0 else T
    M = max(i.shape[-2] for i in tuple(inputs) + tuple(state))
    N = max(i.shape[-1] for i in tuple(inputs) + tuple(state))
    dims = [B, T, H, M, N]
    for i, x in enumerate(inputs):
        assert x.ndim == 5, f'invalid shape {list(x.shape)} of argument #{i+1}'
        for j in range(5):
            assert x.shape[j] in [1, dims[j]], \
                f'shape {list(x.shape)} of argument #{i+1} is incompatible with {dims}'
        assert 1 in x.shape[-2:] or x.shape[1] == 1, \
            f'shape {list(x.shape)} of argument #{i+1} is both a matrix for each head, and depends on time. This is not supported'
        assert x.dtype in SUPPORTED_DTYPES, f'unsupported dtype {x.dtype} of argument #{i+1}'
    for i, x in enumerate(state):
        assert list(x.shape) == [B, H, M, N], \
            f'shape {list(x.shape)} of argument #{i+1+len(inputs)} != {[B, H, M, N]}'
        assert x.dtype in SUPPORTED_DTYPES, f'unsupported dtype {x.dtype} of argument #{i+1+len(inputs)}'
    cls = []
    for x in inputs:
        mn = list(x.shape[-2:])
        if mn == [1, 1]:
            cls.append('scalar')
        elif mn == [M, 1]:
            cls.append('col')
        elif mn == [1, N]:
            cls.append('row')
        else:
            assert mn == [M, N]
            cls.append('mat')
    bcast = [tuple(x.shape[j] == 1 and dims[j] != 1 for j in range(3)) for x in inputs]
    return dims, cls, bcast


def staging_depth(part, N: int, MT: int, W: int, DT: int) -> int:
    """Timesteps staged through LDS at a time by a row-kernel workgroup of W waves that owns MT state rows: as many as
    fit (inputs, prepared rows, per-row results), at most DT."""
    cls = part_input_classes(part)
    ins = sum({'row': N, 'col': MT, 'scalar': 1, 'mat': 0}[c] for c in cls)
    # (values the kernels prepare per (timestep, column) after staging have LDS rows of their own)
    jext = part.joint.ext_table()
    pro = max(sum(N if jext[f][1] else 1 for f in prologue_front([g])) for g in (part.fw, part.dstep))
    per_step = ins + pro + max(part.noutputs + len(part.aux),                                       # forward
                               len(part.aux) + part.noutputs + len(part.col_idx) + len(part.daux)) * (MT + 4)   # reverse scan (+ padding of kept row sums)
    # gfx950 has 160 KB of LDS per compute unit; a workgroup gets the share that still leaves eight waves resident
    budget = max(64 * 1024, LDS_BYTES // max(1, -(-8 // W)))
    TS = DT
    while TS > 1 and per_step * TS * 4 > budget - 256:
        TS //= 2
    if part.dstep_needs_state:
        TS = DT
    return TS


def choose_tiles(B, T, H, M, N, part: Partition, n_cu: int = 256, in_bcast=None) -> TileConfig:
    """Tile heuristics (the counterpart of twopass.py:154-173, for 64-wide waves)."""
    N = 1 << (N - 1).bit_length()          # lanes and tiles cover the padded width
    nst = part.nstates + len(part.mat_idx)

    n_row = sum(1 for i in part.row_idx if in_bcast is None or not in_bcast[i][1])
    r_lds = 1
    while r_lds * 5 < 4 * n_row:
        r_lds *= 2

    def geometry(C_):
        L_ = N // C_
        G_ = 64 // L_
        # rows per lane: bounded by the register budget (state + new state + temporaries) ...
        R_ = _pow2_floor(max(1, min(64 // max(C_ * nst, 1), 8)))
        while R_ > 1 and G_ * R_ > M:          # ... by the rows that exist ...
            R_ //= 2

        def waves_per_wg(r):
            return _pow2_floor(max(1, min(4, M // (G_ * r)))) if G_ * r <= M else 1      # (a power of two; the grid covers ragged rows)

        def total_waves(r):
            w = waves_per_wg(r)
            return B * H * max(1, -(-M // (w * G_ * r))) * w

        # ... and small enough that every SIMD holds at least two waves (latency hiding) ...
        while R_ > 1 and total_waves(R_) < 2 * 4 * n_cu:
            R_ //= 2
        # ... four, where LDS bandwidth allows: every lane reads C values of each staged row
        # operand per step whatever R is, so fewer rows per lane means more LDS traffic per
        # element (measured: 5 row operands at R = 4 keep the LDS half busy)
        while R_ > r_lds and R_ // 2 >= r_lds and total_waves(R_) < 4 * 4 * n_cu:
            R_ //= 2
        return L_, G_, R_, waves_per_wg(R_), total_waves(R_)

    # columns per lane: up to 8, so that a row of up to 128 columns fits one 16-lane DPP row;
    # fewer when the whole problem would otherwise give the chip too few waves (narrow states)
    C = min(N, 8)
    while N // C > 64:
        C *= 2
    L, G, R, W, waves = geometry(C)
    while C > 2 and N // (C // 2) <= 64 and waves < 2 * 4 * n_cu:
        C //= 2
        L, G, R, W, waves = geometry(C)
    if part.dstep_needs_state:
        # several states there leave chunks of under 8 steps at 8 columns per lane, and the forward kernel then
        # spends its time storing checkpoints (S4D, two states: 1.05 -> 0.64 ms with 4 columns per lane)
        while C > 2 and N // (C // 2) <= 64 and 64 // (C * part.nstates) < 8:
            C //= 2
            L, G, R, W, waves = geometry(C)
    MT = W * G * R
    R1 = W1 = 0
    if part.dstep_needs_state:
        # the reverse scan keeps the DT recomputed states of a chunk in registers: one row per
        # lane there, and a chunk short enough for 64 registers of history per state (measured:
        # anything more drops the kernel to one wave per SIMD or spills)
        R1 = 1
        W1 = _pow2_floor(max(1, min(4, M // G))) if G <= M else 1
        DT = max(2, min(16, _pow2_floor(64 // max(C * part.nstates, 1))))
    else:
        DT = 16
    while DT > 1 and DT > T:              # a partial last chunk is handled in the kernels
        DT //= 2
    TS = staging_depth(part, N, MT, W, DT)
    # gradient kernel: one instance per (batch, head, chunk) walks all M rows.  When that gives the
    # chip too few waves (narrow states pack several instances into a wave), the rows are split
    # over MS instances whose row/scalar-input grads meet in fp32 atomics; needs an epilogue that
    # is linear in the row sums.  Walking several heads per instance (HB > 1) saves atomics on
    # head-shared inputs but costs registers and parallelism; measured slower, so it stays 1.
    ipb = max(1, 64 // N)
    waves2 = B * H * -(-(-(-T // DT)) // ipb) * max(1, N // 64)
    MS = 1
    rs = part.row_idx + part.scalar_idx
    shared = in_bcast is not None and all(any(in_bcast[i]) for i in rs)
    # (measured: where splitting would turn plain stores of row gradients into atomics - RWKV-7 at a
    # small batch - it costs more than the extra waves bring; with inputs shared over batch, time or
    # heads the gradients are accumulated atomically anyway - Mamba-1 - and it pays)
    # Otherwise rows are only split when the chip would be mostly idle (under two waves per SIMD).
    if part.epi_linear:
        target = (32 if (shared or N <= 32) else 2) * 4 * n_cu      # (narrow states: light instances, several per wave)
        while waves2 * MS < target and -(-M // (2 * MS)) >= 8:
            MS *= 2
    return TileConfig(L=L, C=C, R=R, W=W, DT=DT, TS=TS, R1=R1, W1=W1, HB=1, MS=MS)


def check_tile(tile: TileConfig, H: int, N: int, part: Partition) -> None:
    """Rejects a tile the kernels cannot run (an override is not trusted): the emitted index
    arithmetic assumes every one of these."""
    t = tile
    for k in ('L', 'C', 'R', 'W', 'DT', 'TS'):
        assert getattr(t, k) >= 1 and _is_pow2(getattr(t, k)), f'tile field {k}={getattr(t, k)} must be a power of two'
    assert t.HB >= 1 and 1 <= t.MS <= 65535, 'HB and MS must be positive (MS is a grid dimension)'
    assert 0 <= t.WPE <= 8 and 0 <= t.WN <= 8, 'WPE and WN are waves per SIMD (0 = no request, at most 8)'
    assert t.UR >= 1 and 0 <= t.NB <= 3 and t.DF in (0, 1) and t.SH in (0, 1), 'UR >= 1, NB in 0..3, DF and SH 0 or 1'
    for k in ('R1', 'W1'):
        assert getattr(t, k) == 0 or _is_pow2(getattr(t, k)), f'tile field {k}={getattr(t, k)} must be 0 or a power of two'
    assert t.L <= 64 and t.L * t.C == N, f'tile covers {t.L}*{t.C} columns, the state has {N}'
    assert t.W <= 16 and (t.W1 or t.W) <= 16, 'at most 16 waves per workgroup'
    assert t.DT % t.TS == 0, 'the checkpoint interval must be a multiple of the staging depth'
    assert not part.dstep_needs_state or t.TS == t.DT, \
        'a reverse scan that recomputes the state stages a whole chunk (TS == DT)'
    assert H % t.HB == 0, f'HB={t.HB} does not divide H={H}'
    assert t.MS == 1 or part.epi_linear, 'rows can only be split (MS > 1) when the gradient epilogue is linear in the row sums'


def part_input_classes(part: Partition) -> List[str]:
    cls = [None] * part.ninputs
    for name, idx in (('col', part.col_idx), ('row', part.row_idx), ('scalar', part.scalar_idx), ('mat', part.mat_idx)):
        for i in idx:
            cls[i] = name
    return cls


def make_plan(step: Callable, inputs, state, tile: Optional[TileConfig] = None) -> Tuple[Plan, tuple, tuple]:
    (B, T, H, M, N), cls, bcast = classify(inputs, state)

    # one timestep's worth of every input, as shapes only (so that T == 0 plans too)
    inputs_t = [th.empty((i.shape[0], *i.shape[2:]), dtype=i.dtype, device='meta') for i in inputs]
    res = step(*inputs_t, *[s.to('meta') for s in state])
    output_t, nstate = [r if isinstance(r, tuple) else (r,) for r in res]
    ninputs, noutputs, nstates = len(inputs_t), len(output_t), len(nstate)
    assert len(nstate) == len(state), 'step must return as many states as it takes'
    assert all(a.shape == b.shape for a, b in zip(nstate, state)), 'new state shape differs from the state shape'
    assert all(list(i.shape) == [B, H, M, 1] for i in output_t), [i.shape for i in output_t]
    assert all(i.dtype in SUPPORTED_DTYPES for i in output_t)

    # Trace on [m, n] shapes.  With a single state row (M == 1) a [1, n] state would be
    # indistinguishable from a row-broadcast operand and the graph would lose its row extents;
    # it is traced with two rows instead (inputs keep their size-1 row axis, i.e. are broadcast
    # over rows, which is the same thing for one row).
    Mt = 2 if M == 1 else M
    metas = tuple(th.empty(j.shape[-2:], dtype=j.dtype, device='meta') for j in inputs_t) \
        + tuple(th.empty((Mt, N), dtype=s.dtype, device='meta') for s in state)
    joint, nfw = tracer.trace_step(step, metas)
    assert nfw == noutputs + nstates
    part = partition(joint, ninputs, nstates, noutputs, cls)

    if tile is None:
        tile = choose_tiles(B, T, H, M, N, part, in_bcast=bcast)
        override = os.environ.get('FLEX_RNN_TILE')          # e.g. "R=2,TS=8" (tuning / tests)
        if override:
            import dataclasses
            tile = dataclasses.replace(tile, **{k: int(v) for k, v in (kv.split('=') for kv in override.split(','))})
    check_tile(tile, H, 1 << (N - 1).bit_length(), part)
    nchunks = -(-T // tile.DT)
    plan = Plan(B, T, H, M, N, part, cls, [i.dtype for i in inputs], bcast,
                [s.dtype for s in state], [o.dtype for o in output_t], tile, nchunks)

    dev = 'meta'
    output_out = tuple(th.empty(B, T, H, M, dtype=o.dtype, device=dev) for o in output_t)
    dstate = tuple(th.empty_like(s, device=dev) for s in state)
    state_store = tuple(th.empty(B, H, nchunks, M, plan.NP, dtype=th.float32, device=dev) for _ in state)
    aux_out = (th.empty(len(part.aux), B, H, T, M, dtype=th.float32, device=dev),)
    dinputs_out = tuple(th.empty_like(i, device=dev) for i in inputs)
    forward_meta = get_meta([*output_out, *dstate, *state_store, *aux_out])
    backward_meta = get_meta([*dinputs_out, *dstate])
    return plan, forward_meta, backward_meta


def build_twopass(step: Callable, inputs, state, dryrun: bool = False, tile: Optional[TileConfig] = None):
    inputs, state = tuple(inputs), tuple(state)
    plan, forward_meta, backward_meta = make_plan(step, inputs, state, tile)
    if dryrun:
        return forward_meta, backward_meta

    from .launch import CompiledPlan
    compiled = CompiledPlan(plan, state_meta=forward_meta[plan.part.noutputs:plan.part.noutputs + plan.part.nstates],
                            device=inputs[0].device)

    in_meta = tuple(th.empty_strided(i.shape, i.stride(), dtype=i.dtype, device='meta') for i in inputs)
    st_meta = tuple(th.empty_strided(s.shape, s.stride(), dtype=s.dtype, device='meta') for s in state)
    fw_out_meta = tuple(th.empty_strided(sh, st, dtype=dt, device='meta') for sh, st, dt in forward_meta)
    nout, nst = plan.part.noutputs, plan.part.nstates

    def forward(inputs_, state0):
        verify_meta(inputs_, in_meta, 'input Tensor metadata doesn\'t match compilation\n')
        verify_meta(state0, st_meta, 'initial state Tensor metadata doesn\'t match compilation\n')
        return compiled.forward(tuple(inputs_), tuple(state0))

    def backward(doutput, dstateT_, inputs_, state_store_, aux_):
        # (gradients arrive in whatever layout autograd gives them; the kernels take them contiguous.  Shape and
        # dtype must be those of the final states this plan produced - twopass.py:346 - or the reverse scan
        # would read them with the wrong element size.)
        for k, (g, m) in enumerate(zip(dstateT_, fw_out_meta[nout:nout + nst])):
            assert g.shape == m.shape and g.dtype == m.dtype, \
                f'final-state gradient #{k+1}: {tuple(g.shape)} {g.dtype} does not match compilation ({tuple(m.shape)} {m.dtype})'
        doutput, dstateT_ = [tuple(i.contiguous() for i in j) for j in (doutput, dstateT_)]
        verify_meta(inputs_, in_meta)
        verify_meta(doutput, fw_out_meta[:nout])
        verify_meta(state_store_, fw_out_meta[nout + nst:nout + 2 * nst])
        verify_meta(aux_, fw_out_meta[nout + 2 * nst:])
        return compiled.backward(doutput, dstateT_, tuple(inputs_), tuple(state_store_), aux_[0])

    def forward_only(inputs_, state0):
        verify_meta(inputs_, in_meta, 'input Tensor metadata doesn\'t match compilation\n')
        verify_meta(state0, st_meta, 'initial state Tensor metadata doesn\'t match compilation\n')
        return compiled.forward_only(tuple(inputs_), tuple(state0))

    forward.compiled = backward.compiled = compiled
    forward.forward_only = forward_only
    return forward, backward, forward_meta, backward_meta
