"""Runs the emitted HIP kernels on the CPU (tests/hipsim) and compares forward results and all
gradients with the oracle.  Every buffer of every launch sits against a guard page, at its end
in one run and at its start in another, so an out-of-bounds index of a generated kernel fails
the test with a signal."""
import os
import subprocess
import sys

import pytest

import cases

HERE = os.path.dirname(os.path.abspath(__file__))
RUNNER = os.path.join(HERE, 'hipsim', 'run_case.py')

# (case, B,T,H,M,N, dtype, guard at end?)
RUNS = [
    ('cfg:delta_rule', '1,64,2,16,16', 'f32', 1),
    ('cfg:mamba1', '2,16,2,128,16', 'f32', 1),      # reverse scan with state recompute, matrix grads, atomics
    ('cfg:mamba2', '1,16,2,64,128', 'bf16', 1),     # scalar inputs, head-broadcast rows
    ('cfg:rwkv7', '1,16,1,128,128', 'bf16', 1),
    ('cfg:gated_delta_rule', '1,16,1,128,128', 'bf16', 1),
    ('rwkv7', '1,16,2,64,64', 'bf16', 0),           # log-decay: exp evaluated while staging / once per chunk
    ('delta_rule_fused', '2,16,2,16,32', 'f32', 1), # in-step normalisation (row-only sum) and gate
    ('rwkv6', '2,8,2,16,16', 'f32', 1),             # time-independent row input
    ('s4d', '2,8,1,8,16', 'f32', 1),                # two states, four matrix inputs
    ('longhorn', '2,8,2,16,8', 'f32', 0),           # row-only forward sum
    ('retention', '1,8,2,8,32', 'f16', 1),
    ('mlstm_cell', '1,8,2,8,8', 'bf16', 1),
    ('hgrn', '2,8,1,64,1', 'f32', 1),               # vector state (N = 1)
    ('rwkv4', '2,8,1,32,1', 'f32', 0),              # three states, comparisons
    ('mlstm_gates', '2,8,2,16,1', 'f32', 1),        # three outputs
    # row counts that are not a power of two (the heuristic once asked for three waves per workgroup there)
    ('cfg:mamba1', '2,35,4,24,16', 'bf16', 1),
    ('cfg:rwkv7', '2,17,2,48,64', 'f32', 0),
    # sequence lengths that are not a multiple of the chunk (partial last chunk), and T = 1
    ('cfg:rwkv7', '1,37,1,128,128', 'f32', 0),
    ('cfg:mamba1', '2,13,2,128,16', 'f32', 1),
    ('cfg:mamba2', '1,21,2,64,128', 'bf16', 0),
    ('rwkv4', '2,11,1,32,1', 'f32', 0),
    ('cfg:gated_delta_rule', '1,1,2,128,128', 'bf16', 1),
    # a single timestep with a matrix input that is broadcast over nothing: its gradient is still formed in
    # fp32 (by the reverse scan for `mamba_bh`, by the gradient kernel for `matgain`) and cast afterwards
    ('mamba_bh', '2,1,2,16,16', 'bf16', 1),
    ('mamba_bh', '2,1,2,16,16', 'bf16', 0),
    ('matgain', '2,1,2,16,16', 'bf16', 1),
    ('matgain', '2,1,2,16,16', 'f16', 0),
    ('matgain', '2,5,2,16,16', 'f64', 1),
    # the emitter's op table (sigmoid, tanh, softplus, where, relu, sqrt, rsqrt, log, min/max, ...)
    ('zoo', '2,8,2,16,16', 'f32', 1),
    ('zoo2', '2,8,2,16,16', 'f32', 0),
    # state heights that are not a power of two (row masking), fp64 and fp16 I/O
    ('cfg:rwkv7', '1,16,1,24,128', 'f32', 0),
    ('gla', '2,8,2,100,32', 'f32', 1),
    ('zoo', '1,8,2,5,8', 'f64', 0),
    ('gla', '1,8,2,16,16', 'f16', 1),
    # state widths that are not a power of two (padding columns: masked sums, guarded loads / stores)
    ('cfg:rwkv7', '1,16,2,24,96', 'f32', 0),
    ('cfg:mamba1', '2,16,2,8,12', 'f32', 1),
    ('cfg:mamba2', '2,16,2,8,160', 'bf16', 1),
    ('cfg:gated_delta_rule', '1,16,2,16,80', 'f32', 0),
    ('zoo2', '1,8,2,4,3', 'f32', 1),
    ('s4d', '2,8,1,8,6', 'f32', 0),
    ('delta_rule_fused', '2,16,2,8,20', 'f32', 1),
    # a single state row (M = 1), down to a scalar state (M = N = 1)
    ('mlstm_gates', '2,8,2,1,1', 'f32', 1),
    ('gla', '2,8,2,1,16', 'f32', 0),
    # steps built by `flex_rnn_amd.layer`: the layer's input preparation (softplus / sigmoid gates, L2-normalised keys,
    # a gate tied to another) evaluated inside the kernels, gradients with respect to the raw projections
    ('layer:rwkv7', '2,19,2,16,16', 'f32', 1),
    ('layer+:rwkv7', '2,19,2,16,16', 'f32', 0),             # (norms along the column axis inside the kernels too)
    ('layer+:gated_delta_rule', '1,16,2,32,32', 'bf16', 0),
    ('layer+:gated_delta_rule', '1,19,1,128,128', 'f32', 1),   # two waves per gradient-kernel instance: batched sums
    ('layer:mamba2', '2,21,2,16,16', 'f32', 1),
    ('layer:hgrn', '2,9,1,32,1', 'f32', 0),
    ('longhorn', '1,8,1,8,128', 'f32', 1),                  # fewer staged timesteps than groups of lanes that sum them
]


@pytest.mark.parametrize('case,dims,dtype,end', RUNS)
def test_emitted_kernels_on_cpu(case, dims, dtype, end):
    r = subprocess.run([sys.executable, RUNNER, case, dims, dtype, str(end)], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, f'rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-3000:]}'


# explicit tile overrides: gradient-kernel instances that split the rows of one chunk (MS), with a
# split that gets no row at all (M = 5 over 4 instances of 2 rows), and instances that walk heads (HB)
TILED = [
    ('cfg:rwkv7', '1,16,2,24,64', 'f32', 0, 'MS=4'),
    ('cfg:mamba1', '2,16,2,5,16', 'f32', 1, 'MS=4'),
    ('cfg:mamba2', '2,21,2,7,128', 'bf16', 1, 'MS=3'),
    ('cfg:mamba2', '2,16,4,16,128', 'f32', 0, 'HB=2,MS=1'),
    ('cfg:mamba2', '2,16,4,16,128', 'f32', 1, 'HB=4,MS=2'),
    # row-kernel tiles that the first-call timing may pick instead of the heuristic's
    ('cfg:rwkv7', '1,16,1,128,128', 'f32', 0, 'R=2,W=8,R1=2,W1=4'),
    ('cfg:mamba2', '1,16,2,64,128', 'f32', 1, 'R=1,W=8,R1=1,W1=8'),
    ('cfg:mamba1', '2,16,2,128,16', 'f32', 0, 'R=1,W=8,R1=1,W1=8'),
    # 16 columns per lane (a state row of 128 in 8 lanes: three reduction steps), one workgroup per head
    ('cfg:rwkv7', '1,19,2,128,128', 'bf16', 1, 'L=8,C=16,R=2,W=8,R1=2,W1=8'),
    ('cfg:mamba2', '1,16,2,64,128', 'f32', 0, 'L=8,C=16,R=1,W=8,R1=1,W1=8'),
    # state rows spread over 32 / 64 lanes: the reductions then use the gfx950 row swaps (emulated by the harness)
    ('cfg:rwkv7', '1,16,1,8,128', 'f32', 1, 'L=32,C=4,R=1,W=1'),
    ('cfg:rwkv7', '1,16,1,8,128', 'f32', 0, 'L=64,C=2,R=1,W=1'),
    # several gradient-kernel instances per wave as consecutive row slices of one chunk (narrow states): ragged slices,
    # a slice with no row, a partial last chunk; their gradients are summed across the wave before one instance stores
    ('cfg:mamba1', '2,21,2,37,16', 'f32', 0, 'MS=8'),
    ('gla', '2,19,2,21,32', 'f32', 1, 'MS=2'),
    # knobs of the row kernels: branch-free stores of the row sums in both kernels, deeper unrolling
    ('cfg:rwkv7', '1,19,1,128,128', 'bf16', 0, 'NB=3,UR=4'),
    ('cfg:mamba2', '1,21,2,64,128', 'f32', 1, 'NB=0'),
    ('cfg:mamba1', '2,16,2,128,16', 'f32', 1, 'NB=3,UR=16'),
    # results leave LDS one chunk later (double-buffered staging, checkpoints stored after the staging wait): partial last
    # chunk, a single chunk, a single timestep, reverse scan with state recompute, vector state, padded width
    ('cfg:rwkv7', '1,37,1,128,128', 'f32', 0, 'DF=1'),
    ('cfg:rwkv7', '1,37,2,16,16', 'bf16', 1, 'DF=1,TS=4,DT=4'),
    ('cfg:mamba1', '2,13,2,128,16', 'f32', 1, 'DF=1'),
    ('cfg:mamba2', '1,21,2,64,128', 'bf16', 0, 'DF=1,NB=3'),
    ('cfg:gated_delta_rule', '1,1,2,128,128', 'bf16', 1, 'DF=1'),
    ('cfg:gated_delta_rule', '1,9,1,16,80', 'f32', 0, 'DF=1'),
    ('cfg:gated_delta_rule', '1,68,1,128,128', 'bf16', 1, 'DF=1,NB=0'),
    ('rwkv4', '2,11,1,32,1', 'f32', 0, 'DF=1'),
    ('s4d', '2,8,1,8,6', 'f32', 1, 'DF=1'),
    # a block's row sums kept in registers and stored once: groups of 64, 16 and 8 lanes (one and two kept steps per lane),
    # partial last block, double-buffered results, the reverse scan with state recompute, padded width, a tile that cannot
    ('cfg:rwkv7', '1,37,1,128,128', 'f32', 0, 'KS=3'),
    ('cfg:rwkv7', '1,19,2,128,128', 'bf16', 1, 'KS=3,L=8,C=16,R=2,W=8,R1=2,W1=8'),
    ('cfg:mamba2', '1,21,2,64,128', 'bf16', 1, 'KS=3,DF=1,L=16,C=8'),
    ('cfg:gated_delta_rule', '1,9,1,16,80', 'f32', 0, 'KS=3,L=16,C=8'),
    ('cfg:mamba1', '2,13,2,128,16', 'f32', 1, 'KS=3,L=8,C=2'),
    ('cfg:mamba1', '2,13,2,128,16', 'f32', 0, 'KS=3'),
    ('mlstm_gates', '2,11,2,16,1', 'f32', 1, 'KS=3'),
]


@pytest.mark.parametrize('case,dims,dtype,end,tile', TILED)
def test_tile_overrides(case, dims, dtype, end, tile):
    # (these runs also take the gradient kernel's two-rows-in-flight variant)
    env = dict(os.environ, FLEX_RNN_TILE=tile, HIPSIM_PREFETCH='2')
    r = subprocess.run([sys.executable, RUNNER, case, dims, dtype, str(end)], capture_output=True, text=True, timeout=900, env=env)
    assert r.returncode == 0, f'rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-3000:]}'
    assert tile.split(',')[0] in r.stdout.replace(' ', '')


# The hardened harness: threads of a workgroup resumed in a fresh random order in every barrier phase and workgroups
# shuffled (a missing barrier, a read of LDS before its write or a dependence on the order of workgroups then shows
# for some seed), LDS poisoned with NaNs at the start of every workgroup, every uninitialised local variable a NaN
# pattern, array-bounds checks on registers and LDS, guard regions of 1 GiB around every tensor, the product's launch
# audit on.  The first rows are the shape of the one GPU memory fault on record (bf16, a partial last chunk, row inputs
# shared over heads), with default knobs and with the deferred flush; `all` runs every candidate build the first call
# would time on a GPU through the product's own choice logic (`CompiledPlan._tune` / `_select`).
HARDENED = [
    ('cfg:mamba2', '2,19,4,64,128', 'bf16', 1, '', 1, False),
    ('cfg:mamba2', '2,19,4,64,128', 'bf16', 0, 'DF=1', 2, False),
    ('cfg:mamba2', '2,19,2,16,128', 'bf16', 1, 'DF=1', 3, True),
    ('cfg:mamba2', '2,19,2,16,128', 'bf16', 0, '', 4, True),
    ('cfg:rwkv7', '1,21,1,32,128', 'bf16', 1, '', 5, False),
    ('cfg:mamba1', '2,13,2,64,16', 'f32', 0, '', 6, False),
    ('cfg:gated_delta_rule', '1,19,2,32,128', 'bf16', 1, 'DF=1', 7, False),
    # traced layers at two waves per gradient-kernel instance: sums inside preparation and epilogue kept in LDS,
    # raw projections loaded where they are used
    ('layer+:gated_delta_rule', '1,19,1,128,128', 'bf16', 1, '', 8, False),
    ('layer:mamba2', '1,19,2,128,128', 'bf16', 0, '', 9, False),
]


@pytest.mark.parametrize('case,dims,dtype,end,tile,seed,every', HARDENED)
def test_hardened_harness(case, dims, dtype, end, tile, seed, every):
    env = dict(os.environ, FLEX_RNN_TILE=tile, HIPSIM_SEED=str(seed), HIPSIM_UNINIT='1', HIPSIM_BOUNDS='1',
               HIPSIM_CANDIDATES='1' if every else '0', FLEX_RNN_CHECK='1')
    r = subprocess.run([sys.executable, RUNNER, case, dims, dtype, str(end)], capture_output=True, text=True, timeout=1500, env=env)
    assert r.returncode == 0, f'rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-3000:]}'
    if every:
        assert 'frnn_fw#1' in r.stdout and 'frnn_bw1#1' in r.stdout and 'frnn_bw2#1' in r.stdout, r.stdout[-600:]


@pytest.mark.parametrize('case,dims', [('rwkv7', '3,32,2,16,16'), ('cfg:mamba1', '2,16,4,32,16')])
def test_more_batch_head_pairs_than_grid_y_allows(case, dims):
    """The gradient kernel then carries both block indices in grid x (limit lowered to 3 so that small sizes reach it)."""
    env = dict(os.environ, FLEX_RNN_MAX_GRID_Y='3')
    r = subprocess.run([sys.executable, RUNNER, case, dims, 'f32', '1'], capture_output=True, text=True, timeout=900, env=env)
    assert r.returncode == 0, f'rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-3000:]}'


def _random_pattern_case(seed):
    """A gated linear-attention step whose five inputs get random classes-compatible broadcast
    patterns over (B, T, H); returns the argument string of run_case.py's `pattern:` mode."""
    import random
    rnd = random.Random(seed)
    spans = []
    for cls in ('row', 'row', 'col', 'row', 'scalar'):
        sp = ''.join(d for d in 'BTH' if rnd.random() < 0.7)
        spans.append(f'{cls}:{sp}')
    # at least one input must span each of B, T, H (the state fixes B and H; T comes from the inputs)
    spans[0] = 'row:BTH'
    return 'pattern:' + ','.join(spans)


@pytest.mark.parametrize('seed', range(4))
def test_random_broadcast_patterns(seed):
    case = _random_pattern_case(seed)
    r = subprocess.run([sys.executable, RUNNER, case, '2,8,3,8,16', 'f32', str(seed % 2)], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, f'{case}\nrc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-3000:]}'


@pytest.mark.parametrize('seed', cases.FUZZ_SEEDS)
def test_random_recurrences(seed):
    """Random step functions (tests/cases.py: random_step) through the emitted kernels."""
    dims = ','.join(str(d) for d in cases.FUZZ_DIMS[seed % 6])
    r = subprocess.run([sys.executable, RUNNER, f'gen:{seed}', dims, 'f32', str(seed % 2), '1e-4'], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, f'rc={r.returncode}\n{r.stdout[-2500:]}\n{r.stderr[-3000:]}'


@pytest.mark.parametrize('dims', [(0, 16, 2, 16, 16), (2, 0, 2, 16, 16)])
def test_empty_batch_and_empty_time(dims):
    """No batch entries or no timesteps: nothing is launched, the state and its gradient pass
    through, outputs and per-step gradients are empty, gradients of broadcast inputs zero."""
    import torch as th
    from flex_rnn_amd import planner
    from hipsim import SimPlan
    step, xs, ss = cases.make_inputs('mamba', *dims, dtype=th.float32)
    ss = [th.randn(s.shape) for s in ss]
    plan, fm, bm = planner.make_plan(step, xs, ss)
    nout, nst = plan.part.noutputs, plan.part.nstates
    sp = SimPlan(plan, state_meta=fm[nout:nout + nst])
    res = sp.forward(tuple(xs), tuple(ss))
    outs, stT, sck, aux = res[:nout], res[nout:nout + nst], res[nout + nst:nout + 2 * nst], res[-1]
    assert [tuple(r.shape) for r in res] == [tuple(sh) for sh, _, _ in fm]
    assert all(th.equal(a, b) for a, b in zip(stT, ss)) and all(o.numel() == 0 for o in outs)
    lean = sp.forward_only(tuple(xs), tuple(ss))
    assert all(th.equal(a, b) for a, b in zip(lean[nout:], ss))
    dS = [th.randn(s.shape) for s in ss]
    dins, dst0 = sp.backward(tuple(th.zeros_like(o) for o in outs), tuple(dS), tuple(xs), sck, aux)
    assert all(th.equal(a, b) for a, b in zip(dst0, dS))
    assert all(d.shape == x.shape and not d.any() for d, x in zip(dins, xs))
