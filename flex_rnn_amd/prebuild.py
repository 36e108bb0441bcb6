"""Ahead-of-time kernel cache warm-up.

Kernels are normally compiled on the first call of a `jit` object; `warm()` runs the
same planner + emitter + hipcc step for a list of workloads without a GPU, so that a
machine without a compiler in the loop (or a test run) finds every code object in the
cache.  `CASES` lists the workloads the test-suite, the smoke test and the benchmark use.
"""
from __future__ import annotations

from concurrent.futures import ThreadPoolExecutor
from typing import Iterable, List, Optional, Tuple

import torch as th

from . import configs, planner
from .launch import compile_plan

# (workload name, (B, T, H, M, N) or None for the full benchmark size, dtype or None)
CASES: List[Tuple[str, Optional[tuple], Optional[th.dtype]]] = [
    # reduced sizes used by the parity tests (same M, N as the full configurations)
    ('delta_rule', None, None),
    ('mamba1', (2, 64, 4, 128, 16), None),
    ('mamba2', (2, 64, 4, 64, 128), None),
    ('rwkv7', (2, 64, 2, 128, 128), None),
    ('rwkv7', (2, 64, 2, 128, 128), th.float32),
    ('gated_delta_rule', (2, 128, 2, 128, 128), None),
    # full benchmark sizes
    ('mamba1', None, None),
    ('mamba2', None, None),
    ('rwkv7', None, None),
    ('gated_delta_rule', None, None),
]


def plan_for(name: str, dims=None, dtype=None, tile=None):
    """Plan for a named workload built from meta tensors only (no data is generated)."""
    dims = dims or configs.DEFAULT_DIMS[name]
    small = configs.make(name, dims=(1, 1, 1, dims[3], dims[4]), dtype=dtype)
    B, T, H, M, N = dims
    full = (B, T, H, M, N)
    ins = []
    for x in small.inputs:
        shape = tuple(full[j] if (x.shape[j] != 1 or _is_full(name, len(ins), j)) else 1 for j in range(5))
        ins.append(th.empty(shape, dtype=x.dtype, device='meta'))
    sts = [th.empty((B, H, M, N), dtype=s.dtype, device='meta') for s in small.states]
    return planner.make_plan(small.step, ins, sts, tile)[0]


# which of (B, T, H) each input of each workload spans (inputs built at B=T=H=1 lose that information)
_SPANS = {
    'delta_rule': ['BTH'] * 4,
    'mamba1': ['BTH', 'BTH', 'H', 'BT', 'BT'],
    'mamba2': ['BTH', 'BTH', 'H', 'BT', 'BT'],
    'rwkv7': ['BTH'] * 6,
    'gated_delta_rule': ['BTH'] * 5,
}


def _is_full(name: str, i: int, j: int) -> bool:
    return j < 3 and 'BTH'[j] in _SPANS[name][i]


EXAMPLE_ARGS = dict(B=2, T=64, D=256, C=128)      # the size the example layers are checked at (`python -m flex_rnn_amd.examples --check-flex`, tests)


def _layer_cases():
    from flex_rnn_amd import examples
    norm = ('rwkv7', 'delta_rule', 'gated_delta_rule')
    return [(op, False, th.float32, False) for op in examples.OPS] + \
           [(op, True, dt, False) for op in examples.RAW_OPS for dt in (th.float32, th.bfloat16)] + \
           [(op, True, dt, True) for op in norm for dt in (th.float32, th.bfloat16)]


# the example layers as `flex_rnn_amd.layer` traces them: (op, raw projections?, dtype, norms moved into the step too?)
LAYER_CASES = _layer_cases()


def example_plans():
    """Dry-runs every example layer on meta tensors and returns the plans its jit objects request."""
    import sys
    import flex_rnn_amd
    jit_mod = sys.modules['flex_rnn_amd.jit']        # (the package attribute `jit` is the class)
    from flex_rnn_amd import examples
    plans = []
    orig = jit_mod.build_twopass

    def capture(step, inputs, state, dryrun=False, tile=None):
        metas = [t.to('meta') for t in inputs], [t.to('meta') for t in state]
        plans.append(planner.make_plan(step, *metas, tile)[0])
        return orig(step, inputs, state, dryrun=True, tile=tile)

    jit_mod.build_twopass = capture
    try:
        for op in examples.OPS:
            a = EXAMPLE_ARGS
            inputs, layer, steps = examples.build(op, a['B'], a['T'], a['D'], a['C'], 'meta')
            layer(*inputs)
        # the same layers traced by `flex_rnn_amd.layer` (plans of the fused steps included)
        for op, raw, dtype, reductions in LAYER_CASES:
            inputs, layer, steps = examples.build(op, a['B'], a['T'], a['D'], a['C'], 'meta', raw=raw)
            flex_rnn_amd.layer(layer, reductions=reductions).graph(*[i.to(dtype) for i in inputs])
    finally:
        jit_mod.build_twopass = orig
    return plans


def warm(cases: Iterable = CASES, verbose: bool = False, force: bool = False, examples: bool = False) -> int:
    """Compiles the kernels of `cases`; with `examples` also those of the example layers (eager adapters and traced
    layers) at `EXAMPLE_ARGS`."""
    cases = list(cases)
    plans = [plan_for(name, dims, dtype) for name, dims, dtype in cases]       # (tracing: one at a time)
    if examples:
        extra = example_plans()
        cases += [('example layer', (pl.B, pl.T, pl.H, pl.M, pl.N), None) for pl in extra]
        plans += extra
    seen = set()
    n = 0
    with ThreadPoolExecutor(max_workers=3) as pool:
        built = pool.map(lambda pl: compile_plan(pl, force=force, seen=seen), plans)
        for (name, dims, dtype), specs in zip(cases, built):
            for spec, path in specs:
                n += 1
                if verbose:
                    print(f'  {name} {dims or "full"} {spec.name}: {path}')
    return n
