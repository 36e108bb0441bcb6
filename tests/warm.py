"""Kernel-cache warm-up for the shapes only the GPU tests use (called by __graft_entry__.build() after the
package's own `flex_rnn_amd.prebuild.warm`; needs no GPU)."""
import os
import sys

import torch as th

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

import cases  # noqa: E402
from flex_rnn_amd import configs, planner, prebuild  # noqa: E402
from flex_rnn_amd.launch import compile_plans  # noqa: E402

OTHER = [('rwkv6', (2, 32, 2, 32, 32)), ('s4d', (2, 32, 1, 16, 32)), ('longhorn', (2, 32, 2, 32, 16)),
         ('hgrn', (2, 64, 1, 256, 1)), ('rwkv4', (2, 32, 1, 64, 1)), ('mlstm_gates', (2, 32, 2, 32, 1)),
         ('retention', (1, 32, 2, 16, 64)), ('mlstm_cell', (1, 32, 2, 32, 32)), ('gla', (1, 16, 1, 16, 16)),
         ('gla', (1, 32, 1, 16, 16)), ('delta_rule', (2, 32, 2, 16, 16)), ('gated_delta_rule', (2, 32, 2, 16, 16)),
         ('zoo', (2, 32, 2, 32, 32)), ('zoo2', (2, 32, 2, 32, 32)), ('gla', (2, 32, 2, 100, 32)),
         ('gla', (1, 16, 2, 16, 16)), ('gla', (3, 50, 2, 16, 16)), ('gla', (2, 33, 2, 16, 16)),
         ('rwkv7', (2, 32, 2, 64, 64)), ('delta_rule_fused', (2, 32, 2, 32, 32)),
         ('rwkv7', (2, 32, 2, 64, 96)), ('mamba', (2, 32, 2, 32, 12)), ('gla', (1, 32, 2, 16, 160))]


# two helper kernels of the test of the launch entry point that allocates nothing: they copy floats out of, and
# add 1 to floats of, a buffer whose address only the runtime library knows
NO_ALLOC_PROBE = r'''
#include <hip/hip_runtime.h>
struct Args { const float* src; float* dst; long long n; };
extern "C" __global__ void probe_copy(Args A) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < A.n; i += (long long)gridDim.x * blockDim.x) A.dst[i] = A.src[i];
}
struct Args1 { float* p; long long n; };
extern "C" __global__ void probe_add_one(Args1 A) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < A.n; i += (long long)gridDim.x * blockDim.x) A.p[i] += 1.0f;
}
'''

NO_ALLOC_DIMS = [('rwkv7', (2, 64, 2, 128, 128)), ('rwkv7', (1, 32, 2, 128, 128))]


def no_alloc_tile(name, dims):
    """The heuristic tile of a workload without row splitting in the gradient kernel (results are then free of
    atomic accumulation and can be compared bit for bit)."""
    import dataclasses
    return dataclasses.replace(prebuild.plan_for(name, dims).tile, MS=1)


# row-kernel code-generation knobs that the size of the test shapes would not make candidates (tests/test_gpu_full.py)
KNOB_CASES = [('rwkv7', (2, 37, 2, 64, 64), 'DF=1,NB=3,UR=4'), ('mamba1', (2, 45, 4, 128, 16), 'DF=1,NB=3'),
              # a block's row sums kept in registers, two kept steps per lane (groups of 8 lanes)
              ('gated_delta_rule', (2, 37, 2, 128, 128), 'KS=3,L=8,C=16')]


# tests/test_gpu_full.py::test_segmented_call_against_oracle: sequences walked SEGMENT timesteps at a time
SEGMENT = 32
SEGMENTED_CASES = [('gated_delta_rule', (2, 77, 2, 128, 128)), ('mamba1', (2, 45, 4, 128, 16))]


EXAMPLE_ARGS, LAYER_CASES, example_plans = prebuild.EXAMPLE_ARGS, prebuild.LAYER_CASES, prebuild.example_plans


GOLDEN = {'delta_rule': (1, 6, 2, 4, 4), 'mamba1': (2, 6, 2, 4, 4), 'mamba2': (2, 6, 2, 4, 8),
          'rwkv7': (2, 6, 2, 4, 8), 'gated_delta_rule': (2, 6, 2, 4, 8)}      # tests/golden/make_vectors.py


def warm(force=False, seen=None):
    from flex_rnn_amd import runtime
    runtime.compile_kernel('probe', NO_ALLOC_PROBE, force=force)
    plans = []          # (the example layers' kernels are built by flex_rnn_amd.prebuild.warm(examples=True))
    for name, dims, knobs in KNOB_CASES:
        old = os.environ.get('FLEX_RNN_TILE')
        os.environ['FLEX_RNN_TILE'] = knobs
        try:
            plans.append(prebuild.plan_for(name, dims))
        finally:
            os.environ.pop('FLEX_RNN_TILE') if old is None else os.environ.__setitem__('FLEX_RNN_TILE', old)
    for name, (B, T, H, M, N) in SEGMENTED_CASES:
        for seg in sorted({min(SEGMENT, T), T % SEGMENT} - {0}):
            plans.append(prebuild.plan_for(name, (B, seg, H, M, N)))
    for name, dims in NO_ALLOC_DIMS:
        plans.append(prebuild.plan_for(name, dims, tile=no_alloc_tile(name, dims)))
    for name, dims in OTHER:
        step, xs, ss = cases.make_inputs(name, *dims, dtype=th.float32)
        plan = planner.make_plan(step, [x.to('meta') for x in xs], [s.to('meta') for s in ss])[0]
        plans.append(plan)
    for dtype in (th.float16, th.float64):
        step, xs, ss = cases.make_inputs('gla', 2, 32, 2, 32, 32, dtype=dtype)
        plan = planner.make_plan(step, [x.to('meta') for x in xs], [s.to('meta') for s in ss])[0]
        plans.append(plan)
    for name in ('mamba_bh', 'matgain'):                # a single timestep with a full matrix input, bf16
        step, xs, ss = cases.make_inputs(name, 2, 1, 2, 16, 16, dtype=th.bfloat16)
        plans.append(planner.make_plan(step, [x.to('meta') for x in xs], [s.to('meta') for s in ss])[0])
    step, xs, ss = cases.make_inputs('gla', 2, 16, 2, 16, 16, dtype=th.float32)      # state dtype / layout variants
    for s0 in (ss[0], ss[0].to(th.bfloat16), ss[0].transpose(-1, -2).contiguous().transpose(-1, -2)):
        plans.append(planner.make_plan(step, [x.to('meta') for x in xs], [s0.to('meta')])[0])
    for seed in cases.FUZZ_SEEDS:                       # tests/test_gpu_fuzz.py
        step, xs, ss = cases.fuzz_case(seed, (th.float32, th.bfloat16)[(seed // 6) % 2])
        plan = planner.make_plan(step, [x.to('meta') for x in xs], [s.to('meta') for s in ss])[0]
        plans.append(plan)
    for name, dims in GOLDEN.items():
        plans.append(prebuild.plan_for(name, dims, th.float32))
    plans.append(prebuild.plan_for('rwkv7', (8, 512, 32, 128, 128)))
    plans.append(prebuild.plan_for('mamba2', (2, 64, 4, 64, 128)))
    for name in ('rwkv7', 'mamba1', 'mamba2'):
        B, T, H, M, N = configs.DEFAULT_DIMS[name]
        plans.append(prebuild.plan_for(name, (2, 77, 2, M, N)))
    for name, dims in [('rwkv7', (2, 77, 2, 128, 128)), ('mamba1', (2, 45, 4, 128, 16)),
                       ('gated_delta_rule', (2, 1, 2, 128, 128)), ('mamba2', (2, 19, 4, 64, 128))]:
        plans.append(prebuild.plan_for(name, dims, th.float32))
    return compile_plans(plans, force=force, seen=seen)
