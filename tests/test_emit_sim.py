"""Runs the emitted HIP kernels on the CPU (tests/hipsim) and compares forward results and all
gradients with the oracle.  Every buffer of every launch sits against a guard page, at its end
in one run and at its start in another, so an out-of-bounds index of a generated kernel fails
the test with a signal."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
RUNNER = os.path.join(HERE, 'hipsim', 'run_case.py')

# (case, B,T,H,M,N, dtype, guard at end?)
RUNS = [
    ('cfg:delta_rule', '1,64,2,16,16', 'f32', 1),
    ('cfg:delta_rule', '1,64,2,16,16', 'f32', 0),
    ('cfg:mamba1', '2,16,2,128,16', 'f32', 1),      # reverse scan with state recompute, matrix grads, atomics
    ('cfg:mamba1', '2,16,2,128,16', 'f32', 0),
    ('cfg:mamba2', '2,16,2,64,128', 'bf16', 1),     # scalar inputs, head-broadcast rows
    ('cfg:rwkv7', '1,16,2,128,128', 'bf16', 1),
    ('cfg:rwkv7', '1,16,2,128,128', 'f32', 0),
    ('cfg:gated_delta_rule', '1,16,2,128,128', 'bf16', 1),
    ('rwkv6', '2,8,2,16,16', 'f32', 1),             # time-independent row input
    ('s4d', '2,8,1,8,16', 'f32', 1),                # two states, four matrix inputs
    ('longhorn', '2,8,2,16,8', 'f32', 0),           # row-only forward sum
    ('retention', '1,8,2,8,32', 'f16', 1),
    ('mlstm_cell', '1,8,2,8,8', 'bf16', 1),
    ('hgrn', '2,8,1,64,1', 'f32', 1),               # vector state (N = 1)
    ('rwkv4', '2,8,1,32,1', 'f32', 0),              # three states, comparisons
    ('mlstm_gates', '2,8,2,16,1', 'f32', 1),        # three outputs
    # sequence lengths that are not a multiple of the chunk (partial last chunk), and T = 1
    ('cfg:rwkv7', '1,37,2,128,128', 'f32', 0),
    ('cfg:mamba1', '2,13,2,128,16', 'f32', 1),
    ('cfg:mamba2', '2,21,2,64,128', 'bf16', 0),
    ('rwkv4', '2,11,1,32,1', 'f32', 0),
    ('cfg:gated_delta_rule', '1,1,2,128,128', 'bf16', 1),
]


@pytest.mark.parametrize('case,dims,dtype,end', RUNS)
def test_emitted_kernels_on_cpu(case, dims, dtype, end):
    r = subprocess.run([sys.executable, RUNNER, case, dims, dtype, str(end)], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, f'rc={r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-3000:]}'
