"""Random sweeps of the CPU harness (a development tool; the committed test cases are in tests/test_emit_sim.py).

    python tests/hipsim/sweep.py <kind> <first seed> <last seed + 1> [workers]

kinds: `gen` random recurrences, `ops` the named recurrences, `cfg` the benchmark recurrences with random row splits,
`tiles` the candidate tiles that the first-call timing would run, `pat` random broadcast patterns.  Every case runs
tests/hipsim/run_case.py in a process of its own at a random (often odd) shape and dtype, guard pages at alternating ends
of every tensor, bounds checks on every register and LDS array; a line per case, failures with the end of their output.
A random recurrence can explode and overflow fp16: such a failure names a non-finite relative error.
"""
import os
import random
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
VEC = ['hgrn', 'rwkv4', 'mlstm_gates']
FULL = ['rwkv7', 'rwkv7_decay', 'rwkv6', 'gla', 'retention', 'delta_rule', 'delta_rule_fused', 'gated_delta_rule', 'mamba2',
        'mamba', 'longhorn', 's4d', 'gsa_slot', 'mlstm_norm', 'mlstm_cell']
CFG = ['mamba2', 'gated_delta_rule', 'rwkv7', 'mamba1', 'delta_rule']
KNOBS = ['DF=1', 'NB=3', 'NB=0', 'UR=4', 'DF=1,NB=3', 'WN=2']


def case(kind, seed):
    """(run_case.py arguments, environment additions) of case `seed`."""
    r = random.Random(f'{kind}{seed}')
    env = {'HIPSIM_PREFETCH': r.choice(['2', '4'])}
    B, H = r.choice([1, 2, 3]), r.choice([1, 2, 3, 5])
    T = r.choice([1, 2, 5, 16, 17, 19, 33, 35])
    dt = r.choice(['f32', 'f32', 'bf16', 'f16'])
    if kind == 'gen':
        M, N = r.choice([1, 4, 7, 16, 21, 32, 64]), r.choice([1, 4, 6, 16, 24, 32, 64, 80, 128])
        name = f'gen:{seed}'
    elif kind == 'ops':
        name = r.choice(FULL + VEC)
        M, N = r.choice([1, 2, 5, 12, 20, 24, 33, 64, 100]), (1 if name in VEC else r.choice([2, 3, 8, 12, 24, 48, 64, 96, 128]))
        dt = r.choice(['f32', 'f32', 'bf16'])
    elif kind in ('cfg', 'tiles'):
        wl = r.choice(CFG)
        name = f'cfg:{wl}'
        M, N = r.choice([8, 16, 24, 64, 128]), (r.choice([8, 16, 32]) if wl == 'mamba1' else r.choice([16, 32, 64, 128]))
        dt = r.choice(['f32', 'bf16', 'bf16', 'f16'] if kind == 'cfg' else ['f32', 'bf16'])
    elif kind == 'pat':
        spans = [f"{c}:{''.join(d for d in 'BTH' if r.random() < 0.6)}" for c in ('row', 'row', 'col', 'row', 'scalar')]
        spans[0] = 'row:BTH'
        name = 'pattern:' + ','.join(spans)
        M, N = r.choice([1, 5, 8, 24, 64]), r.choice([4, 12, 16, 48, 64, 128])
        if r.random() < 0.3:
            env['FLEX_RNN_MAX_GRID_Y'] = '3'
    else:
        raise SystemExit(__doc__)
    tile = []
    if kind == 'tiles':
        sys.path.insert(0, ROOT)
        import torch as th
        from flex_rnn_amd import launch, prebuild
        plan = prebuild.plan_for(name[4:], (B, T, H, M, N), {'f32': th.float32, 'bf16': th.bfloat16}[dt])
        tf, tr = r.choice(launch.row_kernel_tiles(plan, False)), r.choice(launch.row_kernel_tiles(plan, True))
        if tf[:2] != tr[:2]:            # (both kernels share the columns per lane)
            tr = (tf[0], tf[1], tr[2], tr[3]) if plan.part.dstep_needs_state else tf
        tile.append(f'L={tf[0]},C={tf[1]},R={tf[2]},W={tf[3]},R1={tr[2]},W1={tr[3]}')
    elif kind in ('cfg', 'pat', 'ops') and r.random() < 0.5:
        tile.append('MS=%d' % r.choice([2, 4, 8] if kind != 'cfg' else [1, 2, 4, 8, 16]))
    if kind != 'ops' and r.random() < 0.3:
        tile.append(r.choice(KNOBS))
    if tile:
        env['FLEX_RNN_TILE'] = ','.join(tile)
    return [name, f'{B},{T},{H},{M},{N}', dt, str(seed & 1)], env


def run(job):
    kind, seed = job
    args, extra = case(kind, seed)
    env = dict(os.environ, HIPSIM_BOUNDS='1', PYTHONPATH=ROOT, **extra)
    r = subprocess.run([sys.executable, os.path.join(HERE, 'run_case.py'), *args], cwd=ROOT, env=env, capture_output=True,
                       text=True, timeout=1800)
    return seed, r.returncode, ' '.join(args), extra, (r.stdout + r.stderr).strip().splitlines()[-3:]


def main():
    if len(sys.argv) < 4:
        raise SystemExit(__doc__)
    kind, lo, hi = sys.argv[1], int(sys.argv[2]), int(sys.argv[3])
    workers = int(sys.argv[4]) if len(sys.argv) > 4 else 4
    bad = 0
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for seed, rc, what, extra, tail in pool.map(run, [(kind, s) for s in range(lo, hi)]):
            bad += rc != 0
            print('ok  ' if rc == 0 else f'FAIL rc={rc}', seed, what, extra, '' if rc == 0 else tail, flush=True)
    print(f'{hi - lo - bad} of {hi - lo} passed')
    return 1 if bad else 0


if __name__ == '__main__':
    sys.exit(main())
