"""Writes tests/golden/five_configs_fp64.npz: inputs, upstream gradients and the oracle's fp64
results (outputs, final states, all gradients) for the five benchmark recurrences at tiny
shapes.  The reference ships no golden vectors for this path and none of its code is run
here; these vectors come from oracle/recurrence.py (itself pinned by closed forms and
invariants in tests/test_oracle.py) and serve as a fixed point: a later edit of the oracle, of
the input generators or of a step function that changes any number shows up against them.

    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch as th

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from flex_rnn_amd import configs  # noqa: E402
from oracle import recurrence  # noqa: E402

SHAPES = {'delta_rule': (1, 6, 2, 4, 4), 'mamba1': (2, 6, 2, 4, 4), 'mamba2': (2, 6, 2, 4, 8),
          'rwkv7': (2, 6, 2, 4, 8), 'gated_delta_rule': (2, 6, 2, 4, 8)}


def vectors(name):
    wl = configs.make(name, dims=SHAPES[name], dtype=th.float64, seed=7)
    g = th.Generator().manual_seed(11)
    outs, _ = recurrence.run_loop(wl.step, wl.inputs, wl.states)
    dy = [th.randn(o.shape, generator=g, dtype=th.float64) for o in outs]
    dS = [th.randn(s.shape, generator=g, dtype=th.float64) for s in wl.states]
    res = recurrence.loop_with_grads(wl.step, wl.inputs, wl.states, dy, dS)
    out = {}
    for key, ts in (('in', wl.inputs), ('st', wl.states), ('dy', dy), ('dS', dS), ('out', res[0]), ('stT', res[1]),
                    ('din', res[2]), ('dst', res[3])):
        for i, t in enumerate(ts):
            out[f'{name}.{key}{i}'] = t.detach().numpy()
    return out


if __name__ == '__main__':
    data = {}
    for name in SHAPES:
        data.update(vectors(name))
    np.savez_compressed(os.path.join(HERE, 'five_configs_fp64.npz'), **data)
    print(len(data), 'arrays written')
