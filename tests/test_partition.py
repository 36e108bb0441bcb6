"""The graph partition (fw / restep / dstep / drow / epilogue with aux, daux and row-axis
accumulation), executed on the CPU by oracle/plan_exec.py, must reproduce autograd of the
plain loop for every example recurrence."""
import pytest
import torch as th

from flex_rnn_amd import planner
from oracle import plan_exec, recurrence

import cases


def _check(name, B, T, H, M, N, DT):
    step, xs, ss = cases.make_inputs(name, B, T, H, M, N)
    plan, _, _ = planner.make_plan(step, xs, ss)
    g = th.Generator().manual_seed(5)
    want = recurrence.run_loop(step, xs, ss)
    dy = [th.randn(o.shape, generator=g, dtype=th.float64) for o in want[0]]
    dS = [th.randn(s.shape, generator=g, dtype=th.float64) for s in ss]
    want = recurrence.loop_with_grads(step, xs, ss, dy, dS)
    got = plan_exec.run_plan(plan.part, xs, ss, dy, dS, DT=DT)
    for a, b in zip(got, want):
        for x, y in zip(a, b):
            assert x.shape == y.shape
            assert recurrence.rel_err(x, y) < 1e-10, name
    return plan


@pytest.mark.parametrize('name', sorted(cases.CASES))
def test_partition_matches_autograd(name):
    _check(name, 2, 8, 2, 4, 8, DT=4)


@pytest.mark.parametrize('name', sorted(cases.VECTOR_CASES))
def test_partition_vector_state(name):
    _check(name, 2, 8, 2, 8, 1, DT=4)


@pytest.mark.parametrize('name,M,N', [('mlstm_gates', 1, 1), ('gla', 1, 8), ('delta_rule', 1, 4)])
def test_partition_single_row_state(name, M, N):
    _check(name, 2, 8, 2, M, N, DT=4)


@pytest.mark.parametrize('seed', range(30))
def test_partition_of_random_recurrences(seed):
    """Random step functions (tests/cases.py: random_step): whatever the partition accepts must
    reproduce autograd of the plain loop; a rejection must be a named PartitionError."""
    from flex_rnn_amd.partition import PartitionError
    step, spec, nst, src = cases.random_step(seed)
    table = {'gen': (step, spec, nst)}
    step, xs, ss = cases.make_inputs('gen', 2, 8, 2, 4, 8, table=table)
    try:
        plan, _, _ = planner.make_plan(step, xs, ss)
    except PartitionError:
        return
    g = th.Generator().manual_seed(5)
    out = recurrence.run_loop(step, xs, ss)
    dy = [th.randn(o.shape, generator=g, dtype=th.float64) for o in out[0]]
    dS = [th.randn(s_.shape, generator=g, dtype=th.float64) for s_ in ss]
    want = recurrence.loop_with_grads(step, xs, ss, dy, dS)
    got = plan_exec.run_plan(plan.part, xs, ss, dy, dS, DT=4)
    for a, b in zip(got, want):
        for x, y in zip(a, b):
            assert x.shape == y.shape and recurrence.rel_err(x, y) < 1e-9, src


def test_aux_daux_of_rwkv7():
    plan = _check('rwkv7_decay', 1, 4, 1, 4, 4, DT=2)
    p = plan.part
    assert len(p.aux) == 1 and len(p.daux) == 1          # (S a) and (G b): one saved row sum each way
    assert len(p.msums) == 5 and not p.dstep_needs_state  # dr, dw, dk, da, db accumulate over rows
    assert not any(n.op == 'sum' for n in p.restep.nodes + p.drow.nodes)


def test_mamba_needs_state_in_reverse_scan():
    plan = _check('mamba', 1, 4, 2, 4, 4, DT=2)
    assert plan.part.dstep_needs_state and plan.part.mat_idx == [2]


def test_forward_sum_over_rows_is_rejected():
    def bad(x, S):
        S = S + x
        return S.sum(-1, True), S * S.sum(0, True)
    x, S = th.randn(1, 2, 1, 1, 4), th.randn(1, 1, 4, 4)
    with pytest.raises(AssertionError, match='keepdim=True'):
        planner.make_plan(bad, [x], [S])
