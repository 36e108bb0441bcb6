"""Pins the CPU oracle (oracle/recurrence.py) with closed forms, brute force and invariants,
and checks the package's `jit.naive` against it."""
import pytest
import torch as th

import flex_rnn_amd
from flex_rnn_amd import ops
from oracle import recurrence

D = th.float64


def rnd(*shape, seed=0):
    return th.randn(*shape, generator=th.Generator().manual_seed(seed), dtype=D)


def test_decay_linear_attention_closed_form():
    # S_t = S_{t-1} * w_t + v_t k_t^T ;  y_t = S_t q_t
    B, T, H, M, N = 2, 9, 3, 4, 5
    q, k = rnd(B, T, H, 1, N, seed=1), rnd(B, T, H, 1, N, seed=2)
    v = rnd(B, T, H, M, 1, seed=3)
    w = th.sigmoid(rnd(B, T, H, 1, N, seed=4))
    S0 = rnd(B, H, M, N, seed=5)

    def step(q, k, v, w, S):
        S = S * w + v * k
        return (S * q).sum(-1, True), S

    (y,), (ST,) = recurrence.run_loop(step, [q, k, v, w], [S0])
    # closed form with explicit products (no shared code path with the loop)
    logw = th.log(w[:, :, :, 0])                       # [B,T,H,N]
    cum = th.cumsum(logw, dim=1)                       # prod_{r<=t} w_r
    y_ref = th.zeros(B, T, H, M, dtype=D)
    for t in range(T):
        acc = (S0 * th.exp(cum[:, t])[:, :, None, :] * q[:, t]).sum(-1)        # initial-state term
        for s in range(t + 1):
            decay = th.exp(cum[:, t] - cum[:, s])                              # prod_{s<r<=t} w_r
            dot = (q[:, t, :, 0] * k[:, s, :, 0] * decay).sum(-1)              # [B,H]
            acc = acc + v[:, s, :, :, 0] * dot[:, :, None]
        y_ref[:, t] = acc
    assert recurrence.rel_err(y, y_ref) < 1e-12
    ST_ref = S0 * th.exp(cum[:, -1])[:, :, None, :]
    for s in range(T):
        ST_ref = ST_ref + v[:, s] * (k[:, s] * th.exp(cum[:, -1] - cum[:, s])[:, :, None, :])
    assert recurrence.rel_err(ST, ST_ref) < 1e-12


def test_vector_state_scan_closed_form():
    # N = 1: s_t = exp(g_t) s_{t-1} + x_t
    B, T, M = 2, 11, 6
    x, g = rnd(B, T, 1, M, 1, seed=1), -th.sigmoid(rnd(B, T, 1, M, 1, seed=2))
    s0 = rnd(B, 1, M, 1, seed=3)
    (y,), (sT,) = recurrence.run_loop(ops.hgrn, [x, g], [s0])
    G = th.cumsum(g[:, :, 0, :, 0], dim=1)               # [B,T,M]
    ref = th.exp(G) * s0[:, 0, :, 0][:, None]
    for s in range(T):
        ref[:, s:] += th.exp(G[:, s:] - G[:, s:s + 1]) * x[:, s:s + 1, 0, :, 0]
    assert recurrence.rel_err(y[:, :, 0], ref) < 1e-12
    assert recurrence.rel_err(sT[:, 0, :, 0], ref[:, -1]) < 1e-12


def test_single_step_delta_rule_matrix_form():
    B, H, M, N = 2, 2, 3, 4
    q, k = rnd(B, 1, H, 1, N, seed=1), rnd(B, 1, H, 1, N, seed=2)
    v, beta = rnd(B, 1, H, M, 1, seed=3), th.sigmoid(rnd(B, 1, H, 1, 1, seed=4))
    S0 = rnd(B, H, M, N, seed=5)
    (y,), (S1,) = recurrence.run_loop(ops.delta_rule, [q, k, v, beta], [S0])
    kk = k[:, 0, :, 0]                                                    # [B,H,N]
    I = th.eye(N, dtype=D)
    P = I - beta[:, 0, :, 0, 0][:, :, None, None] * kk[..., :, None] * kk[..., None, :]
    ref = S0 @ P + beta[:, 0] * v[:, 0] * k[:, 0]
    assert recurrence.rel_err(S1, ref) < 1e-12
    assert recurrence.rel_err(y[:, 0], (ref @ q[:, 0, :, 0][..., None])[..., 0]) < 1e-12


def test_mamba_constant_inputs_geometric_series():
    B, T, H, M, N = 1, 13, 2, 3, 4
    delta, xval = 0.3, 0.7
    A = -th.arange(1, N + 1, dtype=D).view(1, 1, 1, 1, N).expand(1, 1, H, M, N).contiguous()
    x = th.full((B, T, H, M, 1), xval, dtype=D)
    dl = th.full((B, T, H, M, 1), delta, dtype=D)
    Bm, Cm = th.ones(B, T, 1, 1, N, dtype=D), th.ones(B, T, 1, 1, N, dtype=D)
    S0 = th.zeros(B, H, M, N, dtype=D)
    (y,), (ST,) = recurrence.run_loop(ops.mamba, [x, dl, A, Bm, Cm], [S0])
    r = th.exp(delta * A[0, 0])                                   # [H,M,N]
    ST_ref = delta * xval * (1 - r ** T) / (1 - r)
    assert recurrence.rel_err(ST[0], ST_ref) < 1e-12
    t = 5
    y_ref = (delta * xval * (1 - r ** (t + 1)) / (1 - r)).sum(-1)
    assert recurrence.rel_err(y[0, t], y_ref) < 1e-12


def _rwkv7_inputs(B, T, H, M, N, seed=0):
    r, k = rnd(B, T, H, 1, N, seed=seed), rnd(B, T, H, 1, N, seed=seed + 1)
    w = th.exp(-th.exp(rnd(B, T, H, 1, N, seed=seed + 2)))
    kk = th.nn.functional.normalize(rnd(B, T, H, 1, N, seed=seed + 3), dim=-1)
    a, b = -kk, kk * th.sigmoid(rnd(B, T, H, 1, N, seed=seed + 4))
    v = rnd(B, T, H, M, 1, seed=seed + 5)
    return [r, w, k, v, a, b], [rnd(B, H, M, N, seed=seed + 6)]


def test_invariants_permutation_chunking_broadcast():
    xs, ss = _rwkv7_inputs(3, 8, 2, 4, 4)
    (y,), (ST,) = recurrence.run_loop(ops.rwkv7_decay, xs, ss)
    perm = th.tensor([2, 0, 1])
    (yp,), (STp,) = recurrence.run_loop(ops.rwkv7_decay, [x[perm] for x in xs], [s[perm] for s in ss])
    assert th.equal(yp, y[perm]) and th.equal(STp, ST[perm])
    # chunked call with state hand-off
    (y1,), s1 = recurrence.run_loop(ops.rwkv7_decay, [x[:, :3] for x in xs], ss)
    (y2,), s2 = recurrence.run_loop(ops.rwkv7_decay, [x[:, 3:] for x in xs], s1)
    assert th.equal(th.cat([y1, y2], 1), y) and th.equal(s2[0], ST)
    # broadcast input == materialised input
    xb = list(xs)
    xb[1] = xs[1][:, :1, :1]                                    # decay shared over time and heads
    xm = list(xs)
    xm[1] = xb[1].expand(-1, 8, 2, -1, -1).contiguous()
    ob, om = recurrence.run_loop(ops.rwkv7_decay, xb, ss), recurrence.run_loop(ops.rwkv7_decay, xm, ss)
    assert th.equal(ob[0][0], om[0][0])


def test_gradients_against_finite_differences():
    xs, ss = _rwkv7_inputs(1, 3, 1, 2, 2, seed=7)
    dy, dS = rnd(1, 3, 1, 2, seed=20), rnd(1, 1, 2, 2, seed=21)
    _, _, dins, dst = recurrence.loop_with_grads(ops.rwkv7_decay, xs, ss, [dy], [dS])

    def loss(vals):
        (y,), (ST,) = recurrence.run_loop(ops.rwkv7_decay, vals[:6], vals[6:])
        return (y * dy).sum() + (ST * dS).sum()

    vals = [x.clone() for x in xs + ss]
    grads = dins + dst
    eps = 1e-6
    for i, g in enumerate(grads):
        flat = vals[i].view(-1)
        for j in range(0, flat.numel(), max(1, flat.numel() // 3)):
            old = flat[j].item()
            flat[j] = old + eps
            lp = loss(vals)
            flat[j] = old - eps
            lm = loss(vals)
            flat[j] = old
            fd = (lp - lm) / (2 * eps)
            assert abs(fd - g.reshape(-1)[j]) < 1e-6 * max(1.0, abs(fd)), (i, j, fd, g.reshape(-1)[j])


@pytest.mark.parametrize('dtype', [th.float32, th.bfloat16])
def test_package_naive_matches_oracle(dtype):
    xs, ss = _rwkv7_inputs(2, 6, 2, 4, 8)
    xs = [x.to(dtype) for x in xs]
    ss = [s.to(th.float32).mT.contiguous().mT for s in ss]         # non-contiguous state layout
    f = flex_rnn_amd.jit(ops.rwkv7_decay)
    y, ST = f.naive(*xs, *ss)
    (yo,), (STo,) = recurrence.run_loop(ops.rwkv7_decay, xs, ss, dtype=th.float32)
    assert y.dtype == yo.dtype == th.float32          # outputs come back in the loop dtype
    assert ST.dtype == ss[0].dtype and ST.stride() == ss[0].stride()
    assert recurrence.rel_err(y, yo) == 0 and recurrence.rel_err(ST, STo) == 0
    y64, _ = f.naive_fp64(*xs, *ss)
    assert y64.dtype == th.float64
    (y64o,), _ = recurrence.run_loop(ops.rwkv7_decay, xs, ss, dtype=th.float64)
    assert recurrence.rel_err(y64, y64o) == 0


@pytest.mark.parametrize('name', ['delta_rule', 'mamba1', 'mamba2', 'rwkv7', 'gated_delta_rule'])
def test_committed_vectors(name):
    """tests/golden/five_configs_fp64.npz (written by tests/golden/make_vectors.py from this oracle) is
    a fixed point: the oracle, the package's `naive` and the step functions still give those numbers."""
    import os
    import numpy as np
    import flex_rnn_amd
    from flex_rnn_amd import configs
    z = np.load(os.path.join(os.path.dirname(__file__), 'golden', 'five_configs_fp64.npz'))

    def arrs(key):
        out, i = [], 0
        while f'{name}.{key}{i}' in z:
            out.append(th.from_numpy(z[f'{name}.{key}{i}']))
            i += 1
        return out
    step = configs.make(name, dims=(1, 2, 1, 2, 2), dtype=th.float64).step
    xs, ss, dy, dS = arrs('in'), arrs('st'), arrs('dy'), arrs('dS')
    res = recurrence.loop_with_grads(step, xs, ss, dy, dS)
    for key, got in zip(('out', 'stT', 'din', 'dst'), res):
        for a, b in zip(got, arrs(key)):
            assert a.shape == b.shape and recurrence.rel_err(a, b) < 1e-12, (name, key)
    naive = flex_rnn_amd.jit(step).naive(*xs, *ss, dtype=th.float64)
    for a, b in zip(naive, arrs('out') + arrs('stT')):
        assert recurrence.rel_err(a, b) < 1e-12


# ------------------------------------------------------------------ the metric and the assertion
def test_rel_err_known_values():
    """||a - b|| / max(||b||, 1e-30) with b the trusted value (check_grad.py:20)."""
    import math
    a, b = th.tensor([3.0, 4.0]), th.tensor([0.0, 5.0])
    # a - b = (3, -1): sqrt(10) / 5.  (Squared norms would give 0.4, dividing by ||a|| the same 0.632 only
    # by accident of |a| = |b| = 5, which the next pair tells apart.)
    assert recurrence.rel_err(a, b) == pytest.approx(math.sqrt(10) / 5, rel=1e-15)
    a2, b2 = th.tensor([6.0, 8.0]), th.tensor([0.0, 5.0])
    assert recurrence.rel_err(a2, b2) == pytest.approx(math.sqrt(45) / 5, rel=1e-15)       # divided by ||b|| = 5 ...
    assert recurrence.rel_err(b2, a2) == pytest.approx(math.sqrt(45) / 10, rel=1e-15)      # ... not by ||a|| = 10
    # a zero reference: the 1e-30 floor, no division by zero
    assert recurrence.rel_err(th.zeros(4), th.zeros(4)) == 0.0
    assert recurrence.rel_err(th.tensor([2e-30, 0.0]), th.zeros(2)) == pytest.approx(2.0, rel=1e-6)
    # identical tensors of any dtype and shape
    x = th.randn(3, 5, dtype=th.bfloat16)
    assert recurrence.rel_err(x, x) == 0.0
    # operands are promoted to double before subtracting: 1 + 2^-10 is not a bf16 number (nearest: 1), so
    # a bf16 subtraction of the promoted-late kind would see no difference at all
    one = th.ones(1, dtype=th.bfloat16)
    assert recurrence.rel_err(one, th.tensor([1.0 + 2.0 ** -10], dtype=D)) == pytest.approx(2.0 ** -10 / (1 + 2.0 ** -10), rel=1e-12)
    # and a difference far below float32 resolution survives (no .float() on the way)
    assert recurrence.rel_err(th.tensor([1.0 + 1e-13], dtype=D), th.tensor([1.0], dtype=D)) == pytest.approx(1e-13, rel=1e-2)
    # the whole tensor enters, not the worst element and not the mean
    assert recurrence.rel_err(th.tensor([1.0, 1.0, 1.0, 2.0]), th.ones(4)) == pytest.approx(0.5, rel=1e-15)


@pytest.mark.parametrize('tol', [1e-4, 1e-2])
def test_assert_close_rejects_twice_the_tolerance(tol):
    """Negative test of the assertion the GPU parity tests use: a result whose error is 2 x tol fails, one
    at tol / 2 passes; wrong shapes, NaNs and a wrong count fail."""
    want = rnd(4, 7, 3, seed=1)
    noise = rnd(4, 7, 3, seed=2)
    noise = noise / noise.norm() * want.norm()          # relative size exactly 1
    ok = want + 0.5 * tol * noise
    bad = want + 2.0 * tol * noise
    assert recurrence.assert_close(ok, want, tol) == pytest.approx(0.5 * tol, rel=1e-6)
    with pytest.raises(AssertionError, match='relative error'):
        recurrence.assert_close(bad, want, tol)
    with pytest.raises(AssertionError, match='relative error'):
        recurrence.assert_all_close([ok, bad], [want, want], tol)
    assert recurrence.assert_all_close([ok, want], [want, want], tol)[1] == 0.0
    with pytest.raises(AssertionError, match='shape'):
        recurrence.assert_close(want[:, :, :2], want, tol)
    with pytest.raises(AssertionError, match='shape'):
        recurrence.assert_close(want.reshape(7, 4, 3), want, tol)
    nan = want.clone()
    nan[0, 0, 0] = float('nan')
    with pytest.raises(AssertionError):
        recurrence.assert_close(nan, want, tol)
    with pytest.raises(AssertionError, match='expected'):
        recurrence.assert_all_close([want], [want, want], tol)
    # a dropped contribution (one timestep's share of a sum) and a doubled one are both far outside
    parts = [rnd(5, 6, seed=10 + i) for i in range(16)]
    total = sum(parts)
    with pytest.raises(AssertionError):
        recurrence.assert_close(total - parts[3], total, tol)
    with pytest.raises(AssertionError):
        recurrence.assert_close(total + parts[3], total, tol)


# ------------------------------------------------------------------ chunked backward
@pytest.mark.parametrize('name,dims,chunk', [
    ('rwkv7', (2, 12, 2, 4, 4), 4), ('rwkv7', (1, 13, 2, 4, 8), 5), ('gated_delta_rule', (2, 9, 1, 4, 4), 2),
    ('mamba', (2, 10, 2, 4, 4), 3), ('mamba2', (2, 8, 3, 4, 4), 8), ('s4d', (2, 7, 1, 4, 4), 3),
    ('rwkv6', (2, 6, 2, 4, 4), 1), ('rwkv4', (2, 11, 1, 8, 1), 4), ('mlstm_gates', (2, 5, 2, 4, 1), 16)])
def test_chunked_backward_equals_unchunked(name, dims, chunk):
    """`chunked_loop_with_grads` == `loop_with_grads` in fp64 (1e-12): outputs, final states, every input
    gradient (time-broadcast and matrix inputs, summed over chunks, included) and the initial-state
    gradients; chunk lengths that divide T, that do not, of one step, and longer than T."""
    import cases
    step, xs, ss = cases.make_inputs(name, *dims, dtype=D)
    g = th.Generator().manual_seed(7)
    outs, fin = recurrence.run_loop(step, xs, ss)
    dy = [th.randn(o.shape, generator=g, dtype=D) for o in outs]
    dS = [th.randn(s.shape, generator=g, dtype=D) for s in fin]
    a = recurrence.loop_with_grads(step, xs, ss, dy, dS)
    b = recurrence.chunked_loop_with_grads(step, xs, ss, dy, dS, chunk)
    for part_a, part_b in zip(a, b):
        errs = recurrence.assert_all_close(part_b, part_a, 1e-12, name)
        assert len(errs) == len(part_a)
    # the gradients are not trivially zero (a chunked sweep that dropped the state hand-off would still pass then)
    assert all(float(g_.abs().max()) > 0 for g_ in b[3])
