"""GPU tests at the benchmark sizes and of the calling conventions.

The oracle (oracle/recurrence.py) is plain torch code, so for the full-size checks it runs on
the GPU in fp64: forward over the whole sequence, and forward + gradients with its chunked
backward (autograd through the whole loop would keep every intermediate state alive).
"""
import pytest
import torch as th

import flex_rnn_amd
from flex_rnn_amd import configs, ops, prebuild
from oracle import recurrence

import cases
import warm

pytestmark = pytest.mark.gpu
TOL = {th.float32: 1e-4, th.bfloat16: 1e-2}


def _gpu(xs):
    return [x.cuda() for x in xs]


@pytest.mark.parametrize('name', ['rwkv7', 'mamba2', 'mamba1'])
def test_full_size_forward_against_oracle(name):
    print(f'case full forward {name}', flush=True)
    wl = configs.make(name)
    xs, ss = _gpu(wl.inputs), _gpu(wl.states)
    with th.no_grad():
        (y_ref,), (S_ref,) = recurrence.run_loop(wl.step, xs, ss, dtype=th.float64)
    f = flex_rnn_amd.jit(wl.step)
    y, S = f(*xs, *ss)
    th.cuda.synchronize()
    assert recurrence.rel_err(y, y_ref) < TOL[wl.dtype] and recurrence.rel_err(S, S_ref) < TOL[wl.dtype]


@pytest.mark.parametrize('name,chunk', [('mamba1', 64), ('mamba2', 32), ('rwkv7', 32), ('gated_delta_rule', 64)])
def test_full_size_outputs_states_and_gradients_against_oracle(name, chunk):
    """The four GPU configurations at their full B, T, H, M, N: outputs, final state, the gradient of
    every input (the atomically accumulated ones of inputs shared over batch, time or heads included)
    and of the initial state against the oracle, which runs on the GPU in fp64 with its chunked
    backward (autograd through `chunk` steps at a time; equal to the plain loop, tests/test_oracle.py)."""
    dims = configs.DEFAULT_DIMS[name]
    print(f'case full-size gradients {name} {dims}', flush=True)
    wl = configs.make(name)
    dy, dS = configs.upstream_grads(wl)
    xs, ss = _gpu(wl.inputs), _gpu(wl.states)
    dyq = [g.cuda().to(wl.dtype) for g in dy]
    dSq = [g.cuda().to(wl.dtype) for g in dS]
    f = flex_rnn_amd.jit(wl.step)
    xg = [x.clone().requires_grad_() for x in xs]
    sg = [s.clone().requires_grad_() for s in ss]
    res = f(*xg, *sg)
    grads = th.autograd.grad(res, xg + sg, grad_outputs=dyq + dSq)
    got = [t.detach() for t in list(res) + list(grads)]
    del res, grads, xg, sg
    th.cuda.synchronize()
    want = recurrence.chunked_loop_with_grads(wl.step, xs, ss, dyq, dSq, chunk, dtype=th.float64)
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    assert all(float(w.abs().max()) > 0 for w in want[2:])
    errs = recurrence.assert_all_close(got, want, TOL[wl.dtype], name)
    print(['%.2e' % e for e in errs], flush=True)


def test_chunked_call_equals_single_call_at_full_size():
    """State hand-off: two calls over halves of the sequence give the same outputs, final
    state and gradients as one call (size-independent property, checked at T=1024)."""
    print('case chunked call rwkv7 full', flush=True)
    wl = configs.make('rwkv7')
    xs, ss = _gpu(wl.inputs), _gpu(wl.states)
    T = wl.dims[1]
    f, g = flex_rnn_amd.jit(wl.step), flex_rnn_amd.jit(wl.step)
    y, S = f(*xs, *ss)
    y1, S1 = g(*[x[:, :T // 2] for x in xs], *ss)
    h = flex_rnn_amd.jit(wl.step)
    y2, S2 = h(*[x[:, T // 2:] for x in xs], S1)
    # the same build of the forward kernel runs for both lengths (the timed choice is kept per batch, heads and
    # rows, not per sequence length) and the forward pass accumulates nothing atomically: bit for bit
    assert th.equal(y1, y[:, :T // 2])
    # the hand-off state passes through bf16 storage once more than inside a single call
    assert recurrence.rel_err(y2, y[:, T // 2:]) < 1e-2
    assert recurrence.rel_err(S2, S) < 1e-2


@pytest.mark.parametrize('name', ['rwkv7', 'mamba2', 'mamba1', 'gated_delta_rule'])
def test_backward_is_linear_in_upstream_gradients_at_full_size(name):
    """Size-independent property at the benchmark sizes: the gradients for 0.5 * g1 - 2 * g2 are
    0.5 * grads(g1) - 2 * grads(g2), for every input and the initial state (tolerance: the I/O dtype's
    rounding of three separately rounded results)."""
    print(f'case linear backward {name} full', flush=True)
    wl = configs.make(name)
    f = flex_rnn_amd.jit(wl.step)
    xs = [x.requires_grad_() for x in _gpu(wl.inputs)]
    ss = [s_.requires_grad_() for s_ in _gpu(wl.states)]
    out = f(*xs, *ss)
    gen = th.Generator(device='cuda').manual_seed(1)
    g1 = [th.randn(o.shape, generator=gen, device='cuda').to(o.dtype) for o in out]
    g2 = [th.randn(o.shape, generator=gen, device='cuda').to(o.dtype) for o in out]
    mix = [(0.5 * a.float() - 2.0 * b.float()).to(a.dtype) for a, b in zip(g1, g2)]
    r1 = th.autograd.grad(out, xs + ss, g1, retain_graph=True)
    r2 = th.autograd.grad(out, xs + ss, g2, retain_graph=True)
    rm = th.autograd.grad(out, xs + ss, mix)
    tol = 2e-2 if wl.dtype == th.bfloat16 else 1e-4
    for a, b, m in zip(r1, r2, rm):
        assert recurrence.rel_err(m, 0.5 * a.double() - 2.0 * b.double()) < tol


def test_strided_and_broadcast_views_match_contiguous_copies():
    """The adapter pattern of the reference's examples: [B,T,H,C] tensors unsqueezed, `v.mT`
    and a transposed state, plus an expanded (stride-0) input; no copies are made."""
    print('case strided views', flush=True)
    B, T, H, C = 2, 64, 2, 128
    g = th.Generator().manual_seed(3)
    r, w, k, v, a, b = [th.randn(B, T, H, C, generator=g).cuda() for _ in range(6)]
    w = -th.sigmoid(w)
    a = th.nn.functional.normalize(a, dim=-1)
    b = -a * th.sigmoid(b)
    S = (th.randn(B, H, C, C, generator=g) * 0.1).cuda()
    w_shared = w[:, :1].expand(B, T, H, C)                       # stride 0 over time
    step = flex_rnn_amd.jit(ops.rwkv7)

    def layer(r, w, k, v, a, b, S):
        r, w, k, v, a, b = [i.unsqueeze(-2) for i in (r, w, k, v, a, b)]
        y, S = step(r, w, k, v.mT, a, b, S.mT)
        return y, S.mT

    args = [r, w_shared, k, v, a, b, S]
    args = [x.requires_grad_() for x in args]
    y, ST = layer(*args)
    assert ST.shape == S.shape
    dy, dST = th.randn_like(y), th.randn_like(ST)
    grads = th.autograd.grad([y, ST], args, [dy, dST])
    assert grads[1].stride() == w_shared.contiguous().stride() or grads[1].shape == w_shared.shape
    # oracle on the same views
    xs = [i.detach().unsqueeze(-2) for i in (r, w_shared, k)] + [v.detach().unsqueeze(-2).mT] + [i.detach().unsqueeze(-2) for i in (a, b)]
    want = recurrence.loop_with_grads(ops.rwkv7, xs, [S.detach().mT], [dy], [dST.mT], dtype=th.float64)
    assert recurrence.rel_err(y, want[0][0]) < 1e-4 and recurrence.rel_err(ST.mT, want[1][0]) < 1e-4
    for i, (got, ref) in enumerate(zip(grads[:6], want[2])):
        ref = ref.squeeze(-2) if i != 3 else ref.mT.squeeze(-2)
        assert recurrence.rel_err(got, ref) < 1e-4, i
    assert recurrence.rel_err(grads[6].mT, want[3][0]) < 1e-4


def test_second_call_with_other_shape_is_rejected():
    print('case meta mismatch', flush=True)
    step, xs, ss = cases.make_inputs('gla', 1, 16, 1, 16, 16, dtype=th.float32)
    f = flex_rnn_amd.jit(step)
    f(*_gpu(xs), *_gpu(ss))
    step, xs2, ss2 = cases.make_inputs('gla', 1, 32, 1, 16, 16, dtype=th.float32)
    with pytest.raises(AssertionError, match="doesn't match compilation"):
        f(*_gpu(xs2), *_gpu(ss2))


def test_dynamic_mode_accepts_other_shapes():
    """`jit.dynamic`: batch, sequence length and strides change between calls; every call and its
    gradients match the oracle, and calls of an earlier signature still work afterwards."""
    print('case dynamic signatures', flush=True)
    f = flex_rnn_amd.jit.dynamic(ops.gla)
    for dims in ((1, 16, 2, 16, 16), (3, 50, 2, 16, 16), (1, 16, 2, 16, 16), (2, 33, 2, 16, 16)):
        step, xs, ss = cases.make_inputs('gla', *dims, dtype=th.float32)
        gx = [x.requires_grad_() for x in _gpu(xs)]
        gs = [s_.requires_grad_() for s_ in _gpu(ss)]
        out = f(*gx, *gs)
        g = th.Generator().manual_seed(5)
        dys = [th.randn(o.shape, generator=g) for o in out]
        grads = th.autograd.grad(out, gx + gs, [d.cuda() for d in dys])
        want = recurrence.loop_with_grads(step, xs, ss, dys[:1], dys[1:], dtype=th.float64)
        ref = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
        for a, b in zip(list(out) + list(grads), ref):
            assert recurrence.rel_err(a, b) < 1e-4, dims
    assert len(f._entries) == 3


def test_dynamic_mode_signatures_that_differ_only_in_the_state():
    """Same inputs and checkpoint shapes, the state once in fp32, once in bf16 and once transposed in
    memory: three plans, and each backward call runs the plan of its own forward call (gradient of the
    state in the state's dtype and layout), whatever the order of the backward calls."""
    print('case dynamic state signatures', flush=True)
    f = flex_rnn_amd.jit.dynamic(ops.gla)
    step, xs, ss = cases.make_inputs('gla', 2, 16, 2, 16, 16, dtype=th.float32)
    variants = [ss[0], ss[0].to(th.bfloat16), ss[0].transpose(-1, -2).contiguous().transpose(-1, -2)]
    calls = []
    for s0 in variants:
        gx = [x.requires_grad_() for x in _gpu(xs)]
        gs = s0.cuda().requires_grad_()
        calls.append((gx, gs, f(*gx, gs)))
    assert len(f._entries) == 3
    g = th.Generator().manual_seed(5)
    for k in (1, 2, 0):
        gx, gs, out = calls[k]
        dys = [th.randn(o.shape, generator=g).to(o.dtype) for o in out]
        grads = th.autograd.grad(out, gx + [gs], [d.cuda() for d in dys])
        assert grads[-1].dtype == variants[k].dtype and grads[-1].stride() == variants[k].stride()
        want = recurrence.loop_with_grads(step, xs, [variants[k]], dys[:1], dys[1:], dtype=th.float64)
        ref = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
        recurrence.assert_all_close(list(out) + list(grads), ref, 1e-2 if k == 1 else 1e-4, f'variant {k}')


@pytest.mark.parametrize('name', ['mamba_bh', 'matgain'])
def test_single_timestep_with_a_matrix_input_in_bf16(name):
    """T = 1 and a matrix input that is broadcast over nothing: its gradient is accumulated in fp32 by the
    kernels (reverse scan for `mamba_bh`, gradient kernel for `matgain`) and must come back in bf16."""
    print(f'case T=1 matrix input {name}', flush=True)
    step, xs, ss = cases.make_inputs(name, 2, 1, 2, 16, 16, dtype=th.bfloat16)
    f = flex_rnn_amd.jit(step)
    gx = [x.requires_grad_() for x in _gpu(xs)]
    gs = [s_.requires_grad_() for s_ in _gpu(ss)]
    out = f(*gx, *gs)
    g = th.Generator().manual_seed(5)
    dys = [th.randn(o.shape, generator=g).to(o.dtype) for o in out]
    grads = th.autograd.grad(out, gx + gs, [d.cuda() for d in dys])
    assert all(gr.dtype == th.bfloat16 and gr.shape == x.shape for gr, x in zip(grads, xs + ss))
    want = recurrence.loop_with_grads(step, xs, ss, dys[:1], dys[1:], dtype=th.float64)
    ref = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    recurrence.assert_all_close(list(out) + list(grads), ref, 1e-2, name)


_OFF = pytest.mark.skip(reason='ended in a GPU memory fault (reported while the gradient-kernel candidates were timed) '
                               'whose cause was not found: the same kernels pass on the CPU harness with guard pages and '
                               'array bounds checks.  The two experimental knobs of this case (operand read-ahead, scheduling '
                               'barrier) were taken out of the emitter afterwards; the case stays off the GPU')


@pytest.mark.parametrize('name,dims,knobs', warm.KNOB_CASES + [
    pytest.param('mamba2', (2, 19, 4, 64, 128), 'DF=1,PF=1,SB=1', marks=_OFF)])
def test_row_kernel_knobs_against_oracle(name, dims, knobs, monkeypatch):
    """The code-generation knobs of the row kernels that are timed candidates at the benchmark sizes (branch-free
    row sums, row sums kept per block, deferred output flush, deeper unrolling), forced at small sizes with a partial last chunk: outputs,
    final state and all gradients against the oracle."""
    print(f'case knobs {name} {dims} {knobs}', flush=True)
    monkeypatch.setenv('FLEX_RNN_TILE', knobs)
    from test_gpu_parity import run_case
    errs, got, wl = run_case(name, dims, None)
    tile = prebuild.plan_for(name, dims).tile
    assert all(getattr(tile, k) == int(v) for k, v in (kv.split('=') for kv in knobs.split(',')))


@pytest.mark.parametrize('name,dims', warm.SEGMENTED_CASES)
def test_segmented_call_against_oracle(name, dims):
    """`jit.segmented` (32 timesteps at a time under activation checkpointing, a shorter last segment): outputs, final
    state and all gradients against the oracle's single pass over the whole sequence."""
    print(f'case segmented {name} {dims}', flush=True)
    wl = configs.make(name, dims=dims)
    dy, dS = configs.upstream_grads(wl)
    want = recurrence.loop_with_grads(wl.step, wl.inputs, wl.states, dy, dS, dtype=th.float64)
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    f = flex_rnn_amd.jit(wl.step)
    xg = [x.requires_grad_() for x in _gpu(wl.inputs)]
    sg = [s.requires_grad_() for s in _gpu(wl.states)]
    res = f.segmented(*xg, *sg, segment=warm.SEGMENT)
    grads = th.autograd.grad(res, xg + sg, grad_outputs=[g.cuda().to(r.dtype) for g, r in zip(dy + dS, res)])
    recurrence.assert_all_close(list(res) + list(grads), want, TOL[wl.dtype], f'segmented {name}')


@pytest.mark.parametrize('name', ['rwkv7', 'mamba1', 'mamba2'])
def test_infer_matches_call(name):
    """`jit.infer` (no checkpoints, no saved sums) returns what a normal call returns."""
    print(f'case infer {name}', flush=True)
    B, T, H, M, N = configs.DEFAULT_DIMS[name]
    wl = configs.make(name, dims=(2, 77, 2, M, N))
    f = flex_rnn_amd.jit(wl.step)
    xs, ss = _gpu(wl.inputs), _gpu(wl.states)
    a = f.infer(*xs, *ss)
    b = f(*xs, *ss)
    # (the two kernels may have been given different tiles by the first-call timing, hence a
    # different order of the additions inside a row sum: equal up to rounding of the I/O dtype)
    tol = 1e-2 if wl.dtype == th.bfloat16 else 1e-5
    assert len(a) == len(b) and all(recurrence.rel_err(x, y) < tol for x, y in zip(a, b))
    assert not any(t.requires_grad for t in a)


def test_torch_compile_no_graph_break():
    print('case torch.compile', flush=True)
    step, xs, ss = cases.make_inputs('delta_rule', 2, 32, 2, 16, 16, dtype=th.float32)
    f = flex_rnn_amd.jit(step)
    xs, ss = _gpu(xs), _gpu(ss)

    def layer(q, k, v, beta, S):
        y, S = f(q * 1.0, k, v, beta, S)
        return y * 2.0, S

    ref = layer(*[x.clone().requires_grad_() for x in xs + ss])
    compiled = th.compile(layer, backend='aot_eager', fullgraph=True)
    args = [x.clone().requires_grad_() for x in xs + ss]
    out = compiled(*args)
    assert th.allclose(out[0], ref[0]) and th.allclose(out[1], ref[1])
    gy = [th.ones_like(o) for o in out]
    g1 = th.autograd.grad(out, args, gy)
    args2 = [x.clone().requires_grad_() for x in xs + ss]
    g2 = th.autograd.grad(layer(*args2), args2, gy)
    for a, b in zip(g1, g2):
        assert th.allclose(a, b, rtol=1e-5, atol=1e-6)


def test_check_grad_and_benchmark_helpers():
    print('case check_grad helper', flush=True)
    step, xs, ss = cases.make_inputs('gated_delta_rule', 2, 32, 2, 16, 16, dtype=th.float32)
    f = flex_rnn_amd.jit(step)
    err = flex_rnn_amd.check_grad(f, f.naive_fp64, _gpu(xs) + _gpu(ss), verbose=False, tol=1e-4)
    assert err < 1e-4
    ms = flex_rnn_amd.benchmark(f, _gpu(xs) + _gpu(ss), warmup=5, rep=20, verbose=False)      # (time budgets in ms)
    assert ms > 0


@pytest.mark.parametrize('name,dims', [('rwkv6', (2, 32, 2, 32, 32)), ('s4d', (2, 32, 1, 16, 32)), ('longhorn', (2, 32, 2, 32, 16)),
                                       ('hgrn', (2, 64, 1, 256, 1)), ('rwkv4', (2, 32, 1, 64, 1)), ('mlstm_gates', (2, 32, 2, 32, 1)),
                                       ('retention', (1, 32, 2, 16, 64)), ('mlstm_cell', (1, 32, 2, 32, 32)),
                                       ('zoo', (2, 32, 2, 32, 32)), ('zoo2', (2, 32, 2, 32, 32)), ('gla', (2, 32, 2, 100, 32)),
                                       # pointwise preparation inside the step: log-decay, in-step normalisation
                                       ('rwkv7', (2, 32, 2, 64, 64)), ('delta_rule_fused', (2, 32, 2, 32, 32)),
                                       # state widths that are not a power of two
                                       ('rwkv7', (2, 32, 2, 64, 96)), ('mamba', (2, 32, 2, 32, 12)), ('gla', (1, 32, 2, 16, 160))])
def test_other_recurrences(name, dims):
    print(f'case {name} {dims}', flush=True)
    step, xs, ss = cases.make_inputs(name, *dims, dtype=th.float32)
    f = flex_rnn_amd.jit(step)
    xg = [x.requires_grad_() for x in _gpu(xs)]
    sg = [s.requires_grad_() for s in _gpu(ss)]
    res = f(*xg, *sg)
    g = th.Generator().manual_seed(9)
    gy = [th.randn(r.shape, generator=g).cuda() for r in res]
    grads = th.autograd.grad(res, xg + sg, gy, allow_unused=True)
    want = recurrence.loop_with_grads(step, xs, ss, [t.cpu() for t in gy[:f.noutputs]], [t.cpu() for t in gy[f.noutputs:]])
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    got = list(res) + [th.zeros_like(p) if t is None else t for t, p in zip(grads, xg + sg)]
    errs = [recurrence.rel_err(a, b) for a, b in zip(got, want)]
    assert max(errs) < 1e-4, errs


@pytest.mark.parametrize('name,dims', [('rwkv7', (2, 77, 2, 128, 128)), ('mamba1', (2, 45, 4, 128, 16)),
                                       ('gated_delta_rule', (2, 1, 2, 128, 128)), ('mamba2', (2, 19, 4, 64, 128))])
def test_sequence_length_not_a_multiple_of_the_chunk(name, dims):
    """The reference requires T % chunk == 0 (twopass.py:173); here the last chunk may be
    partial, down to a single decode step (T = 1)."""
    print(f'case tail {name} {dims}', flush=True)
    wl = configs.make(name, dims=dims, dtype=th.float32)
    dy, dS = configs.upstream_grads(wl)
    want = recurrence.loop_with_grads(wl.step, wl.inputs, wl.states, dy, dS, dtype=th.float64)
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    f = flex_rnn_amd.jit(wl.step)
    xg = [x.requires_grad_() for x in _gpu(wl.inputs)]
    sg = [s.requires_grad_() for s in _gpu(wl.states)]
    res = f(*xg, *sg)
    grads = th.autograd.grad(res, xg + sg, grad_outputs=[g.cuda() for g in dy + dS])
    errs = [recurrence.rel_err(a, b) for a, b in zip(list(res) + list(grads), want)]
    assert max(errs) < 1e-4, errs


@pytest.mark.parametrize('dtype,tol', [(th.float16, 3e-3), (th.float64, 1e-4)])
def test_half_and_double_io(dtype, tol):
    """fp16 I/O; fp64 I/O is accepted and computed in fp32, as in the reference (to_cuda.py:169)."""
    print(f'case io dtype {dtype}', flush=True)
    step, xs, ss = cases.make_inputs('gla', 2, 32, 2, 32, 32, dtype=dtype)
    f = flex_rnn_amd.jit(step)
    xg = [x.requires_grad_() for x in _gpu(xs)]
    sg = [s.requires_grad_() for s in _gpu(ss)]
    res = f(*xg, *sg)
    assert res[0].dtype == dtype and res[1].dtype == dtype
    g = th.Generator().manual_seed(9)
    gy = [th.randn(r.shape, generator=g).to(dtype) for r in res]
    grads = th.autograd.grad(res, xg + sg, [t.cuda() for t in gy])
    want = recurrence.loop_with_grads(step, xs, ss, gy[:1], gy[1:])
    want = list(want[0]) + list(want[1]) + list(want[2]) + list(want[3])
    errs = [recurrence.rel_err(a, b) for a, b in zip(list(res) + list(grads), want)]
    assert max(errs) < tol, errs


def test_torch_compile_default_backend_and_side_stream():
    """The default torch.compile backend (inductor) fuses the pointwise work around the op; and
    launches follow torch's current stream."""
    print('case inductor + side stream', flush=True)
    step, xs, ss = cases.make_inputs('delta_rule', 2, 32, 2, 16, 16, dtype=th.float32)
    f = flex_rnn_amd.jit(step)
    xs, ss = _gpu(xs), _gpu(ss)

    def layer(q, k, v, beta, S):
        y, S = f(th.tanh(q), k, v, th.sigmoid(beta), S)
        return y * 2.0 + 1.0, S

    def run(fn):
        args = [x.clone().requires_grad_() for x in xs + ss]
        out = fn(*args)
        return list(out) + list(th.autograd.grad(out, args, [th.ones_like(o) for o in out]))

    ref = run(layer)
    got = run(th.compile(layer, fullgraph=True))
    assert max(recurrence.rel_err(a, b) for a, b in zip(got, ref)) < 1e-5
    side = th.cuda.Stream()
    with th.cuda.stream(side):
        got = run(layer)
    side.synchronize()
    assert all(th.equal(a, b) for a, b in zip(got, ref))


def test_hip_graph_capture_and_replay():
    """Forward + backward captured in a HIP graph (torch.cuda.CUDAGraph) and replayed with new input
    contents; every replay is compared with the eager result.  Eager work and synchronisations sit
    between the replays."""
    print('case hip graph', flush=True)
    wl = configs.make('mamba2', dims=(2, 64, 4, 64, 128))          # head-shared inputs: zero-filled fp32 scratch + atomics
    f = flex_rnn_amd.jit(wl.step)
    xs = [x.clone().requires_grad_() for x in _gpu(wl.inputs)]
    ss = [s_.clone().requires_grad_() for s_ in _gpu(wl.states)]

    def fb():
        out = f(*xs, *ss)
        return list(out) + list(th.autograd.grad(out, xs + ss, [th.ones_like(o) for o in out]))

    side = th.cuda.Stream()
    side.wait_stream(th.cuda.current_stream())
    with th.cuda.stream(side):
        for _ in range(3):                       # builds, tunes and warms the allocator outside the capture
            fb()
    th.cuda.current_stream().wait_stream(side)
    th.cuda.synchronize()
    graph = th.cuda.CUDAGraph()
    with th.cuda.graph(graph):
        static_out = fb()
    g = th.Generator().manual_seed(3)
    for it in range(3):
        with th.no_grad():
            for x, ref in zip(xs, wl.inputs):
                if x.shape[1] > 1 and x.shape[-2:] != (1, 1):          # new values for the per-step vector inputs
                    x.copy_((th.randn(ref.shape, generator=g) * 0.5).to(x.dtype))
        graph.replay()
        th.cuda.synchronize()
        got = [t.clone() for t in static_out]
        want = fb()                              # eager, same buffers
        th.cuda.synchronize()
        for a, b in zip(got, want):          # equal up to the order of fp32 atomic additions
            assert recurrence.rel_err(a, b) < 5e-3, it


@pytest.mark.parametrize('dims', [(0, 16, 2, 16, 16), (2, 0, 2, 16, 16)])
def test_empty_batch_and_empty_time(dims):
    """Nothing to scan: outputs are empty, the state passes through, and so does its gradient."""
    print(f'case empty {dims}', flush=True)
    step, xs, ss = cases.make_inputs('mamba', *dims, dtype=th.float32)
    xg = [x.cuda().requires_grad_() for x in xs]
    sg = [th.randn(s.shape).cuda().requires_grad_() for s in ss]
    f = flex_rnn_amd.jit(step, n_step_args=len(xs) + len(ss))
    y, S = f(*xg, *sg)
    assert y.shape == (dims[0], dims[1], dims[2], dims[3]) and th.equal(S, sg[0])
    dS = th.randn_like(S)
    grads = th.autograd.grad([y, S], xg + sg, [th.zeros_like(y), dS])
    assert th.equal(grads[-1], dS)
    assert all(g.shape == x.shape and not g.any() for g, x in zip(grads, xg))
    y2, S2 = f.infer(*xg, *sg)
    assert y2.shape == y.shape and th.equal(S2, sg[0])
