"""Parity and timing helpers with the reference's protocol
(/root/reference/flex_rnn/check_grad.py:12-67): per-tensor error
||a-b||_2 / max(||b||_2, 1e-30), maximum over all outputs and all input gradients, one
random cotangent per output, the first function's gradients scrambled before the second
function runs; timing = memory of one call, then median and 20%/80% quantiles of event-timed calls
over a fixed time budget (500 ms of warm-up, 1000 ms of measurement, the L2 flushed before every
call: what `triton.testing.do_bench(warmup=500, rep=1000)` does there).  No dependency on triton."""
import torch as th


def clone_strided(x):
    """Copy that keeps strides even for expanded / non-dense tensors."""
    r = th.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=x.device)
    r.copy_(x)
    return r


def rel_err(a, b):
    return ((a - b).norm() / max(b.norm(), 1e-30)).item()


def check_grad(f1, f2, inputs, backward=True, aux=(), tol=1e-2, verbose=True):
    inputs = [clone_strided(p) for p in inputs]
    if backward:
        inputs = [p.requires_grad_() for p in inputs]
    y1, y2 = f1(*inputs, *aux), f2(*inputs, *aux)
    y1 = y1 if type(y1) == tuple else (y1,)
    y2 = y2 if type(y2) == tuple else (y2,)
    worst = 0.0
    if verbose:
        print('Forward rel. error' + 's' * (len(y1) > 1))
    for a, b in zip(y1, y2):
        assert a.shape == b.shape, 'Shape mismatch ' + str([(p.shape, q.shape) for p, q in zip(y1, y2)])
        e = rel_err(a, b)
        worst = max(worst, e)
        if verbose:
            print(f'{e:.2e}  ({b.norm():.0e})')
    if not backward:
        return worst
    dy = tuple(th.randn_like(i) for i in y1)
    d1 = th.autograd.grad(y1, inputs, grad_outputs=tuple(clone_strided(i) for i in dy), allow_unused=True)
    for p in inputs:                # (check_grad.py:31-34) so that an uninitialised buffer cannot "recover" a gradient
        if p.grad is not None:
            p.grad.random_()
        p.grad = None
    d2 = th.autograd.grad(y2, inputs, grad_outputs=tuple(d.to(y.dtype) for d, y in zip(dy, y2)), allow_unused=True)
    if verbose:
        print('Gradient rel. errors')
    for a, b, p in zip(d1, d2, inputs):
        a = th.zeros_like(p) if a is None else a
        b = th.zeros_like(p) if b is None else b
        e = rel_err(a, b)
        worst = max(worst, e)
        if verbose:
            print(f'{e:.2e}  ({b.norm():.0e})')
    assert worst < tol, f'Large grad_check error: {worst*100:.1f}%!'
    return worst


def benchmark(f, params, backward=True, aux=(), warmup=500, rep=1000, verbose=True):
    """Prints the peak memory of one call and returns the median milliseconds per call (forward, or
    forward + gradients).  `warmup` and `rep` are time budgets in milliseconds (check_grad.py:59-66)."""
    if backward:
        for p in params:
            p.requires_grad_()
    dy = None

    def run():
        nonlocal dy
        y = f(*params, *aux)
        if not backward:
            return y
        y = y if type(y) == tuple else (y,)
        if dy is None:
            dy = tuple(th.randn_like(i) for i in y)
        return th.autograd.grad(y, params, grad_outputs=dy, allow_unused=True)

    run()                           # first call: builds and loads the kernels
    th.cuda.synchronize()
    th.cuda.reset_peak_memory_stats()
    run()                           # measure memory
    th.cuda.synchronize()
    mem = th.cuda.max_memory_allocated() / 2 ** 30
    if verbose:
        print(f'memory {mem:.2f} GB')
    flush = th.empty(256 << 20, dtype=th.int8, device='cuda')         # larger than the last-level cache

    def timed():
        flush.zero_()
        e0, e1 = th.cuda.Event(enable_timing=True), th.cuda.Event(enable_timing=True)
        e0.record()
        run()
        e1.record()
        return e0, e1

    est = []
    for _ in range(5):
        e0, e1 = timed()
        e1.synchronize()
        est.append(e0.elapsed_time(e1))
    per_call = max(sum(est) / len(est), 1e-3)
    for _ in range(max(1, int(warmup / per_call))):
        timed()
    events = [timed() for _ in range(max(1, int(rep / per_call)))]
    th.cuda.synchronize()
    times = sorted(e0.elapsed_time(e1) for e0, e1 in events)
    q = lambda f_: times[min(len(times) - 1, int(f_ * len(times)))]
    ms, lo, hi = q(0.5), q(0.2), q(0.8)
    if verbose:
        print(f'{ms:.2f} ms ({lo:.2f} - {hi:.2f})')
    return ms
