"""The launch entry point that allocates nothing (`frnn_launch_static`, include/frnn_rt.h) against
`frnn_launch`: the same kernels of a plan, once with torch-allocated hidden buffers (checkpoints, saved
sums), once with those buffers in the library's static scratch buffer.  Results must be identical
bit for bit (the recurrences used here accumulate nothing atomically).  Two calls in a row, the second on
a smaller input that finds the first call's contents in the buffer."""
import struct

import pytest
import torch as th

from flex_rnn_amd import configs, planner, runtime

pytestmark = pytest.mark.gpu

import warm


def _plan(name, dims):
    wl = configs.make(name, dims=dims)
    xs, ss = [x.cuda() for x in wl.inputs], [s.cuda() for s in wl.states]
    # (one gradient-kernel instance per chunk walks all rows: with split rows the row gradients would meet in atomics)
    fwd, bwd, fm, bm = planner.build_twopass(wl.step, xs, ss, tile=warm.no_alloc_tile(name, dims))
    dy, dS = configs.upstream_grads(wl)
    return wl, xs, ss, fwd.compiled, [g.cuda().to(wl.dtype) for g in dy], [g.cuda().to(wl.dtype) for g in dS]


def _both_ways(name, dims, probe_copy):
    wl, xs, ss, cp, dy, dS = _plan(name, dims)
    pl, p = cp.plan, cp.plan.part
    nout, nst = p.noutputs, p.nstates
    assert not pl.atomic, 'this test compares bit for bit: no atomically accumulated gradients'
    # 1. the existing entry point, hidden buffers allocated by torch (this also settles which build of each kernel runs)
    res = cp.forward(tuple(xs), tuple(ss))
    outs, stT, sck, aux = res[:nout], res[nout:nout + nst], res[nout + nst:nout + 2 * nst], res[-1]
    dins, dst0 = cp.backward(tuple(dy), tuple(dS), tuple(xs), sck, aux)
    th.cuda.synchronize()
    # 2. the same kernels through frnn_launch_static
    layout, total = cp.static_layout()
    outs2 = [th.empty_like(o) for o in outs]
    stT2 = [th.empty_like(s_) for s_ in stT]
    dins2 = [th.empty_like(d) for d in dins]
    dst02 = [th.empty_like(d) for d in dst0]
    tensors = {}
    for i, x in enumerate(xs):
        tensors[f'in{i}'], tensors[f'din{i}'] = x, dins2[i]
    for k in range(nst):
        tensors[f'st{k}'], tensors[f'stT{k}'], tensors[f'dstT{k}'], tensors[f'dst{k}'] = ss[k], stT2[k], dS[k].contiguous(), dst02[k]
    for k in range(nout):
        tensors[f'out{k}'], tensors[f'dout{k}'] = outs2[k], dy[k].contiguous()
    before = th.cuda.memory_allocated()
    cp.launch_static('frnn_fw', tensors, layout)
    cp.launch_static('frnn_bw1', tensors, layout)
    cp.launch_static('frnn_bw2', tensors, layout)
    assert th.cuda.memory_allocated() == before
    # the checkpoints the forward kernel left in the scratch buffer, read back through the same entry point
    off, n = layout['sck0']
    back = th.empty(n // 4, dtype=th.float32, device='cuda')
    args = struct.pack('<qqq', 0, back.data_ptr(), n // 4)
    probe_copy.launch_static((256, 1, 1), (256, 1, 1), args, [(0, off, n, 0)], stream=th.cuda.current_stream().cuda_stream)
    th.cuda.synchronize()
    for a, b in zip(outs2 + stT2 + dins2 + dst02, list(outs) + list(stT) + list(dins) + list(dst0)):
        assert th.equal(a, b), f'{name} {dims}: the static-scratch launch differs from frnn_launch'
    assert th.equal(back, sck[0].flatten())
    return total


def test_static_scratch_launch_matches_frnn_launch():
    print('case no-alloc launch', flush=True)
    mod = runtime.Module(runtime.compile_kernel('probe', warm.NO_ALLOC_PROBE))
    probe_copy, probe_add = mod.kernel('probe_copy'), mod.kernel('probe_add_one')
    big = _both_ways('rwkv7', (2, 64, 2, 128, 128), probe_copy)
    small = _both_ways('rwkv7', (1, 32, 2, 128, 128), probe_copy)      # finds the first call's data in the buffer
    assert small < big <= runtime.STATIC_SCRATCH_BYTES

    # `clear`: two launches that add 1 to a region, the second after a zero fill
    n = 5000
    out = th.empty(n, dtype=th.float32, device='cuda')
    st = th.cuda.current_stream().cuda_stream
    add_args, copy_args = struct.pack('<qq', 0, n), struct.pack('<qqq', 0, out.data_ptr(), n)
    probe_add.launch_static((8, 1, 1), (256, 1, 1), add_args, [(0, 512, 4 * n, 1)], stream=st)
    probe_add.launch_static((8, 1, 1), (256, 1, 1), add_args, [(0, 512, 4 * n, 0)], stream=st)
    probe_copy.launch_static((8, 1, 1), (256, 1, 1), copy_args, [(0, 512, 4 * n, 0)], stream=st)
    th.cuda.synchronize()
    assert bool((out == 2.0).all())
    probe_add.launch_static((8, 1, 1), (256, 1, 1), add_args, [(0, 512, 4 * n, 1)], stream=st)
    probe_copy.launch_static((8, 1, 1), (256, 1, 1), copy_args, [(0, 512, 4 * n, 0)], stream=st)
    th.cuda.synchronize()
    assert bool((out == 1.0).all())

    # sizes beyond the buffer, misaligned and overlapping regions are refused with a clear message
    cap = runtime.STATIC_SCRATCH_BYTES
    for slots, msg in [([(0, 0, cap + 256, 0)], 'do not fit'), ([(0, cap - 256, 512, 0)], 'do not fit'),
                       ([(0, 128, 256, 0)], 'multiple of 256'), ([(0, 0, 1024, 0), (8, 512, 1024, 0)], 'overlap'),
                       ([(24, 0, 256, 0)], 'outside'), ([(4, 0, 256, 0)], 'outside')]:
        with pytest.raises(RuntimeError, match=msg):
            probe_copy.launch_static((1, 1, 1), (64, 1, 1), copy_args, slots, stream=st)
    # a plan whose hidden buffers do not fit says so before anything is launched
    wl = configs.make('rwkv7', dims=(1, 1, 1, 128, 128))
    from flex_rnn_amd import prebuild
    from flex_rnn_amd.launch import CompiledPlan
    cp = CompiledPlan.__new__(CompiledPlan)
    cp.plan = prebuild.plan_for('rwkv7')
    with pytest.raises(AssertionError, match='static scratch buffer holds'):
        cp.static_layout()
