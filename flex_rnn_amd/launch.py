"""Host side of the compiled path: builds the three kernels of a plan through the C-ABI
runtime, allocates results / hidden buffers with torch, packs the kernel argument block
and launches on torch's current stream.

Counterpart of the reference's `forward` / `backward` closures
(/root/reference/flex_rnn/twopass.py:224-237, 343-363): same buffers in the same order
(outputs, final states, state checkpoints, packed aux | input grads, initial-state grads),
fp32 scratch + cast-back for gradients of inputs broadcast over batch / time / head
(twopass.py:181, 355, 359-360).  There is no CPU execution path here.
"""
from __future__ import annotations

import os
import struct
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List, Sequence, Tuple

import torch as th

from . import runtime
from .emit_hip import Emitter, KernelSpec, needs_gradient_kernel


def _strides5(t: th.Tensor) -> Tuple[int, ...]:
    s = [st if n > 1 else 0 for st, n in zip(t.stride(), t.shape)]
    return tuple(s + [0] * (5 - len(s)))


def kernel_specs(plan, prefetch: int = 4) -> List[KernelSpec]:
    em = Emitter(plan)
    return [em.fw(), em.bw1()] + ([em.bw2(prefetch=prefetch)] if needs_gradient_kernel(plan.part) else [])


MAX_SPILL_BYTES = 64      # per lane; the untimed choice among gradient-kernel builds does not accept more


def _compile(specs, force, seen):
    jobs = []
    for s in specs:
        key = runtime.source_key(s.name, s.source)
        again = force and (seen is None or key not in seen)
        if seen is not None:
            seen.add(key)
        jobs.append((s, again))
    # independent compiler processes: wait for them side by side (the runtime call releases the GIL)
    with ThreadPoolExecutor(max_workers=max(1, len(jobs))) as pool:
        paths = list(pool.map(lambda j: runtime.compile_kernel(j[0].name, j[0].source, force=j[1]), jobs))
    return [(s, path) for (s, _), path in zip(jobs, paths)]


def gradient_kernel_builds(plan, force: bool = False, seen=None):
    """Candidate builds of the gradient kernel, best guess first: [(spec, path, resources)].

    The kernel is register-hungry (a chunk of accumulators per lane; RWKV-7 sits a few registers
    below the limit for two waves per SIMD) and hides memory latency only through the waves
    resident on its SIMD, so small changes of the generated code move it across occupancy
    cliffs.  Builds with 4 and 2 checkpoint rows in flight are made, each also with a request
    for one more wave per SIMD when that looks feasible.  Without a timing the order is decided
    by the compiler's resource report: at most `MAX_SPILL_BYTES` spilled per lane, then more
    waves per SIMD, then fewer spills, then the deeper prefetch.  `CompiledPlan` times them on
    the first backward call and keeps the fastest."""
    em = Emitter(plan)
    cands, seen_src = [], set()

    def add(spec):
        if spec.source in seen_src:
            return None
        seen_src.add(spec.source)
        path = _compile([spec], force, seen)[0][1]
        res = runtime.kernel_resources(path)
        cands.append((spec, path, res))
        return res

    for pd in (4, 2):
        res = add(em.bw2(prefetch=pd))
        if res is not None and res['occupancy'] < 4 and (res['occupancy'] < 2 or res['vgprs'] <= 224):
            add(em.bw2(waves_per_simd=res['occupancy'] + 1, prefetch=pd))

    def rank(c):
        res = c[2]
        if res is None:
            return (1, 0, 0)
        return (0 if res['scratch'] <= MAX_SPILL_BYTES else 1, -res['occupancy'], res['scratch'])

    order = sorted(range(len(cands)), key=lambda i: (rank(cands[i]), i))
    return [cands[i] for i in order]


def compile_plan(plan, force: bool = False, seen=None) -> List[Tuple[KernelSpec, str]]:
    """Emit + compile (or fetch from the cache) the kernels of a plan, every candidate build of
    the gradient kernel included; returns the forward kernel, the reverse scan and the
    first-ranked gradient kernel.  Needs no GPU.  With `force` a cached code object is rebuilt,
    once per key recorded in `seen`."""
    em = Emitter(plan)
    built = _compile([em.fw(), em.bw1(), em.fw(save=False)], force, seen)[:2]
    if needs_gradient_kernel(plan.part):
        spec, path, _ = gradient_kernel_builds(plan, force, seen)[0]
        built.append((spec, path))
    return built


class CompiledPlan:
    _tune_pending = False

    def __init__(self, plan, state_meta=None):
        self.plan = plan
        # (shape, stride, dtype) of the initial states: gradients w.r.t. them are laid out alike
        self.state_meta = state_meta
        # when set to a list, every launch appends (kernel name, start event, end event)
        self.profile_events = None
        em = Emitter(plan)
        built = _compile([em.fw(), em.bw1()], False, None)
        self.kernels = {}
        self.modules = []

        def load(spec, path):
            try:
                mod = runtime.Module(path)
                kern = mod.kernel(spec.name)
            except runtime.RuntimeError_ as first:
                if 'no HIP runtime' in str(first) or 'no ROCm-capable device' in str(first).lower():
                    raise
                # a truncated / corrupt cache entry: rebuild it once, then give up loudly
                path = runtime.compile_kernel(spec.name, spec.source, force=True)
                mod = runtime.Module(path)
                kern = mod.kernel(spec.name)
            self.modules.append(mod)
            return kern

        self._load = load
        for spec, path in built:
            self.kernels[spec.name] = (spec, load(spec, path))
        # gradient kernel: every candidate build is loaded; the first backward call times them
        self.bw2_builds = []
        self.bw2_times = None
        if needs_gradient_kernel(plan.part):
            for spec, path, res in gradient_kernel_builds(plan):
                self.bw2_builds.append((spec, load(spec, path), res))
            self.kernels['frnn_bw2'] = self.bw2_builds[0][:2]
        self._tune_pending = len(self.bw2_builds) > 1 and os.environ.get('FLEX_RNN_TUNE', '1') != '0'
        # per kernel: grid (fixed by the plan's sizes) and one packer for the whole argument block
        self._grid, self._packer = {}, {}
        for k, (s, _) in self.kernels.items():
            self._register(k, s)

    def _register(self, name, spec):
        pl = self.plan
        env = dict(B=pl.B, T=pl.T, H=pl.H, M=pl.M, nch=pl.nchunks)
        self._grid[name] = tuple(int(eval(g, {}, env)) for g in spec.grid)
        self._packer[name] = struct.Struct('<' + 'q5q' * max(len(spec.tensors), 1) + '5q')

    def _add_kernel(self, spec):
        path = _compile([spec], False, None)[0][1]
        self.kernels[spec.name] = (spec, self._load(spec, path))
        self._register(spec.name, spec)

    # ------------------------------------------------------------------ launch helper
    def _launch(self, kname: str, tensors: Dict[str, th.Tensor]):
        spec, kern = self.kernels[kname]
        pl = self.plan
        vals = []
        dev = None
        for name in spec.tensors:
            t = tensors[name]
            assert t.is_cuda, f'{name}: the compiled path runs on the GPU only (got a {t.device} tensor)'
            dev = t.device if dev is None else dev
            assert t.device == dev, 'all tensors must live on the same device'
            vals.append(t.data_ptr())
            vals.extend(_strides5(t))
        if not spec.tensors:
            vals = [0] * 6
        buf = self._packer[kname].pack(*vals, pl.B, pl.T, pl.H, pl.M, pl.nchunks)
        grid = self._grid[kname]
        with th.cuda.device(dev):
            stream = th.cuda.current_stream(dev).cuda_stream
            if self.profile_events is not None:
                e0, e1 = th.cuda.Event(enable_timing=True), th.cuda.Event(enable_timing=True)
                e0.record()
                kern.launch(grid, (spec.block, 1, 1), buf, stream=stream)
                e1.record()
                self.profile_events.append((kname, e0, e1))
            else:
                kern.launch(grid, (spec.block, 1, 1), buf, stream=stream)

    def _tune_gradient_kernel(self, tensors, accumulators):
        """Times every candidate build of the gradient kernel once on the tensors of this call
        (after one untimed run each) and keeps the fastest.  The kernel only stores and
        accumulates; what it accumulated into is cleared again afterwards.  Synchronises."""
        self._tune_pending = False
        saved = [a.clone() for a in accumulators]       # the reverse scan has already added its share
        times = []
        for spec, kern, res in self.bw2_builds:
            self.kernels['frnn_bw2'] = (spec, kern)
            self._launch('frnn_bw2', tensors)
            e0, e1 = th.cuda.Event(enable_timing=True), th.cuda.Event(enable_timing=True)
            e0.record()
            self._launch('frnn_bw2', tensors)
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1))
        best = min(range(len(times)), key=times.__getitem__)
        self.kernels['frnn_bw2'] = self.bw2_builds[best][:2]
        self.bw2_times = times
        for a, s_ in zip(accumulators, saved):
            a.copy_(s_)

    # ------------------------------------------------------------------ forward
    def forward(self, inputs: Sequence[th.Tensor], state0: Sequence[th.Tensor]):
        pl, p = self.plan, self.plan.part
        dev = inputs[0].device
        B, T, H, M, N = pl.B, pl.T, pl.H, pl.M, pl.N
        outs = tuple(th.empty(B, T, H, M, dtype=dt, device=dev) for dt in pl.out_dtypes)
        stT = tuple(th.empty_like(s) for s in state0)
        sck = tuple(th.empty(B, H, pl.nchunks, M, N, dtype=th.float32, device=dev) for _ in state0)
        aux = th.empty(len(p.aux), B, H, T, M, dtype=th.float32, device=dev)
        tensors = {'aux': aux}
        for i, x in enumerate(inputs):
            tensors[f'in{i}'] = x
        for k in range(p.nstates):
            tensors[f'st{k}'] = state0[k]
            tensors[f'stT{k}'] = stT[k]
            tensors[f'sck{k}'] = sck[k]
        for k in range(p.noutputs):
            tensors[f'out{k}'] = outs[k]
        self._launch('frnn_fw', tensors)
        return (*outs, *stT, *sck, aux)

    def forward_only(self, inputs: Sequence[th.Tensor], state0: Sequence[th.Tensor]):
        """Outputs and final states only (inference): a forward kernel that writes no checkpoints and
        no saved row sums, built on first use."""
        if 'frnn_fwi' not in self.kernels:
            self._add_kernel(Emitter(self.plan).fw(save=False))
        pl, p = self.plan, self.plan.part
        dev = inputs[0].device
        outs = tuple(th.empty(pl.B, pl.T, pl.H, pl.M, dtype=dt, device=dev) for dt in pl.out_dtypes)
        stT = tuple(th.empty_like(s) for s in state0)
        tensors = {}
        for i, x in enumerate(inputs):
            tensors[f'in{i}'] = x
        for k in range(p.nstates):
            tensors[f'st{k}'] = state0[k]
            tensors[f'stT{k}'] = stT[k]
        for k in range(p.noutputs):
            tensors[f'out{k}'] = outs[k]
        self._launch('frnn_fwi', tensors)
        return (*outs, *stT)

    # ------------------------------------------------------------------ backward
    def backward(self, doutput, dstateT, inputs, state_store, aux):
        pl, p = self.plan, self.plan.part
        dev = inputs[0].device
        B, T, H, M, N = pl.B, pl.T, pl.H, pl.M, pl.N
        atomic = set(pl.atomic)
        daux = th.empty(len(p.daux), B, H, T, M, dtype=th.float32, device=dev)
        dck = tuple(th.empty(B, H, pl.nchunks, M, N, dtype=th.float32, device=dev) for _ in state_store) \
            if 'frnn_bw2' in self.kernels else ()
        if self.state_meta is not None:
            dst0 = tuple(th.empty_strided(sh, st, dtype=dt, device=dev) for sh, st, dt in self.state_meta)
        else:
            dst0 = tuple(th.empty_like(s) for s in dstateT)
        dins = []
        for i, x in enumerate(inputs):
            if i in atomic:
                dins.append(th.zeros(x.shape, dtype=th.float32, device=dev))
            else:
                dins.append(th.empty_like(x))
        tensors = {'aux': aux, 'daux': daux}
        for i, x in enumerate(inputs):
            tensors[f'in{i}'] = x
            tensors[f'din{i}'] = dins[i]
        for k in range(p.nstates):
            tensors[f'dstT{k}'] = dstateT[k]
            tensors[f'dst{k}'] = dst0[k]
            tensors[f'sck{k}'] = state_store[k]
            if dck:
                tensors[f'dck{k}'] = dck[k]
        for k in range(p.noutputs):
            tensors[f'dout{k}'] = doutput[k]
        self._launch('frnn_bw1', tensors)
        if 'frnn_bw2' in self.kernels:
            if self._tune_pending and not th.cuda.is_current_stream_capturing():
                self._tune_gradient_kernel(tensors, [dins[i] for i in atomic])
            self._launch('frnn_bw2', tensors)
        for i in atomic:
            x = inputs[i]
            g = th.empty_like(x)
            g.copy_(dins[i])
            dins[i] = g
        return tuple(dins), dst0
