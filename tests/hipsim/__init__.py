"""CPU execution of the emitted HIP kernels (test tool).

`SimPlan` is `flex_rnn_amd.launch.CompiledPlan` with the device-facing steps swapped:
kernels are compiled for the host against `hipsim.h` (fibers as GPU threads, see there) and a
launch runs the workgroups one after another on CPU tensors.  Every tensor of a launch is
copied into a buffer that ends (or, on a second pass, starts) at an inaccessible guard region, so
an out-of-bounds access by the kernel kills the process with SIGSEGV; callers run it in a
subprocess.  All host logic - allocation of results and hidden buffers, the choice among the
candidate builds of a kernel with its re-registration of grid and argument layout (`_tune`,
`_select`), argument packing, the launch audit, launch order, scratch handling - is the product's
own code.

Environment: HIPSIM_SEED=<n> shuffles threads and workgroups (hipsim.h); HIPSIM_BOUNDS=1 checks
every index into a declared array; HIPSIM_UNINIT=1 builds with clang and fills every uninitialised
local variable with a NaN pattern; HIPSIM_CANDIDATES=1 makes `SimPlan` hold every candidate build
the product would time on a GPU and run each of them once per kernel before settling on one (the last; with
FLEX_RNN_PICK="<kernel>=<index>" the named candidate alone, so that its results are the ones compared).
"""
from __future__ import annotations

import contextlib
import ctypes
import hashlib
import os
import re
import subprocess
import tempfile

import torch as th

from flex_rnn_amd import launch
from flex_rnn_amd.launch import CompiledPlan, kernel_specs

_HERE = os.path.dirname(os.path.abspath(__file__))
_CACHE = os.path.join(tempfile.gettempdir(), 'frnn_hipsim')
_CLANG = '/opt/rocm/lib/llvm/bin/clang++'
LDS_LIMIT = 160 * 1024          # bytes of LDS a gfx950 workgroup may use

_SHARED_DECL = re.compile(r'__shared__\s+float\s+(\w+)((?:\[[^\]]+\])+);')


def _compile_host(spec) -> str:
    src = spec.source.replace('#include <hip/hip_runtime.h>', '#include "hipsim.h"')
    assert 'hipsim.h' in src
    src = re.sub(r'__attribute__\(\(amdgpu_waves_per_eu\([^)]*\)\)\)', '', src)      # (an occupancy request; means nothing on the host)
    src = src.replace('"+v"', '"+r"')      # (the register class of an empty asm statement that hides a value's origin)
    # LDS arrays start a workgroup with undefined contents: poison each one where it is declared
    src, n = _SHARED_DECL.subn(lambda m: f'__shared__ float {m.group(1)}{m.group(2)}; sim_lds_poison({m.group(1)}, sizeof({m.group(1)}));', src)
    assert n == src.count('__shared__'), 'a __shared__ declaration the harness does not recognise'
    src += f'''
extern "C" int sim_launch_{spec.name}(const void* argbuf, int gx, int gy, int gz, int bx) {{
  Args A;
  memcpy(&A, argbuf, sizeof(Args));
  return sim_run_grid([&] {{ {spec.name}(A); }}, gx, gy, gz, bx);
}}
extern "C" int sim_args_size_{spec.name}() {{ return (int)sizeof(Args); }}
'''
    hdr = open(os.path.join(_HERE, 'hipsim.h')).read()
    # HIPSIM_BOUNDS=1: every index into a declared array (registers, LDS) is checked, a bad one traps
    extra = ['-fsanitize=bounds', '-fsanitize-undefined-trap-on-error'] if os.environ.get('HIPSIM_BOUNDS', '0') == '1' else []
    cxx = 'g++'
    if os.environ.get('HIPSIM_UNINIT', '0') == '1':
        # registers hold no zeros either: every local variable the code does not initialise starts as a NaN pattern
        assert os.access(_CLANG, os.X_OK), f'HIPSIM_UNINIT needs {_CLANG}'
        cxx, extra = _CLANG, extra + ['-ftrivial-auto-var-init=pattern']
    key = hashlib.sha256((hdr + src + cxx + ' '.join(extra)).encode()).hexdigest()[:20]
    os.makedirs(_CACHE, exist_ok=True)
    so = os.path.join(_CACHE, f'{spec.name}_{key}.so')
    if not os.path.isfile(so):
        cpp = os.path.join(_CACHE, f'{spec.name}_{key}.cpp')
        with open(cpp, 'w') as f:
            f.write(src)
        tmp = so + f'.tmp{os.getpid()}'
        cmd = [cxx, '-O1', '-std=c++17', '-shared', '-fPIC', '-w', *extra, '-I', _HERE, cpp, '-o', tmp]
        subprocess.run(cmd, check=True)
        os.replace(tmp, so)
    return so


class SimKernel:
    """A host build of one emitted kernel; stands where the product holds a `runtime.Kernel`."""

    def __init__(self, spec):
        self.spec = spec
        self.lib = ctypes.CDLL(_compile_host(spec))
        self.lib.sim_alloc.restype = ctypes.c_void_p
        self.lib.sim_alloc.argtypes = [ctypes.c_size_t, ctypes.c_int]
        self.lib.sim_free.argtypes = [ctypes.c_void_p]
        self.lib.sim_lds_peak_bytes.restype = ctypes.c_size_t
        self.fn = getattr(self.lib, f'sim_launch_{spec.name}')
        self.fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        self.arg_bytes = int(getattr(self.lib, f'sim_args_size_{spec.name}')())


@contextlib.contextmanager
def poisoned_empty():
    """While active, `torch.empty` / `empty_like` / `empty_strided` hand out floating-point memory filled with NaN: on a GPU
    such memory holds whatever was there before, here fresh pages would read as zeros and hide a kernel that reads what
    nothing has written (or leaves part of a result unwritten)."""
    real = {n: getattr(th, n) for n in ('empty', 'empty_like', 'empty_strided')}

    def wrap(fn):
        def alloc(*a, **k):
            t = fn(*a, **k)
            if t.is_floating_point() and t.device.type == 'cpu' and t.numel():
                th.as_strided(t, (t.untyped_storage().nbytes() // t.element_size(),), (1,), 0).fill_(float('nan'))
            return t
        return alloc
    try:
        for n, fn in real.items():
            setattr(th, n, wrap(fn))
        yield
    finally:
        for n, fn in real.items():
            setattr(th, n, fn)


class SimPlan(CompiledPlan):
    _on_gpu = False
    _tune_rounds = 2

    def forward(self, *a, **k):
        with poisoned_empty():
            return super().forward(*a, **k)

    def forward_only(self, *a, **k):
        with poisoned_empty():
            return super().forward_only(*a, **k)

    def backward(self, *a, **k):
        with poisoned_empty():
            return super().backward(*a, **k)

    def __init__(self, plan, state_meta=None, against_end=True):
        self.plan = plan
        self.state_meta = state_meta
        self.against_end = against_end
        self.device = None
        self.profile_events = None
        self.kernels, self.modules = {}, []
        self.builds, self.build_times, self._grid, self._packer = {}, {}, {}, {}
        self.build_source = {}
        self.launches = []          # (kernel name, candidate number) of every launch, in order
        self._fixed = {}
        self._tune_on = True
        self.lds_peak = {}
        if plan.B == 0 or plan.T == 0:
            return
        candidates = os.environ.get('HIPSIM_CANDIDATES', '0') == '1'
        if candidates:
            # every candidate build the product would time on the first call of a problem large enough to time the
            # code-generation knobs too
            old = launch.TUNE_KNOBS_FROM
            if os.environ.get('HIPSIM_KNOBS', '1') == '1':      # (HIPSIM_KNOBS=0: the candidate list this problem size gets on a GPU)
                launch.TUNE_KNOBS_FROM = 0
            try:
                sets = {'frnn_fw': launch.row_kernel_specs(plan, False), 'frnn_bw1': launch.row_kernel_specs(plan, True),
                        'frnn_fwi': launch.row_kernel_specs(plan, False, save=False)}
            finally:
                launch.TUNE_KNOBS_FROM = old
            if launch.needs_gradient_kernel(plan.part):
                sets['frnn_bw2'] = launch.gradient_kernel_specs(plan)
        else:
            # HIPSIM_PREFETCH selects the gradient kernel's variant with that many checkpoint rows in flight
            specs = kernel_specs(plan, prefetch=int(os.environ.get('HIPSIM_PREFETCH', '4')))
            from flex_rnn_amd.emit_hip import Emitter
            specs.append(Emitter(plan).fw(save=False))          # the inference kernel, used by forward_only()
            sets = {s_.name: [s_] for s_ in specs}
        from concurrent.futures import ThreadPoolExecutor
        flat = [s_ for v in sets.values() for s_ in v]
        with ThreadPoolExecutor(max_workers=min(8, len(flat))) as pool:      # host compiler runs side by side
            list(pool.map(_compile_host, flat))
        fixed = launch._fixed_picks()       # FLEX_RNN_PICK="frnn_fw=2": that candidate alone runs, so that its results are what is checked
        for name, specs in sets.items():
            self.builds[name] = [(s_, SimKernel(s_), None) for s_ in specs]
            if len(specs) > 1 and name not in fixed:
                self._tune_pending = set(self._tune_pending) | {name}
            self._select(name, min(fixed.get(name, 0), len(specs) - 1))

    def _device_name(self):
        return 'hipsim'

    def _capturing(self):
        return False

    _WRITTEN = ('out', 'stT', 'sck', 'aux', 'din', 'dst', 'dck', 'daux')      # tensors a kernel stores or accumulates into

    def _tune(self, name, tensors, accumulators=()):
        self._acc = [(a, a.clone()) for a in accumulators]
        self._first = None
        try:
            super()._tune(name, tensors, accumulators)
        finally:
            self._acc, self._first = [], None

    def _timed_launch(self, kname, tensors):
        """A launch of the selected candidate; the "time" makes the last candidate the winner of `_tune`, so
        that the launch after the timing rounds runs a build other than the first.  Every candidate starts from the
        same accumulator contents and must leave what the first candidate left, up to the order of additions (tiles
        differ in it): a candidate with wrong values is caught even when another one wins."""
        for a, saved in getattr(self, '_acc', []):
            a.copy_(saved)
        self._launch(kname, tensors)
        spec = self.kernels[kname][0]
        index = next(i for i, b in enumerate(self.builds[kname]) if b[0] is spec)
        got = {n: tensors[n] for n in spec.tensors
               if n.startswith(self._WRITTEN) and not n.startswith(('dstT', 'dout')) and tensors[n].is_floating_point() and tensors[n].numel()}
        if getattr(self, '_first', None) is None:
            self._first = (index, {n: t.clone() for n, t in got.items()})
        else:
            i0, ref = self._first
            self.compared = getattr(self, 'compared', 0) + 1
            for n, t in got.items():
                a, b = t.double(), ref[n].double()
                assert bool((th.isnan(a) == th.isnan(b)).all()), f'{kname}: candidates {i0} and {index} leave different parts of {n} unwritten'
                a, b = th.nan_to_num(a), th.nan_to_num(b)
                tol = 2e-2 if t.element_size() == 2 else 1e-4
                err = (a - b).abs().max().item()
                assert err <= tol * max(b.abs().max().item(), 1e-30), f'{kname}: candidate {index} differs from candidate {i0} in {n}: {err:.3e}'
        return float(len(self.builds[kname]) - index)

    def _launch(self, kname, tensors):
        spec, kern = self.kernels[kname]
        self.launches.append((kname, next(i for i, b in enumerate(self.builds[kname]) if b[0] is spec)))
        lib = kern.lib
        staged, guarded = [], {}
        for name in spec.tensors:
            t = tensors[name]
            assert not t.is_cuda
            # span of the view inside its storage
            span = 1 + sum((n - 1) * s for n, s in zip(t.shape, t.stride()) if n > 0) if t.numel() else 0
            nbytes = span * t.element_size()
            p = lib.sim_alloc(nbytes, 1 if self.against_end else 0)
            assert p, 'sim_alloc failed'
            if nbytes:
                ctypes.memmove(p, th.as_strided(t, (span,), (1,)).data_ptr(), nbytes)
                raw = th.frombuffer((ctypes.c_char * nbytes).from_address(p), dtype=t.dtype, count=span)
                guarded[name] = th.as_strided(raw, t.shape, t.stride())
            else:
                guarded[name] = t
            staged.append((t, p, nbytes, span))
        buf, _ = self._pack(kname, guarded)         # (the product's packing and, with FLEX_RNN_CHECK=1, its audit)
        assert len(buf) == kern.arg_bytes, (kern.arg_bytes, len(buf))      # the block must match the kernel's parameter list
        grid = self._grid[kname]
        cbuf = ctypes.create_string_buffer(bytes(buf), len(buf))
        rc = kern.fn(cbuf, grid[0], grid[1], grid[2], spec.block)
        assert rc == 0, f'hipsim launch of {kname} failed'
        peak = int(lib.sim_lds_peak_bytes())
        self.lds_peak[kname] = max(self.lds_peak.get(kname, 0), peak)
        assert peak <= LDS_LIMIT, f'{kname} uses {peak} bytes of LDS per workgroup, gfx950 has {LDS_LIMIT}'
        for t, p, nbytes, span in staged:
            if nbytes:
                ctypes.memmove(th.as_strided(t, (span,), (1,)).data_ptr(), p, nbytes)
            lib.sim_free(p)
