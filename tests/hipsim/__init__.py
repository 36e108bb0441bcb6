"""CPU execution of the emitted HIP kernels (test tool).

`SimPlan` is `flex_rnn_amd.launch.CompiledPlan` with the two device-facing steps swapped:
kernels are compiled for the host against `hipsim.h` (fibers as GPU threads, see there) and a
launch runs the workgroups one after another on CPU tensors.  Every tensor of a launch is
copied into a buffer that ends (or, on a second pass, starts) at an inaccessible guard page, so
an out-of-bounds access by the kernel kills the process with SIGSEGV; callers run it in a
subprocess.  All host logic (allocation, argument packing, launch order, scratch handling) is
the product's own code.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import struct
import subprocess
import tempfile

import torch as th

from flex_rnn_amd.launch import CompiledPlan, kernel_specs, _strides5

_HERE = os.path.dirname(os.path.abspath(__file__))
_CACHE = os.path.join(tempfile.gettempdir(), 'frnn_hipsim')


def _compile_host(spec) -> str:
    src = spec.source.replace('#include <hip/hip_runtime.h>', '#include "hipsim.h"')
    assert 'hipsim.h' in src
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
    key = hashlib.sha256((hdr + src + ' '.join(extra)).encode()).hexdigest()[:20]
    os.makedirs(_CACHE, exist_ok=True)
    so = os.path.join(_CACHE, f'{spec.name}_{key}.so')
    if not os.path.isfile(so):
        cpp = os.path.join(_CACHE, f'{spec.name}_{key}.cpp')
        with open(cpp, 'w') as f:
            f.write(src)
        tmp = so + f'.tmp{os.getpid()}'
        cmd = ['g++', '-O1', '-std=c++17', '-shared', '-fPIC', '-w', *extra, '-I', _HERE, cpp, '-o', tmp]
        subprocess.run(cmd, check=True)
        os.replace(tmp, so)
    return so


class SimPlan(CompiledPlan):
    def __init__(self, plan, state_meta=None, against_end=True):
        self.plan = plan
        self.state_meta = state_meta
        self.against_end = against_end
        self.kernels = {}
        # HIPSIM_PREFETCH selects the gradient kernel's variant with that many checkpoint rows in flight
        specs = kernel_specs(plan, prefetch=int(os.environ.get('HIPSIM_PREFETCH', '4')))
        from flex_rnn_amd.emit_hip import Emitter
        specs.append(Emitter(plan).fw(save=False))          # the inference kernel, used by forward_only()
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=len(specs)) as pool:      # host compiler runs side by side
            list(pool.map(_compile_host, specs))
        for spec in specs:
            self._add_kernel(spec)

    def _tune(self, name, tensors, accumulators=()):
        pass

    def _add_kernel(self, spec):
        lib = ctypes.CDLL(_compile_host(spec))
        lib.sim_alloc.restype = ctypes.c_void_p
        lib.sim_alloc.argtypes = [ctypes.c_size_t, ctypes.c_int]
        lib.sim_free.argtypes = [ctypes.c_void_p]
        fn = getattr(lib, f'sim_launch_{spec.name}')
        fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        self.kernels[spec.name] = (spec, lib, fn)

    def _launch(self, kname, tensors):
        spec, lib, fn = self.kernels[kname]
        pl = self.plan
        buf = bytearray()
        staged = []
        for name in spec.tensors:
            t = tensors[name]
            assert not t.is_cuda
            # span of the view inside its storage
            span = 1 + sum((n - 1) * s for n, s in zip(t.shape, t.stride()) if n > 0) if t.numel() else 0
            nbytes = span * t.element_size()
            p = lib.sim_alloc(nbytes, 1 if self.against_end else 0)
            assert p, 'sim_alloc failed'
            if nbytes:
                flat = th.as_strided(t, (span,), (1,))
                ctypes.memmove(p, flat.data_ptr(), nbytes)
            staged.append((t, p, nbytes, span))
            buf += struct.pack('<q5q', p, *_strides5(t))
        if not spec.tensors:
            buf += struct.pack('<q5q', 0, 0, 0, 0, 0, 0)
        buf += struct.pack('<5q', pl.B, pl.T, pl.H, pl.M, pl.nchunks)
        size = getattr(lib, f'sim_args_size_{spec.name}')()
        assert len(buf) == size, (size, len(buf))      # the block must match the kernel's parameter list
        env = dict(B=pl.B, T=pl.T, H=pl.H, M=pl.M, nch=pl.nchunks)
        grid = tuple(int(eval(g, {}, env)) for g in spec.grid)
        cbuf = ctypes.create_string_buffer(bytes(buf), len(buf))
        rc = fn(cbuf, grid[0], grid[1], grid[2], spec.block)
        assert rc == 0, f'hipsim launch of {kname} failed'
        for t, p, nbytes, span in staged:
            if nbytes:
                flat = th.as_strided(t, (span,), (1,))
                ctypes.memmove(flat.data_ptr(), p, nbytes)
            lib.sim_free(p)
