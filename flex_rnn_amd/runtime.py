"""ctypes binding of the C-ABI kernel runtime (`libfrnn_rt.so`, include/frnn_rt.h).

`build_library()` compiles the runtime in-tree; `lib()` loads it and fails loudly
when it has not been built.  `compile_kernel()` turns HIP source into a cached
gfx950 code object (no GPU needed); `Module` / `Kernel` load and launch it.
"""
from __future__ import annotations

import ctypes
import hashlib
import json
import os
import re
import subprocess
import threading
from typing import Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
LIB_PATH = os.path.join(_HERE, 'libfrnn_rt.so')
ARCH = 'gfx950'
STATIC_SCRATCH_BYTES = 64 << 20       # FRNN_STATIC_SCRATCH_BYTES of include/frnn_rt.h
# (the resource-usage remarks land in the compile log; `kernel_resources` reads them back)
EMITTER_OPTS = '-ffp-contract=fast -munsafe-fp-atomics -Rpass-analysis=kernel-resource-usage'

# flags `frnn_compile` always passes (flex_rnn_amd/csrc/frnn_rt.cpp); part of the cache key, like the compiler's version
FIXED_FLAGS = '--genco -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops'

_lib = None
_toolchain = None


def toolchain_id() -> str:
    """What identifies the compiler behind `frnn_compile`: the ROCm release named in `<rocm>/.info/version` and
    the resolved path and size of the clang binary hipcc drives.  A code object built by another compiler
    release must not be taken from the cache.  Read from files, not by running the compiler: a process that
    already uses the GPU (under a profiler, say) should not start programs it does not have to."""
    global _toolchain
    if _toolchain is None:
        hipcc = os.environ.get('FRNN_HIPCC') or next(
            (p for p in (os.path.join(os.environ.get('ROCM_PATH', '/opt/rocm'), 'bin', 'hipcc'), '/opt/rocm/bin/hipcc')
             if os.access(p, os.X_OK)), '')
        root = os.path.dirname(os.path.dirname(os.path.realpath(hipcc))) if hipcc else ''
        parts = []
        try:
            with open(os.path.join(root, '.info', 'version')) as f:
                parts.append('rocm version ' + f.read().strip())
        except OSError:
            pass
        for clang in (os.path.join(root, 'lib', 'llvm', 'bin', 'clang++'), os.path.join(root, 'llvm', 'bin', 'clang++')):
            try:
                real = os.path.realpath(clang)
                parts.append(f'{os.path.basename(real)} {os.path.getsize(real)} bytes')
                break
            except OSError:
                continue
        _toolchain = ' | '.join(parts) or 'unknown'
    return _toolchain


class RuntimeError_(RuntimeError):
    pass


def build_library(verbose: bool = False) -> str:
    """Compile flex_rnn_amd/csrc/{frnn_rt.cpp, frnn_static.hip} -> flex_rnn_amd/libfrnn_rt.so (hipcc, gfx950: the
    second file holds device code, the static scratch buffer and its fill kernel)."""
    srcs = [os.path.join(_HERE, 'csrc', 'frnn_rt.cpp'), os.path.join(_HERE, 'csrc', 'frnn_static.hip')]
    inc = os.path.join(_ROOT, 'include')
    tmp = LIB_PATH + f'.tmp{os.getpid()}'
    hipcc = os.environ.get('FRNN_HIPCC') or '/opt/rocm/bin/hipcc'
    # (no absolute run path to the toolchain's HIP runtime: the library binds to the copy the process holds, by soname)
    rocm_lib = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(hipcc))), 'lib')
    cmd = [hipcc, f'--offload-arch={ARCH}', '-O2', '-std=c++17', '-shared', '-fPIC', '-Wall', '-no-hip-rt', '-L', rocm_lib, '-lamdhip64',
           '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
           '-I', inc, '-I', os.path.join(_HERE, 'csrc'), *srcs, '-o', tmp, '-ldl', '-pthread']
    if verbose:
        print(' '.join(cmd))
    subprocess.run(cmd, check=True)
    os.replace(tmp, LIB_PATH)
    global _lib
    _lib = None
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.isfile(LIB_PATH):
        raise RuntimeError_(
            f'{LIB_PATH} is missing: the HIP kernel runtime has not been built. '
            'Run `python -c "import __graft_entry__ as g; g.build()"` (or flex_rnn_amd.runtime.build_library()). '
            'There is no CPU fallback for the compiled path; use `.naive` for a pure-PyTorch run.')
    try:
        import torch  # noqa: F401  (its bundled HIP runtime must be in the process first: the library binds to the
        #                            loaded copy by soname instead of bringing in a second one)
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    L.frnn_version.restype = ctypes.c_int
    L.frnn_last_error.restype = ctypes.c_char_p
    L.frnn_compile.restype = ctypes.c_int
    L.frnn_compile.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p, ctypes.c_char_p,
                               ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t]
    L.frnn_module_load.restype = ctypes.c_int
    L.frnn_module_load.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
    L.frnn_get_kernel.restype = ctypes.c_int
    L.frnn_get_kernel.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
    L.frnn_kernel_arg_bytes.restype = ctypes.c_int
    L.frnn_kernel_arg_bytes.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_size_t)]
    L.frnn_launch.restype = ctypes.c_int
    L.frnn_launch.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
                              ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    L.frnn_launch_static.restype = ctypes.c_int
    L.frnn_launch_static.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
                                     ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                     ctypes.c_void_p, ctypes.c_size_t]
    L.frnn_module_free.restype = ctypes.c_int
    L.frnn_module_free.argtypes = [ctypes.c_void_p]
    L.frnn_device_cus.restype = ctypes.c_int
    _lib = L
    return L


EXPORTS = ('frnn_version', 'frnn_last_error', 'frnn_compile', 'frnn_module_load', 'frnn_get_kernel',
           'frnn_kernel_arg_bytes', 'frnn_launch', 'frnn_launch_static', 'frnn_module_free', 'frnn_device_cus')


def _check(rc: int, what: str):
    if rc != 0:
        msg = lib().frnn_last_error().decode('utf-8', 'replace')
        raise RuntimeError_(f'{what} failed (code {rc}): {msg}')


def cache_dir() -> str:
    d = os.environ.get('FLEX_RNN_CACHE')
    if d:
        return d
    d = os.path.join(_HERE, '_kcache')
    try:
        os.makedirs(d, exist_ok=True)
        if os.access(d, os.W_OK):
            return d
    except OSError:
        pass
    return os.path.join(os.path.expanduser('~'), '.cache', 'flex_rnn_amd')


def source_key(name: str, src: str, opts: str = EMITTER_OPTS) -> str:
    h = hashlib.sha256()
    h.update(ARCH.encode())
    h.update(b'\0')
    h.update(FIXED_FLAGS.encode())
    h.update(b'\0')
    h.update(toolchain_id().encode())
    h.update(b'\0')
    h.update(opts.encode())
    h.update(b'\0')
    h.update(src.encode())
    return f'{name}_{h.hexdigest()[:24]}'


def compile_kernel(name: str, src: str, opts: str = EMITTER_OPTS, force: bool = False) -> str:
    """Returns the path of the gfx950 code object for `src`, compiling on a cache miss
    (or always, with `force`)."""
    key = source_key(name, src, opts)
    if force:
        try:
            os.remove(os.path.join(cache_dir(), key + '.hsaco'))
        except FileNotFoundError:
            pass
    out = ctypes.create_string_buffer(4096)
    b = src.encode()
    rc = lib().frnn_compile(b, len(b), ARCH.encode(), opts.encode(), cache_dir().encode(), key.encode(), out, 4096)
    _check(rc, f'compiling kernel {name}')
    path = out.value.decode()
    _record_resources(path)
    return path


_RES_FIELDS = {'vgprs': r'\bVGPRs: (\d+)', 'scratch': r'ScratchSize \[bytes/lane\]: (\d+)',
               'occupancy': r'Occupancy \[waves/SIMD\]: (\d+)', 'lds': r'LDS Size \[bytes/block\]: (\d+)'}


def _record_resources(hsaco: str) -> None:
    """After a compile, condenses the compiler's resource-usage remarks (registers, spill bytes,
    waves per SIMD, LDS) into `<key>.res` next to the code object; the log itself need not be
    kept."""
    base = hsaco[:-len('.hsaco')]
    if os.path.exists(base + '.res') and os.path.getmtime(base + '.res') >= os.path.getmtime(hsaco):
        return
    try:
        with open(base + '.log') as f:
            log = f.read()
    except OSError:
        return
    vals = {}
    for k, pat in _RES_FIELDS.items():
        m = re.search(pat, log)
        if m:
            vals[k] = int(m.group(1))
    if len(vals) == len(_RES_FIELDS):
        tmp = f'{base}.res.tmp{os.getpid()}_{threading.get_ident()}'      # (threads of one process compile side by side)
        with open(tmp, 'w') as f:
            json.dump(vals, f)
        os.replace(tmp, base + '.res')


def kernel_resources(hsaco: str):
    """{'vgprs', 'scratch' (spill bytes per lane), 'occupancy' (waves per SIMD), 'lds'} of a
    compiled kernel, or None when unknown."""
    try:
        with open(hsaco[:-len('.hsaco')] + '.res') as f:
            return json.load(f)
    except (OSError, ValueError):
        return None


_U3 = ctypes.c_uint32 * 3


class Kernel:
    def __init__(self, module: 'Module', name: str):
        self.module = module
        self.name = name
        h = ctypes.c_void_p()
        _check(lib().frnn_get_kernel(module.handle, name.encode(), ctypes.byref(h)), f'looking up kernel {name}')
        self.handle = h
        n = ctypes.c_size_t()
        _check(lib().frnn_kernel_arg_bytes(h, ctypes.byref(n)), f'reading the argument size of kernel {name}')
        self.arg_bytes = int(n.value)      # what the code object declares; 0 = unknown

    def launch(self, grid: Sequence[int], block: Sequence[int], args: bytes, stream: int = 0, lds_bytes: int = 0):
        g = _U3(*grid)
        b = _U3(*block)
        _check(lib().frnn_launch(self.handle, g, b, lds_bytes, ctypes.c_void_p(stream), args, len(args)),
               f'launching kernel {self.name}')


    def launch_static(self, grid: Sequence[int], block: Sequence[int], args: bytes, slots, stream: int = 0, lds_bytes: int = 0):
        """`launch` with the hidden buffers named by `slots` - (byte offset of the pointer field in `args`,
        byte offset inside the library's static scratch buffer, size in bytes, clear first?) each - placed
        in that buffer by the library; allocates nothing."""
        g = _U3(*grid)
        b = _U3(*block)
        arr = (ctypes.c_uint64 * (4 * max(len(slots), 1)))(*[int(v) for s in slots for v in s])
        _check(lib().frnn_launch_static(self.handle, g, b, lds_bytes, ctypes.c_void_p(stream), args, len(args),
                                        ctypes.cast(arr, ctypes.c_void_p), len(slots)),
               f'launching kernel {self.name} on the static scratch buffer')


class Module:
    def __init__(self, path: str):
        self.path = path
        h = ctypes.c_void_p()
        _check(lib().frnn_module_load(path.encode(), ctypes.byref(h)), f'loading code object {path}')
        self.handle = h

    def kernel(self, name: str) -> Kernel:
        return Kernel(self, name)

    def close(self):
        if self.handle:
            lib().frnn_module_free(self.handle)
            self.handle = None


def device_cus() -> int:
    return lib().frnn_device_cus()
