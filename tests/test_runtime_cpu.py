"""CPU tests of the C-ABI runtime: exported symbols, compile cache, error reporting, and the
launch marshalling (against a stand-in HIP runtime)."""
import ctypes
import os
import re
import subprocess
import sys
import textwrap

import pytest

from flex_rnn_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRIVIAL = '#include <hip/hip_runtime.h>\nextern "C" __global__ void k(float* p) { p[threadIdx.x] = 1.0f; }\n'


def test_library_exports_every_declared_symbol(runtime_lib):
    hdr = open(os.path.join(ROOT, 'include', 'frnn_rt.h')).read()
    declared = set(re.findall(r'\b(frnn_\w+)\s*\(', hdr))
    declared -= {'frnn_module_s'}
    assert declared == set(runtime.EXPORTS)
    for name in declared:
        assert hasattr(runtime_lib, name), name
    assert runtime_lib.frnn_version() >= 100


def test_compile_cache_hit_and_miss(runtime_lib, tmp_path, monkeypatch):
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    p1 = runtime.compile_kernel('k', TRIVIAL)
    assert os.path.getsize(p1) > 0 and p1.startswith(str(tmp_path)) and p1.endswith('.hsaco')
    assert os.path.isfile(p1[:-6] + '.hip')
    m1 = os.path.getmtime(p1)
    assert runtime.compile_kernel('k', TRIVIAL) == p1 and os.path.getmtime(p1) == m1     # hit
    p2 = runtime.compile_kernel('k', TRIVIAL + '// other\n')
    assert p2 != p1                                                                       # key = source hash
    # a truncated cache entry is rebuilt when asked to
    runtime.compile_kernel('k', TRIVIAL, force=True)
    assert os.path.getsize(p1) > 0


def test_threads_compiling_the_same_key(runtime_lib, tmp_path, monkeypatch):
    """Warm-up compiles plans from several threads, and plans share kernels: the compiler runs once,
    every thread gets the same path, and no temporary file of one thread is taken by another."""
    from concurrent.futures import ThreadPoolExecutor
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    src = TRIVIAL + '// threads\n'
    with ThreadPoolExecutor(max_workers=4) as pool:
        paths = list(pool.map(lambda _: runtime.compile_kernel('k', src), range(4)))
    assert len(set(paths)) == 1 and os.path.getsize(paths[0]) > 0
    assert not [f for f in os.listdir(tmp_path) if '.tmp' in f]


def test_compile_error_is_reported(runtime_lib, tmp_path, monkeypatch):
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    with pytest.raises(RuntimeError, match='hipcc failed'):
        runtime.compile_kernel('bad', 'this is not HIP\n')
    assert not [f for f in os.listdir(tmp_path) if f.endswith('.hsaco')]


def test_bad_key_and_null_arguments(runtime_lib, tmp_path):
    out = ctypes.create_string_buffer(256)
    rc = runtime_lib.frnn_compile(b'x', 1, b'gfx950', b'', str(tmp_path).encode(), b'../evil', out, 256)
    assert rc == 1 and b'key' in runtime_lib.frnn_last_error()
    rc = runtime_lib.frnn_compile(None, 0, b'gfx950', b'', str(tmp_path).encode(), b'k', out, 256)
    assert rc == 1


def test_load_without_gpu_fails_loudly(runtime_lib, tmp_path, monkeypatch):
    import torch
    if torch.cuda.is_available():
        pytest.skip('a GPU is present')
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    path = runtime.compile_kernel('k', TRIVIAL)
    with pytest.raises(RuntimeError):
        runtime.Module(path)


def test_launch_marshalling_against_stand_in_hip(runtime_lib, tmp_path):
    so = tmp_path / 'libfakehip.so'
    subprocess.run(['g++', '-shared', '-fPIC', '-o', str(so), os.path.join(ROOT, 'tests', 'fakehip', 'fakehip.cpp')], check=True)
    code = textwrap.dedent(f'''
        import ctypes, struct, sys
        sys.path.insert(0, {ROOT!r})
        fake = ctypes.CDLL({str(so)!r}, mode=ctypes.RTLD_GLOBAL)
        from flex_rnn_amd import runtime
        assert runtime.device_cus() == 256
        open({str(so)!r} + '.img', 'wb').write(bytes([127]) + b'ELF' + bytes(100)); m = runtime.Module({str(so)!r} + '.img'); k = m.kernel('x')
        buf = struct.pack('<q5q', 0x7f0012345678, 1, 2, 3, 4, 5) + struct.pack('<5q', 7, 8, 9, 10, 11)
        k.launch((2, 3, 4), (64, 1, 1), buf, stream=0xabc)
        n = ctypes.c_size_t.in_dll(fake, 'g_nargs').value
        got = bytes((ctypes.c_ubyte * 8192).in_dll(fake, 'g_args'))[:n]
        assert got == buf and ctypes.c_int.in_dll(fake, 'g_extra_ok').value == 1
        assert list((ctypes.c_uint * 7).in_dll(fake, 'g_dims')) == [2, 3, 4, 64, 1, 1, 0]
        assert ctypes.c_void_p.in_dll(fake, 'g_stream').value == 0xabc
        for bad in [dict(args=buf[:-4]), dict(grid=(0, 1, 1)), dict(block=(2048, 1, 1)), dict(grid=(1, 70000, 1))]:
            kw = dict(grid=(1, 1, 1), block=(64, 1, 1), args=buf); kw.update(bad)
            try:
                k.launch(kw['grid'], kw['block'], kw['args'])
            except RuntimeError as e:
                assert 'frnn_launch' in str(e), e
            else:
                raise SystemExit('accepted ' + str(bad))
        open({str(so)!r} + '.bad', 'wb').write(b'not a code object')
        try:
            runtime.Module({str(so)!r} + '.bad')
        except RuntimeError as e:
            assert 'not a code object' in str(e), e
        else:
            raise SystemExit('loaded garbage')
        print('ok')
    ''')
    r = subprocess.run([sys.executable, '-c', code], capture_output=True, text=True)
    assert r.returncode == 0 and 'ok' in r.stdout, r.stdout + r.stderr


def test_argument_block_is_checked_against_the_code_object(runtime_lib, tmp_path, monkeypatch):
    """`frnn_get_kernel` reads the kernel's argument-segment size from the code object's metadata note;
    `frnn_launch` rejects a block of any other size (a block that is short would leave the kernel with
    unset pointers), and the host refuses to register a kernel whose packed block has another size."""
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    src = ('#include <hip/hip_runtime.h>\nstruct TArg { void* p; long long s[5]; };\n'
           'struct Args { TArg t[3]; long long B, T, H, M, nch; };\n'
           'extern "C" __global__ void one(Args A) { ((float*)A.t[0].p)[threadIdx.x] = (float)A.B; }\n'
           'extern "C" __global__ void two(float* p, int n, double x) { if ((int)threadIdx.x < n) p[threadIdx.x] = (float)x; }\n'
           # (uses the grid size: the compiler appends hidden arguments, which the launcher fills in, not the caller)
           'extern "C" __global__ void three(float* p, int n) { for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 1.0f; }\n')
    path = runtime.compile_kernel('pair', src)
    so = tmp_path / 'libfakehip.so'
    subprocess.run(['g++', '-shared', '-fPIC', '-o', str(so), os.path.join(ROOT, 'tests', 'fakehip', 'fakehip.cpp')], check=True)
    code = textwrap.dedent(f'''
        import ctypes, struct, sys
        sys.path.insert(0, {ROOT!r})
        fake = ctypes.CDLL({str(so)!r}, mode=ctypes.RTLD_GLOBAL)
        from flex_rnn_amd import runtime
        m = runtime.Module({path!r})
        one, two = m.kernel('one'), m.kernel('two')
        assert one.arg_bytes == 3 * 48 + 40, one.arg_bytes
        assert two.arg_bytes == 24, two.arg_bytes
        assert m.kernel('three').arg_bytes == 16
        assert m.kernel('absent_from_metadata').arg_bytes == 0        # (the stand-in resolves any name)
        good = bytes(3 * 48 + 40)
        one.launch((1, 1, 1), (64, 1, 1), good)
        for bad in (good[:-8], good + bytes(8), good[:48]):
            try:
                one.launch((1, 1, 1), (64, 1, 1), bad)
            except RuntimeError as e:
                assert 'declares 184' in str(e), e
            else:
                raise SystemExit('accepted a block of %d bytes' % len(bad))
        # the host side: a plan whose packer disagrees with the code object is refused before any launch
        from flex_rnn_amd.launch import CompiledPlan
        from flex_rnn_amd.emit_hip import KernelSpec
        class P: B = T = H = M = nchunks = 1
        cp = CompiledPlan.__new__(CompiledPlan)
        cp.plan, cp.kernels, cp._grid, cp._packer = P, {{}}, {{}}, {{}}
        cp.builds = {{'one': [(KernelSpec('one', '', ['a', 'b', 'c'], 64, ('1', '1', '1')), one, None)],
                     'short': [(KernelSpec('one', '', ['a', 'b'], 64, ('1', '1', '1')), one, None)]}}
        cp._select('one', 0)
        try:
            cp._select('short', 0)
        except AssertionError as e:
            assert 'declares 184' in str(e), e
        else:
            raise SystemExit('registered a mis-sized argument block')
        print('ok')
    ''')
    r = subprocess.run([sys.executable, '-c', code], capture_output=True, text=True)
    assert r.returncode == 0 and 'ok' in r.stdout, r.stdout + r.stderr


def test_cache_key_covers_fixed_flags_and_compiler(monkeypatch):
    """The key of a cached code object changes with the source, the options, the flags the runtime always
    passes (which must be the ones named in the C++ source) and the compiler's version."""
    cpp = open(os.path.join(ROOT, 'flex_rnn_amd', 'csrc', 'frnn_rt.cpp')).read()
    for flag in runtime.FIXED_FLAGS.split():
        assert f'"{flag}"' in cpp, flag
    assert 'version' in runtime.toolchain_id()
    base = runtime.source_key('k', 'src')
    assert base == runtime.source_key('k', 'src') and base != runtime.source_key('k', 'src2')
    assert base != runtime.source_key('k', 'src', opts='-O1')
    monkeypatch.setattr(runtime, 'FIXED_FLAGS', runtime.FIXED_FLAGS + ' -g')
    assert runtime.source_key('k', 'src') != base
    monkeypatch.undo()
    monkeypatch.setattr(runtime, '_toolchain', 'HIP version: 0.0 | clang version 0')
    assert runtime.source_key('k', 'src') != base


def test_static_scratch_launch_validates_before_touching_the_device(runtime_lib, tmp_path):
    """`frnn_launch_static` refuses regions that do not fit its buffer, are misaligned, overlap or name a
    pointer field outside the argument block - all before any device call, so this runs without a GPU."""
    hdr = open(os.path.join(ROOT, 'include', 'frnn_rt.h')).read()
    assert re.search(r'#define FRNN_STATIC_SCRATCH_BYTES \(64ull << 20\)', hdr) and runtime.STATIC_SCRATCH_BYTES == 64 << 20
    so = tmp_path / 'libfakehip.so'
    subprocess.run(['g++', '-shared', '-fPIC', '-o', str(so), os.path.join(ROOT, 'tests', 'fakehip', 'fakehip.cpp')], check=True)
    code = textwrap.dedent(f'''
        import ctypes, sys
        sys.path.insert(0, {ROOT!r})
        fake = ctypes.CDLL({str(so)!r}, mode=ctypes.RTLD_GLOBAL)
        from flex_rnn_amd import runtime
        open({str(so)!r} + '.img', 'wb').write(bytes([127]) + b'ELF' + bytes(100)); k = runtime.Module({str(so)!r} + '.img').kernel('x')
        cap = runtime.STATIC_SCRATCH_BYTES
        args = bytes(48)
        cases = [([(0, 0, cap + 1, 0)], 'do not fit'), ([(0, cap, 256, 0)], 'do not fit'), ([(0, 256, 0, 0)], 'do not fit'),
                 ([(0, 100, 256, 0)], 'multiple of 256'), ([(0, 0, 300, 0), (8, 256, 256, 0)], 'overlap'),
                 ([(0, 0, 256, 0), (0, 256, 256, 0)], 'same pointer field'), ([(48, 0, 256, 0)], 'outside'),
                 ([(12, 0, 256, 0)], 'misaligned'), ([(0, i * 256, 256, 0) for i in range(65)], 'at most 64')]
        for slots, msg in cases:
            try:
                k.launch_static((1, 1, 1), (64, 1, 1), args, slots)
            except RuntimeError as e:
                assert msg in str(e), (msg, str(e))
            else:
                raise SystemExit('accepted ' + str(slots))
        for kw, msg in [(dict(args=bytes(44)), 'multiple of 8'), (dict(args=bytes(8192)), 'at most 4096'), (dict(grid=(0, 1, 1)), 'empty grid')]:
            a = dict(grid=(1, 1, 1), args=args); a.update(kw)
            try:
                k.launch_static(a['grid'], (64, 1, 1), a['args'], [])
            except RuntimeError as e:
                assert msg in str(e), (msg, str(e))
            else:
                raise SystemExit('accepted ' + str(kw))
        print('ok')
    ''')
    r = subprocess.run([sys.executable, '-c', code], capture_output=True, text=True)
    assert r.returncode == 0 and 'ok' in r.stdout, r.stdout + r.stderr


def test_launch_audit_rejects_what_the_kernels_take_on_trust(runtime_lib, tmp_path):
    """FLEX_RNN_CHECK=1: before a launch, every tensor must have the shape and element type the kernel's index
    arithmetic was emitted for, hidden buffers must be contiguous, and the grid must cover the plan.  Runs the real
    host path (planned, compiled and loaded kernels; the stand-in HIP answers the module calls) up to the launch."""
    so = tmp_path / 'libfakehip.so'
    subprocess.run(['g++', '-shared', '-fPIC', '-o', str(so), os.path.join(ROOT, 'tests', 'fakehip', 'fakehip.cpp')], check=True)
    code = textwrap.dedent(f'''
        import ctypes, os, sys
        os.environ['FLEX_RNN_CHECK'] = '1'
        os.environ['FLEX_RNN_TUNE'] = '0'
        sys.path.insert(0, {ROOT!r}); sys.path.insert(0, os.path.join({ROOT!r}, 'tests'))
        fake = ctypes.CDLL({str(so)!r}, mode=ctypes.RTLD_GLOBAL)
        import torch as th
        import cases
        from flex_rnn_amd import planner, launch
        step, xs, ss = cases.make_inputs('gla', 2, 16, 2, 16, 16, dtype=th.float32)
        plan, fm, bm = planner.make_plan(step, xs, ss)
        class OnHost(launch.CompiledPlan):
            _on_gpu = False
        cp = OnHost(plan)
        B, T, H, M, N = 2, 16, 2, 16, 16
        good = {{'aux': th.empty(len(plan.part.aux), B, H, T, M), 'out0': th.empty(B, T, H, M), 'st0': ss[0], 'stT0': th.empty_like(ss[0]),
                'sck0': th.empty(B, H, plan.nchunks, M, plan.NP)}}
        for i, x in enumerate(xs):
            good[f'in{{i}}'] = x
        buf, _ = cp._pack('frnn_fw', good)
        assert len(buf) == cp.kernels['frnn_fw'][1].arg_bytes
        def refused(change, msg):
            bad = dict(good); bad.update(change)
            try:
                cp._pack('frnn_fw', bad)
            except AssertionError as e:
                assert msg in str(e), (msg, str(e))
            else:
                raise SystemExit('accepted ' + str({{k: tuple(v.shape) for k, v in change.items()}}))
        refused({{'out0': th.empty(B, T - 1, H, M)}}, 'the kernel indexes')
        refused({{'sck0': th.empty(B, H, plan.nchunks - 1 or 2, M, plan.NP)}}, 'the kernel indexes')
        refused({{'in0': xs[0].to(th.bfloat16)}}, 'was emitted for')
        refused({{'sck0': th.empty(B, H, plan.nchunks, plan.NP, M).transpose(-1, -2)}}, 'must be contiguous')
        refused({{'st0': ss[0][:, :1]}}, 'the kernel indexes')
        try:
            cp._pack('frnn_fw', {{k: v for k, v in good.items() if k != 'out0'}})
        except AssertionError as e:
            assert 'takes a tensor called out0' in str(e), e
        else:
            raise SystemExit('packed without out0')
        cp._grid['frnn_fw'] = (cp._grid['frnn_fw'][0] + 1,) + cp._grid['frnn_fw'][1:]
        refused({{}}, 'does not cover')
        print('ok')
    ''')
    r = subprocess.run([sys.executable, '-c', code], capture_output=True, text=True)
    assert r.returncode == 0 and 'ok' in r.stdout, r.stdout + r.stderr
