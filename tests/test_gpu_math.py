"""Accuracy of the emitter's fast math helpers (reciprocal-based division, sigmoid, tanh, the cancellation-free
log1p) on the GPU against fp64: they replace correctly rounded library routines inside every generated kernel."""
import struct

import pytest
import torch as th

from flex_rnn_amd import runtime
from flex_rnn_amd.emit_hip import PRELUDE

pytestmark = pytest.mark.gpu

PROBE = PRELUDE + r'''
struct Args { const float* a; const float* b; float* o; long long n; };
extern "C" __global__ void __launch_bounds__(256) frnn_math_probe(Args A) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= A.n) return;
  const float a = A.a[i], b = A.b[i];
  A.o[i] = f_div(a, b);
  A.o[A.n + i] = f_rcp(b);
  A.o[2 * A.n + i] = f_log1p(a);
  A.o[3 * A.n + i] = f_sigmoid(a);
  A.o[4 * A.n + i] = f_tanh(a);
}
'''


def _run(a, b):
    n = a.numel()
    out = th.empty(5, n, dtype=th.float32, device=a.device)
    mod = runtime.Module(runtime.compile_kernel('frnn_math_probe', PROBE))
    kern = mod.kernel('frnn_math_probe')
    args = struct.pack('<QQQq', a.data_ptr(), b.data_ptr(), out.data_ptr(), n)
    kern.launch((-(-n // 256), 1, 1), (256, 1, 1), args, stream=th.cuda.current_stream().cuda_stream)
    th.cuda.synchronize()
    return out.double()


def _rel(x, ref):
    return ((x - ref).abs() / ref.abs().clamp_min(1e-300)).max().item()


def test_fast_math_helpers_against_fp64():
    dev = th.device('cuda:0')
    g = th.Generator().manual_seed(0)
    n = 1 << 16
    # quotients over 60 binades either side, divisors up to the top of the fp32 range
    a = (th.randn(n, generator=g) * th.exp2(th.randint(-60, 60, (n,), generator=g).float())).to(dev)
    b = (th.randn(n, generator=g).abs().add(0.1) * th.exp2(th.randint(-60, 126, (n,), generator=g).float())
         * (th.randint(0, 2, (n,), generator=g) * 2 - 1)).to(dev)
    out = _run(a, b)
    q = a.double() / b.double()
    ok = q.abs() > 1e-30                     # (a quotient in the denormals is flushed, like every fp32 result here)
    assert _rel(out[0][ok], q[ok]) < 4e-7
    big = b.abs() < 1e37                     # (the reciprocal of anything larger is a denormal)
    assert _rel(out[1][big], 1.0 / b.double()[big]) < 2.5e-7
    # log1p: tiny, ordinary and large arguments, negative ones down to -0.99
    x = th.cat([th.exp2(th.linspace(-40, 30, n // 2)), -th.exp2(th.linspace(-40, -0.015, n // 2))]).to(dev)
    out = _run(x, th.ones_like(x))
    assert _rel(out[2], th.log1p(x.double())) < 1e-6
    # sigmoid and tanh over the range where they are not saturated, absolute error
    x = th.linspace(-30, 30, n).to(dev)
    out = _run(x, th.ones_like(x))
    assert (out[3] - th.sigmoid(x.double())).abs().max().item() < 2e-7
    assert (out[4] - th.tanh(x.double())).abs().max().item() < 4e-7
    # edge values: 0, 1 + x rounding to 1, -1, overflow of exp
    x = th.tensor([0.0, 1e-10, -1e-10, -1.0, 100.0, -100.0], device=dev)
    out = _run(x, th.ones_like(x)).float()
    assert out[2][0] == 0.0 and out[2][1] == x[1] and out[2][2] == x[2] and out[2][3] == float('-inf')
    assert out[3][4] == 1.0 and out[3][5] == 0.0 and out[4][4] == 1.0 and out[4][5] == -1.0
