"""GPU tests of the C-ABI runtime: compile -> load -> launch with a packed argument block.

The probe kernel only writes when two magic values in its argument block arrive intact, and
then only into a 256-entry buffer indexed by the thread id, so a broken launch path shows up
as zeros, not as a memory fault.
"""
import struct

import pytest
import torch as th

from flex_rnn_amd import runtime

pytestmark = pytest.mark.gpu

PROBE = r'''
#include <hip/hip_runtime.h>
typedef long long i64;
struct TArg { void* p; i64 s[5]; };
struct Args { TArg t[2]; i64 B, T, H, M, nch; };
template <int CTRL> __device__ __forceinline__ float dpp_mov(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
extern "C" __global__ void __launch_bounds__(64) frnn_probe(Args A) {
  if (A.nch != 0x5A5A1234 || A.t[1].s[4] != 0x1122334455667788LL) return;
  __shared__ float sh[64];
  const int tid = threadIdx.x;
  i64* out = (i64*)A.t[0].p;                       // 256 entries
  const int blk = blockIdx.x + 2 * blockIdx.y;     // grid (2, 2, 1)
  if (blk == 0) {
    // echo the second tensor slot and the scalars
    i64 v = tid;
    if (tid < 6) v = ((const i64*)&A.t[1])[tid];
    if (tid == 6) v = A.B;
    if (tid == 7) v = A.T;
    if (tid == 8) v = A.H;
    if (tid == 9) v = A.M;
    out[tid] = v;
  } else if (blk == 1) {
    // LDS + barrier + DPP all-reduce over 16 lanes
    sh[tid] = (float)tid;
    __syncthreads();
    float x = sh[63 - tid];
    x += dpp_mov<0xB1>(x);
    x += dpp_mov<0x4E>(x);
    x += dpp_mov<0x141>(x);
    x += dpp_mov<0x140>(x);
    out[64 + tid] = (i64)x;
  } else {
    out[blk * 64 + tid] = 1000 * blk + tid;
  }
}
'''


def test_probe_launch():
    path = runtime.compile_kernel('frnn_probe', PROBE)
    mod = runtime.Module(path)
    k = mod.kernel('frnn_probe')
    out = th.zeros(256, dtype=th.int64, device='cuda')
    buf = struct.pack('<q5q', out.data_ptr(), 1, 2, 3, 4, 5)
    buf += struct.pack('<q5q', 0x0BADC0DE, 11, 22, 33, 44, 0x1122334455667788)
    buf += struct.pack('<5q', 7, 8, 9, 10, 0x5A5A1234)
    stream = th.cuda.current_stream().cuda_stream
    k.launch((2, 2, 1), (64, 1, 1), buf, stream=stream)
    th.cuda.synchronize()
    got = out.cpu().tolist()
    assert got[:10] == [0x0BADC0DE, 11, 22, 33, 44, 0x1122334455667788, 7, 8, 9, 10], got[:10]
    assert got[10:64] == list(range(10, 64))
    # lanes hold 63 - tid; sum over each aligned group of 16 lanes
    want = []
    for tid in range(64):
        g = tid // 16
        want.append(sum(63 - t for t in range(16 * g, 16 * g + 16)))
    assert got[64:128] == want
    assert got[128:192] == [2000 + t for t in range(64)]
    assert got[192:256] == [3000 + t for t in range(64)]
    mod.close()


def test_device_cus():
    assert runtime.device_cus() > 0


def test_corrupt_cache_entry_is_rebuilt(tmp_path, monkeypatch):
    """A damaged code object in the cache is recompiled on load instead of failing for good."""
    import glob
    import os

    import flex_rnn_amd
    from flex_rnn_amd import ops
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    g = th.Generator().manual_seed(0)
    q, k = [th.randn(1, 16, 1, 1, 16, generator=g).cuda() for _ in range(2)]
    v = th.randn(1, 16, 1, 16, 1, generator=g).cuda()
    gate = -th.rand(1, 16, 1, 1, 16, generator=g).cuda()
    S = th.zeros(1, 1, 16, 16).cuda()
    y0, _ = flex_rnn_amd.jit(ops.gla)(q, k, v, gate, S)          # fills the cache
    files = glob.glob(os.path.join(str(tmp_path), 'frnn_fw_*.hsaco'))
    assert len(files) >= 1                                      # (one per candidate tile)
    for path in files:
        with open(path, 'wb') as f:
            f.write(b'not a code object')
    y1, _ = flex_rnn_amd.jit(ops.gla)(q, k, v, gate, S)          # new instance: loads from the cache
    th.cuda.synchronize()
    assert (y0 - y1).abs().max().item() < 1e-5 and all(os.path.getsize(p_) > 1000 for p_ in files)
