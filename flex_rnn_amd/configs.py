"""Synthetic workloads: the five benchmark configurations, with seeded inputs.

All values are drawn on the CPU in fp32 from `torch.Generator(seed)` and then cast
and moved, so a CPU checker and the GPU see identical numbers.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Callable, Dict, List, Tuple

import torch as th
import torch.nn.functional as F

from . import ops


@dataclass
class Workload:
    name: str
    step: Callable
    inputs: List[th.Tensor]
    states: List[th.Tensor]
    dims: Tuple[int, int, int, int, int]        # B, T, H, M, N
    dtype: th.dtype


DEFAULT_DIMS: Dict[str, Tuple[int, int, int, int, int]] = {
    'delta_rule': (1, 64, 2, 16, 16),
    'mamba1': (8, 1024, 32, 128, 16),
    'mamba2': (8, 1024, 64, 64, 128),
    'rwkv7': (8, 1024, 32, 128, 128),
    'gated_delta_rule': (4, 8192, 32, 128, 128),
}
DEFAULT_DTYPE = {
    'delta_rule': th.float32, 'mamba1': th.float32, 'mamba2': th.bfloat16,
    'rwkv7': th.bfloat16, 'gated_delta_rule': th.bfloat16,
}


def make(name: str, dims=None, dtype=None, device='cpu', seed: int = 0) -> Workload:
    B, T, H, M, N = dims or DEFAULT_DIMS[name]
    dtype = dtype or DEFAULT_DTYPE[name]
    g = th.Generator().manual_seed(seed)

    def randn(*shape):
        return th.randn(*shape, generator=g)

    def fin(x):
        return x.to(dtype).to(device)

    if name == 'delta_rule':
        q, k = randn(B, T, H, 1, N), F.normalize(randn(B, T, H, 1, N), dim=-1)
        v = randn(B, T, H, M, 1)
        beta = th.sigmoid(randn(B, T, H, 1, 1))
        S0 = th.zeros(B, H, M, N)
        step, xs = ops.delta_rule, [q, k, v, beta]
    elif name == 'mamba1':
        x = randn(B, T, H, M, 1)
        delta = F.softplus(randn(B, T, H, M, 1) - 3)
        A = -th.arange(1, N + 1, dtype=th.float32).view(1, 1, 1, 1, N).expand(1, 1, H, M, N).contiguous()
        Bm, Cm = randn(B, T, 1, 1, N), randn(B, T, 1, 1, N)
        S0 = th.zeros(B, H, M, N)
        step, xs = ops.mamba, [x, delta, A, Bm, Cm]
    elif name == 'mamba2':
        x = randn(B, T, H, M, 1)
        dt = F.softplus(randn(B, T, H, 1, 1) - 3)
        A = -th.exp(th.rand(1, 1, H, 1, 1, generator=g) * math.log(16))
        Bm, Cm = randn(B, T, 1, 1, N) / math.sqrt(N), randn(B, T, 1, 1, N) / math.sqrt(N)
        S0 = th.zeros(B, H, M, N)
        step, xs = ops.mamba2, [x, dt, A, Bm, Cm]
    elif name == 'rwkv7':
        r, k = randn(B, T, H, 1, N), randn(B, T, H, 1, N)
        w = th.exp(-th.exp(randn(B, T, H, 1, N) * 0.5 - 0.6))
        kk = F.normalize(randn(B, T, H, 1, N), dim=-1)
        a = -kk
        b = kk * th.sigmoid(randn(B, T, H, 1, N))
        v = randn(B, T, H, M, 1)
        S0 = randn(B, H, M, N) * 0.1
        step, xs = ops.rwkv7_decay, [r, w, k, v, a, b]
    elif name == 'gated_delta_rule':
        q = F.normalize(randn(B, T, H, 1, N), dim=-1)
        k = F.normalize(randn(B, T, H, 1, N), dim=-1)
        v = randn(B, T, H, M, 1)
        beta = th.sigmoid(randn(B, T, H, 1, 1))
        gate = th.exp(-F.softplus(randn(B, T, H, 1, 1)) * 0.1)
        S0 = th.zeros(B, H, M, N)
        step, xs = ops.gated_delta_rule_decay, [q, k, v, beta, gate]
    else:
        raise KeyError(name)
    return Workload(name, step, [fin(x) for x in xs], [fin(S0)], (B, T, H, M, N), dtype)


def upstream_grads(wl: Workload, jit_obj=None, seed: int = 1, device='cpu'):
    """N(0,1) cotangents for the output [B,T,H,M] and the final state [B,H,M,N]."""
    B, T, H, M, N = wl.dims
    g = th.Generator().manual_seed(seed)
    dy = th.randn(B, T, H, M, generator=g).to(device)
    dS = th.randn(B, H, M, N, generator=g).to(device)
    return [dy], [dS]
