"""flex_rnn for AMD MI355X (gfx950): `@jit` compiles a single-timestep PyTorch function
into fused forward / recompute-backward HIP kernels.  Public surface as in the
reference package (/root/reference/flex_rnn/__init__.py:1-3)."""
from .jit import jit
from .layer import layer
from .check_grad import check_grad, benchmark

__version__ = '0.2'
