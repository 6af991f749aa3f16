"""gla_jax_amd — Gated Linear Attention (zhixuan-lin/gla-jax's hot path) for AMD MI355X / gfx950.

Public surface, mirroring the reference's modules:
    gla.py : chunk_gla, recurrent_gla, recurrent_gla_naive
    ops.py : cumsum_recursive, rnn_recursive
All of them run hand-written HIP kernels from libgla_hip.so; there is no CPU or eager fallback.
"""
from . import _lib
from .gla import chunk_gla, recurrent_gla, recurrent_gla_naive
from .ops import cumsum_recursive, rnn_recursive

__all__ = ["chunk_gla", "recurrent_gla", "recurrent_gla_naive", "cumsum_recursive", "rnn_recursive"]
