"""The scan operators of the reference's ops.py, on MI355X.

`cumsum_recursive` and `rnn_recursive` keep the reference's names, argument meaning and shape
checks (ops.py:234-284, 396-456); they call the HIP kernels of csrc/gla_scan.hip through the C ABI.
Inputs are CUDA(ROCm) torch tensors; math is float32 as in the reference kernels (ops.py:159-161,
312-315).  The blocking knob `block_size_t` is accepted and ignored: the kernels need no recursion.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _require_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("gla_jax_amd operators need tensors on the GPU; there is no CPU path")


def cumsum_recursive(src: torch.Tensor, axis: int, init: Optional[torch.Tensor] = None,
                     reverse: bool = False, block_size_t: int = 2048) -> torch.Tensor:
    """Inclusive cumulative sum of `src` along `axis` plus `init` (shape = src.shape without `axis`),
    from the far end when `reverse` (ops.py:234-284).  Computed in float32, returned in src.dtype."""
    _require_cuda(src, init)
    axis = axis % src.ndim
    pre, T, post = src.shape[:axis], src.shape[axis], src.shape[axis + 1:]
    if init is not None and tuple(init.shape) != tuple(pre + post):
        raise AssertionError(f"init shape {tuple(init.shape)} != {tuple(pre + post)}")   # ops.py:254
    n_outer = 1
    for s in pre:
        n_outer *= s
    n_inner = 1
    for s in post:
        n_inner *= s
    x = src.contiguous().to(torch.float32)
    i = None if init is None else init.contiguous().to(torch.float32)
    dst = torch.empty_like(x)
    lib = _lib.load()
    # grid.y carries the outer index: split very large outer counts
    step = 65535
    for o0 in range(0, n_outer, step):
        o1 = min(n_outer, o0 + step)
        off = o0 * T * n_inner * 4
        rc = lib.gla_cumsum_f32(_stream(), x.data_ptr() + off,
                                None if i is None else i.data_ptr() + o0 * n_inner * 4,
                                dst.data_ptr() + off, o1 - o0, T, n_inner, int(bool(reverse)))
        _lib.check("gla_cumsum_f32", rc)
    return dst.to(src.dtype)


def rnn_recursive(log_fgate: torch.Tensor, kv: torch.Tensor,
                  init_log_fgate: Optional[torch.Tensor] = None, init_kv: Optional[torch.Tensor] = None,
                  block_size_t: int = 256, reverse: bool = False):
    """Diagonal linear recurrence x_n = exp(a_n)[:,None] * x_{n-1} + b_n over the leading axis of
    log_fgate [T,K] / kv [T,K,V] with optional initial pair, backwards in n when `reverse`
    (ops.py:396-456).  Returns (running sum of a, states), states in kv.dtype (ops.py:373-374).
    A leading batch axis on all arguments is accepted."""
    _require_cuda(log_fgate, kv, init_log_fgate, init_kv)
    if (init_log_fgate is None) != (init_kv is None):
        raise AssertionError("init_log_fgate and init_kv go together")                   # ops.py:407
    batched = kv.ndim == 4
    a = log_fgate if batched else log_fgate[None]
    b = kv if batched else kv[None]
    Bn, T, K, V = b.shape
    if tuple(a.shape) != (Bn, T, K):
        raise AssertionError(f"log_fgate shape {tuple(log_fgate.shape)} does not match kv")  # ops.py:405
    af = a.contiguous().to(torch.float32)
    bf = b.contiguous().to(torch.float32)
    ia = ib = None
    if init_kv is not None:
        ia = (init_log_fgate if batched else init_log_fgate[None]).contiguous().to(torch.float32)
        ib = (init_kv if batched else init_kv[None]).contiguous().to(torch.float32)
    out_a = torch.empty_like(af)
    out_x = torch.empty_like(bf)
    rc = _lib.load().gla_rnn_scan_f32(_stream(), af.data_ptr(), bf.data_ptr(),
                                      None if ia is None else ia.data_ptr(),
                                      None if ib is None else ib.data_ptr(),
                                      out_a.data_ptr(), out_x.data_ptr(), Bn, T, K, V, int(bool(reverse)))
    _lib.check("gla_rnn_scan_f32", rc)
    out_a = out_a.to(log_fgate.dtype)
    out_x = out_x.to(kv.dtype)
    if not batched:
        out_a, out_x = out_a[0], out_x[0]
    return out_a, out_x
