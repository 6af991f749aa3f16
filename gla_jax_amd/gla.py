"""Gated Linear Attention on MI355X behind the reference's Python interface.

`chunk_gla`, `recurrent_gla` and `recurrent_gla_naive` keep the names, argument order
(hidden_init, log_fgate, value, key, query, ...), shapes and dtype rules of gla.py:657-692,
405-439 and 26-47 of zhixuan-lin/gla-jax.  Arrays are torch tensors on the GPU; the forward and
backward rules of the reference's `jax.custom_vjp` (gla.py:628-655, 362-388, 441) are
`torch.autograd.Function`s whose bodies are single calls into libgla_hip.so.  Batching: the
reference uses `jax.vmap` over a leading axis of all five arrays (gla.py:1335); here any number of
leading axes may simply be present, and `torch.func.vmap` works through the functions' vmap rule.

Shapes (unbatched):  hidden_init [H,DK,DV];  log_fgate, key, query [T,H,DK];  value [T,H,DV].
Returns (hidden_final [H,DK,DV] in hidden_init.dtype, out [T,H,DV] in value.dtype) — gla.py:538, 727.
"""
from __future__ import annotations

import torch

from . import _lib

_DT = {torch.float32: _lib.GLA_F32, torch.bfloat16: _lib.GLA_BF16}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _canon(hidden_init, log_fgate, value, key, query):
    """Checks the reference's shape contract and returns 4-D contiguous views
    (h0 [B,H,DK,DV], g/k/q [B,T,H,DK], v [B,T,H,DV]) plus the leading batch shape."""
    for name, t in (("hidden_init", hidden_init), ("log_fgate", log_fgate), ("value", value),
                    ("key", key), ("query", query)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor")
        if not t.is_cuda:
            raise ValueError(f"{name} must live on the GPU; gla_jax_amd has no CPU path")
    if key.ndim < 3:
        raise AssertionError("key must be [..., T, H, DK]")
    lead = tuple(key.shape[:-3])
    T, H, DK = key.shape[-3:]
    DV = value.shape[-1]
    if tuple(value.shape) != lead + (T, H, DV):
        raise AssertionError(f"value shape {tuple(value.shape)} != {lead + (T, H, DV)}")
    if tuple(query.shape) != tuple(key.shape) or tuple(log_fgate.shape) != tuple(key.shape):
        raise AssertionError("log_fgate, key and query must share one shape")          # gla.py:499
    if tuple(hidden_init.shape) != lead + (H, DK, DV):
        raise AssertionError(f"hidden_init shape {tuple(hidden_init.shape)} != {lead + (H, DK, DV)}")
    dt = value.dtype
    if dt not in _DT or key.dtype != dt or query.dtype != dt or hidden_init.dtype != dt:
        raise TypeError("hidden_init, value, key, query must share one dtype (float32 or bfloat16)")
    B = 1
    for s in lead:
        B *= s
    h0 = hidden_init.reshape(B, H, DK, DV).contiguous()
    g = log_fgate.reshape(B, T, H, DK).to(torch.float32).contiguous()      # gates are fp32 (gla.py:495)
    v = value.reshape(B, T, H, DV).contiguous()
    k = key.reshape(B, T, H, DK).contiguous()
    q = query.reshape(B, T, H, DK).contiguous()
    return (h0, g, v, k, q), lead, (B, T, H, DK, DV)


def _batched_vmap(fn_apply, n_tensor_args):
    """vmap rule shared by the Functions below: every tensor argument already accepts leading batch
    axes, so a vmapped call is the same call with the mapped axis moved to the front."""
    def rule(info, in_dims, *args):
        moved = []
        for a, d in zip(args[:n_tensor_args], in_dims[:n_tensor_args]):
            if d is None:
                a = a.unsqueeze(0).expand(info.batch_size, *a.shape)
            else:
                a = a.movedim(d, 0)
            moved.append(a)
        outs = fn_apply(*moved, *args[n_tensor_args:])
        return outs, tuple(0 for _ in outs)
    return rule


# ------------------------------------------------------------------------------------------------
# chunk_gla
# ------------------------------------------------------------------------------------------------
class _ChunkGLA(torch.autograd.Function):
    """forward = chunk_gla_forward (gla.py:483-550); backward = chunk_gla_backward (gla.py:552-625)."""

    @staticmethod
    def forward(hidden_init, log_fgate, value, key, query, chunk_size):
        (h0, g, v, k, q), lead, (B, T, H, DK, DV) = _canon(hidden_init, log_fgate, value, key, query)
        lib = _lib.load()
        dt = _DT[v.dtype]
        if DK != DV:
            raise AssertionError("chunk_gla needs key and value head dims to be equal")   # gla.py:499
        if chunk_size <= 0 or chunk_size & (chunk_size - 1):
            raise AssertionError(f"Chunk length must be power of 2, but got {chunk_size}")  # gla.py:500
        if T % chunk_size:
            raise AssertionError(f"sequence length {T} is not a multiple of chunk_size {chunk_size}")
        ws_bytes = lib.gla_chunk_fwd_workspace_bytes(B, T, H, DK, DV, chunk_size, dt)
        st_bytes = lib.gla_chunk_states_bytes(B, T, H, DK, DV, chunk_size, dt)
        if ws_bytes == 0 or st_bytes == 0:
            _lib.check("gla_chunk_fwd", -7)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device)
        states = torch.empty(st_bytes, dtype=torch.uint8, device=v.device)
        hT = torch.empty_like(h0)
        out = torch.empty_like(v)
        rc = lib.gla_chunk_fwd(_stream(), B, T, H, DK, DV, chunk_size, dt, _ptr(h0), _ptr(g), _ptr(v),
                               _ptr(k), _ptr(q), _ptr(hT), _ptr(out), _ptr(states), _ptr(ws), ws_bytes)
        _lib.check("gla_chunk_fwd", rc)
        return hT.reshape(lead + (H, DK, DV)), out.reshape(lead + (T, H, DV)), states

    @staticmethod
    def setup_context(ctx, inputs, output):
        hidden_init, log_fgate, value, key, query, chunk_size = inputs
        states = output[2]
        (_, g, v, k, q), lead, _ = _canon(hidden_init, log_fgate, value, key, query)
        ctx.save_for_backward(states, g, v, k, q)
        ctx.chunk_size = chunk_size
        ctx.lead = lead
        ctx.g_dtype = log_fgate.dtype
        ctx.mark_non_differentiable(states)

    @staticmethod
    def backward(ctx, dhT, dout, dstates=None):
        states, g, v, k, q = ctx.saved_tensors
        B, T, H, DK = k.shape
        DV = v.shape[-1]
        lib = _lib.load()
        dt = _DT[v.dtype]
        dhT = (torch.zeros(B, H, DK, DV, dtype=v.dtype, device=v.device) if dhT is None
               else dhT.reshape(B, H, DK, DV).to(v.dtype).contiguous())
        dout = (torch.zeros_like(v) if dout is None else dout.reshape(B, T, H, DV).to(v.dtype).contiguous())
        ws_bytes = lib.gla_chunk_bwd_workspace_bytes(B, T, H, DK, DV, ctx.chunk_size, dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device)
        dh0 = torch.empty_like(dhT)
        dg = torch.empty_like(g)
        dv, dk, dq = torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)
        rc = lib.gla_chunk_bwd(_stream(), B, T, H, DK, DV, ctx.chunk_size, dt, _ptr(g), _ptr(v), _ptr(k),
                               _ptr(q), _ptr(states), _ptr(dhT), _ptr(dout), _ptr(dh0), _ptr(dg),
                               _ptr(dv), _ptr(dk), _ptr(dq), _ptr(ws), ws_bytes)
        _lib.check("gla_chunk_bwd", rc)
        lead = ctx.lead
        return (dh0.reshape(lead + (H, DK, DV)), dg.reshape(lead + (T, H, DK)).to(ctx.g_dtype),
                dv.reshape(lead + (T, H, DV)), dk.reshape(lead + (T, H, DK)),
                dq.reshape(lead + (T, H, DK)), None)

    @staticmethod
    def vmap(info, in_dims, *args):
        outs, dims = _batched_vmap(_ChunkGLA.apply, 5)(info, in_dims, *args)
        # the residual is flattened over the batch; it carries no mapped axis of its own
        return outs, (0, 0, None)


def chunk_gla(hidden_init, log_fgate, value, key, query, chunk_size, block_size_t: int = 64,
              block_size_d: int = 64, interpret: bool = False, num_warps: int = 4, num_stages: int = 2):
    """Chunk-wise parallel form of gated linear attention (gla.py:657-692).

    Same result as `recurrent_gla_naive` up to rounding.  `chunk_size` must be a power of two that
    divides T (gla.py:500, 674), at least 32; since the result does not depend on it, the kernels run
    with the largest tile built that divides T, whatever size is given.  `block_size_t`, `block_size_d`, `interpret`, `num_warps`,
    `num_stages` tune the reference's Triton kernels; they are accepted for signature compatibility
    and have no effect here.  Differentiable in all five array arguments (gla.py:625)."""
    if interpret:
        raise ValueError("interpret=True asks for the reference's CPU interpreter; this build has no CPU path")
    hT, out = _ChunkGLA.apply(hidden_init, log_fgate, value, key, query, int(chunk_size))[:2]
    return hT, out


# ------------------------------------------------------------------------------------------------
# recurrent_gla / recurrent_gla_naive
# ------------------------------------------------------------------------------------------------
class _RecurrentGLA(torch.autograd.Function):
    """forward = recurrent_gla_forward (gla.py:99-170); backward = recurrent_gla_backward
    (gla.py:172-269).  `out_fp32` selects the fp32 output of the naive flavour (gla.py:37)."""

    @staticmethod
    def forward(hidden_init, log_fgate, value, key, query, reverse, out_fp32):
        (h0, g, v, k, q), lead, (B, T, H, DK, DV) = _canon(hidden_init, log_fgate, value, key, query)
        if DK != DV:
            raise AssertionError("Not supported yet: key and value head dims differ")      # gla.py:120, 391
        lib = _lib.load()
        dt = _DT[v.dtype]
        odt = _lib.GLA_F32 if out_fp32 else dt
        hT = torch.empty_like(h0)
        out = torch.empty(v.shape, dtype=torch.float32 if out_fp32 else v.dtype, device=v.device)
        rc = lib.gla_recurrent_fwd(_stream(), B, T, H, DK, DV, dt, odt, int(bool(reverse)), _ptr(h0),
                                   _ptr(g), _ptr(v), _ptr(k), _ptr(q), _ptr(hT), _ptr(out))
        _lib.check("gla_recurrent_fwd", rc)
        return hT.reshape(lead + (H, DK, DV)), out.reshape(lead + (T, H, DV))

    @staticmethod
    def setup_context(ctx, inputs, output):
        hidden_init, log_fgate, value, key, query, reverse, out_fp32 = inputs
        hT = output[0]
        (h0, g, v, k, q), lead, _ = _canon(hidden_init, log_fgate, value, key, query)
        ctx.save_for_backward(h0, g, v, k, q, hT)          # residuals of gla.py:169
        ctx.reverse = bool(reverse)
        ctx.out_fp32 = bool(out_fp32)
        ctx.lead = lead
        ctx.g_dtype = log_fgate.dtype

    @staticmethod
    def backward(ctx, dhT, dout):
        h0, g, v, k, q, hT = ctx.saved_tensors
        B, T, H, DK = k.shape
        DV = v.shape[-1]
        lib = _lib.load()
        dt = _DT[v.dtype]
        odt = _lib.GLA_F32 if ctx.out_fp32 else dt
        o_torch = torch.float32 if ctx.out_fp32 else v.dtype
        dhT = (torch.zeros_like(h0) if dhT is None else dhT.reshape(B, H, DK, DV).to(v.dtype).contiguous())
        dout = (torch.zeros(v.shape, dtype=o_torch, device=v.device) if dout is None
                else dout.reshape(B, T, H, DV).to(o_torch).contiguous())
        hTc = hT.reshape(B, H, DK, DV).contiguous()
        dh0 = torch.empty_like(h0)
        dg = torch.empty_like(g)
        dv, dk, dq = torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)
        rc = lib.gla_recurrent_bwd(_stream(), B, T, H, DK, DV, dt, odt, int(ctx.reverse), _ptr(h0), _ptr(g),
                                   _ptr(v), _ptr(k), _ptr(q), _ptr(hTc), _ptr(dhT), _ptr(dout),
                                   _ptr(dh0), _ptr(dg), _ptr(dv), _ptr(dk), _ptr(dq))
        _lib.check("gla_recurrent_bwd", rc)
        lead = ctx.lead
        return (dh0.reshape(lead + (H, DK, DV)), dg.reshape(lead + (T, H, DK)).to(ctx.g_dtype),
                dv.reshape(lead + (T, H, DV)), dk.reshape(lead + (T, H, DK)),
                dq.reshape(lead + (T, H, DK)), None, None)

    @staticmethod
    def vmap(info, in_dims, *args):
        outs, dims = _batched_vmap(_RecurrentGLA.apply, 5)(info, in_dims, *args)
        return outs, (0, 0)


def recurrent_gla(hidden_init, log_fgate, value, key, query, reverse: bool = False,
                  max_block_size: int = 64, num_warps: int = 1, num_stages: int = 1,
                  interpret: bool = False):
    """Recurrent form (gla.py:405-439): one rank-1 state update per timestep, the state never
    leaves registers.  `reverse` scans from the last timestep (gla.py:421-438).  `max_block_size`,
    `num_warps`, `num_stages`, `interpret` are the reference's Triton knobs: accepted, no effect."""
    if interpret:
        raise ValueError("interpret=True asks for the reference's CPU interpreter; this build has no CPU path")
    hT, out = _RecurrentGLA.apply(hidden_init, log_fgate, value, key, query, bool(reverse), False)[:2]
    return hT, out


def recurrent_gla_naive(hidden, log_fgate, value, key, query, reverse):
    """The definition (gla.py:26-47): S_t = exp(g_t)*S_{t-1} + k_t v_t^T, o_t = S_t^T q_t with an fp32
    state.  `out` comes back in float32 (promotion at gla.py:37), `hidden` in its input dtype
    (gla.py:46).  On this build it runs the same per-timestep HIP kernel as `recurrent_gla`, writing
    fp32 outputs."""
    hT, out = _RecurrentGLA.apply(hidden, log_fgate, value, key, query, bool(reverse), True)[:2]
    return hT, out
