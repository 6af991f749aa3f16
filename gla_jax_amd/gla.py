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


def _prep(hidden_init, log_fgate, value, key, query):
    """Checks the reference's shape contract and returns the canonical 4-D views the kernels take
    (h0 [B,H,DK,DV], g/k/q [B,T,H,DK], v [B,T,H,DV]; dense, gates fp32, hidden in its own dtype when that is
    float32 or bfloat16, else in float32), the leading batch shape and the dims.  Everything here is a differentiable torch op (reshape, cast, copy),
    so autograd carries gradients back to the caller's own layouts and dtypes; for arrays that are
    already dense and typed as the kernels want them nothing is copied."""
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
    if dt not in _DT or key.dtype != dt or query.dtype != dt:
        raise TypeError("value, key, query must share one dtype (float32 or bfloat16)")
    if not hidden_init.dtype.is_floating_point:
        raise TypeError("hidden_init must be a floating-point tensor")
    B = 1
    for s in lead:
        B *= s
    # the state enters the kernels in its own dtype: the reference loads it uncast into an fp32 state
    # (gla.py:44, 89; the chunk scan takes it uncast too, gla.py:711-716) and stores hidden_final back in
    # hidden_init's dtype (gla.py:46, 97, 727).  Other float types (half, double) go through float32.
    h0 = _as(hidden_init, (B, H, DK, DV), hidden_init.dtype if hidden_init.dtype in _DT else torch.float32)
    g = _as(log_fgate, (B, T, H, DK), torch.float32)                       # gates are fp32 (gla.py:495)
    v = _as(value, (B, T, H, DV), dt)
    k = _as(key, (B, T, H, DK), dt)
    q = _as(query, (B, T, H, DK), dt)
    return (h0, g, v, k, q), lead, (B, T, H, DK, DV)


def _as(t, shape, dtype):
    """`t` dense, in `shape` and `dtype`: the tensor itself when it already is (no op, no autograd node: a step
    at the benchmark shape is bound by the host, every node costs microseconds), else a differentiable copy."""
    if tuple(t.shape) == shape and t.dtype == dtype and t.is_contiguous():
        return t
    return t.reshape(shape).to(dtype).contiguous()


_transforms_active = getattr(torch._C, "_are_functorch_transforms_active", None)


def _twin(cls):
    """A twin of a setup_context-style Function in the older style (forward takes ctx).  `Function.apply` of the
    newer style binds the arguments through `inspect.signature` on every call (tens of microseconds), which it
    needs for function transforms only; `_apply` picks the twin when no transform is active."""
    class Twin(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *args):
            out = cls.forward(*args)
            cls.setup_context(ctx, args, out)
            return out

        backward = staticmethod(cls.backward)

    Twin.__name__ = Twin.__qualname__ = cls.__name__ + "Twin"
    return Twin


def _apply(cls, *args):
    if _transforms_active is None or _transforms_active():
        return cls.apply(*args)
    return cls._twin.apply(*args)


def _merge_mapped(info, in_dims, tensors):
    """vmap rule helper: every Function below takes canonical arrays with ONE batch axis in front, so a mapped
    call is the same call with the mapped axis folded into that batch axis.  Unmapped arguments are
    broadcast.  Flat byte buffers (the residual of chunk_gla) carry no axis of their own and pass through."""
    out = []
    for a, d in zip(tensors, in_dims):
        if a.dtype == torch.uint8:
            out.append(a)
            continue
        a = a.unsqueeze(0).expand(info.batch_size, *a.shape) if d is None else a.movedim(d, 0)
        out.append(a.reshape((a.shape[0] * a.shape[1],) + tuple(a.shape[2:])))
    return out


def _split_mapped(info, outs):
    return tuple(o if o.dtype == torch.uint8 else o.reshape((info.batch_size, -1) + tuple(o.shape[1:]))
                 for o in outs)


def _no_double_backward(name):
    raise NotImplementedError(f"{name}: second-order gradients are not provided "
                              "(the reference defines first-order custom_vjp rules only)")


# ------------------------------------------------------------------------------------------------
# chunk_gla
# ------------------------------------------------------------------------------------------------
def _chunk_forward(h0, g, v, k, q, chunk_size, residual):
    """One call of gla_chunk_fwd on canonical arrays; `residual` False: no chunk states are kept."""
    # the kernels take dense arrays by address; a transform may hand over views (a broadcast hidden_init)
    h0, g, v, k, q = (t.contiguous() for t in (h0, g, v, k, q))
    B, T, H, DK = k.shape
    DV = v.shape[-1]
    lib = _lib.load()
    dt = _DT[v.dtype]
    ws_bytes = lib.gla_chunk_fwd_workspace_bytes(B, T, H, DK, DV, chunk_size, dt)
    st_bytes = lib.gla_chunk_states_bytes(B, T, H, DK, DV, chunk_size, dt)
    if ws_bytes == 0 or st_bytes == 0:
        _lib.check("gla_chunk_fwd", -7)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device)
    # without a residual (nothing to differentiate) the scan skips the [dk][dv] copy of the chunk states
    states = torch.empty(st_bytes, dtype=torch.uint8, device=v.device) if residual else None
    hT = torch.empty_like(h0)
    out = torch.empty_like(v)
    rc = lib.gla_chunk_fwd(_stream(), B, T, H, DK, DV, chunk_size, dt, _DT[h0.dtype], _ptr(h0), _ptr(g), _ptr(v),
                           _ptr(k), _ptr(q), _ptr(hT), _ptr(out), _ptr(states), _ptr(ws), ws_bytes)
    _lib.check("gla_chunk_fwd", rc)
    return hT, out, states


class _ChunkGLA(torch.autograd.Function):
    """forward = chunk_gla_forward (gla.py:483-550); backward = chunk_gla_backward (gla.py:552-625).
    Arguments are the canonical arrays of `_prep`."""

    @staticmethod
    def forward(h0, g, v, k, q, chunk_size):
        return _chunk_forward(h0, g, v, k, q, chunk_size, True)

    @staticmethod
    def setup_context(ctx, inputs, output):
        h0, g, v, k, q, chunk_size = inputs
        states = output[2]
        ctx.save_for_backward(states, g, v, k, q)          # residuals of gla.py:542-549
        ctx.chunk_size = chunk_size
        ctx.hidden_dtype = h0.dtype
        ctx.mark_non_differentiable(states)
        # no zeros for the cotangents nobody computed: `states` would get a 25 MB fill per step at B4 T4096 H6 D128;
        # backward() makes the zeros that hidden_final and out need
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, dhT, dout, dstates=None):
        states, g, v, k, q = ctx.saved_tensors
        B, T, H, DK = k.shape
        DV = v.shape[-1]
        dhT = torch.zeros(B, H, DK, DV, dtype=ctx.hidden_dtype, device=v.device) if dhT is None else dhT
        dout = torch.zeros_like(v) if dout is None else dout
        return _apply(_ChunkGLABwd, states, g, v, k, q, dhT, dout, ctx.chunk_size) + (None,)

    @staticmethod
    def vmap(info, in_dims, *args):
        outs = _ChunkGLA.apply(*_merge_mapped(info, in_dims[:5], args[:5]), args[5])
        # the residual is one flat buffer over the merged batch; it carries no mapped axis of its own
        return _split_mapped(info, outs), (0, 0, None)


class _ChunkGLABwd(torch.autograd.Function):
    """The backward rule as a function of its own, so that function transforms (torch.func.grad, vmap of a
    gradient) reach the kernels with plain tensors."""

    @staticmethod
    def forward(states, g, v, k, q, dhT, dout, chunk_size):
        states, g, v, k, q = (t.contiguous() for t in (states, g, v, k, q))
        B, T, H, DK = k.shape
        DV = v.shape[-1]
        lib = _lib.load()
        dt = _DT[v.dtype]
        # the cotangent of hidden_final arrives in the state's dtype; dhidden_init goes back in it
        dhT = dhT.to(dhT.dtype if dhT.dtype in _DT else torch.float32).contiguous()
        dout = dout.to(v.dtype).contiguous()
        ws_bytes = lib.gla_chunk_bwd_workspace_bytes(B, T, H, DK, DV, chunk_size, dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device)
        dh0 = torch.empty_like(dhT)
        dg = torch.empty_like(g)
        dv, dk, dq = torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)
        rc = lib.gla_chunk_bwd(_stream(), B, T, H, DK, DV, chunk_size, dt, _DT[dhT.dtype], _ptr(g), _ptr(v), _ptr(k),
                               _ptr(q), _ptr(states), _ptr(dhT), _ptr(dout), _ptr(dh0), _ptr(dg),
                               _ptr(dv), _ptr(dk), _ptr(dq), _ptr(ws), ws_bytes)
        _lib.check("gla_chunk_bwd", rc)
        return dh0, dg, dv, dk, dq

    @staticmethod
    def setup_context(ctx, inputs, output):
        pass

    @staticmethod
    def backward(ctx, *grads):
        _no_double_backward("chunk_gla")

    @staticmethod
    def vmap(info, in_dims, *args):
        outs = _ChunkGLABwd.apply(*_merge_mapped(info, in_dims[:7], args[:7]), args[7])
        return _split_mapped(info, outs), (0,) * 5


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
    chunk_size = int(chunk_size)
    (h0, g, v, k, q), lead, (B, T, H, DK, DV) = _prep(hidden_init, log_fgate, value, key, query)
    if DK != DV:
        raise AssertionError("chunk_gla needs key and value head dims to be equal")   # gla.py:499
    if chunk_size <= 0 or chunk_size & (chunk_size - 1):
        raise AssertionError(f"Chunk length must be power of 2, but got {chunk_size}")  # gla.py:500
    if T % chunk_size:
        raise AssertionError(f"sequence length {T} is not a multiple of chunk_size {chunk_size}")
    if _transforms_active is not None and not _transforms_active() and not (
            torch.is_grad_enabled() and any(t.requires_grad for t in (h0, g, v, k, q))):
        hT, out, _ = _chunk_forward(h0, g, v, k, q, chunk_size, False)
    else:
        hT, out = _apply(_ChunkGLA, h0, g, v, k, q, chunk_size)[:2]
    return _as(hT, lead + (H, DK, DV), hidden_init.dtype), _as(out, lead + (T, H, DV), out.dtype)


# ------------------------------------------------------------------------------------------------
# recurrent_gla / recurrent_gla_naive
# ------------------------------------------------------------------------------------------------
class _RecurrentGLA(torch.autograd.Function):
    """forward = recurrent_gla_forward (gla.py:99-170); backward = recurrent_gla_backward
    (gla.py:172-269).  `out_fp32` selects the fp32 output of the naive flavour (gla.py:37).
    Arguments are the canonical arrays of `_prep`."""

    @staticmethod
    def forward(h0, g, v, k, q, reverse, out_fp32):
        h0, g, v, k, q = (t.contiguous() for t in (h0, g, v, k, q))
        B, T, H, DK = k.shape
        DV = v.shape[-1]
        lib = _lib.load()
        dt = _DT[v.dtype]
        odt = _lib.GLA_F32 if out_fp32 else dt
        hT = torch.empty_like(h0)
        out = torch.empty(v.shape, dtype=torch.float32 if out_fp32 else v.dtype, device=v.device)
        # a workspace where the library can use one: head dimension 256 (two passes of the 128-feature kernels) and
        # few long sequences (each runs as segments side by side); zero bytes elsewhere
        ws_bytes = lib.gla_recurrent_fwd_workspace_bytes(B, T, H, DK, DV, dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device) if ws_bytes else None
        rc = lib.gla_recurrent_fwd_ws(_stream(), B, T, H, DK, DV, dt, _DT[h0.dtype], odt, int(bool(reverse)), _ptr(h0),
                                      _ptr(g), _ptr(v), _ptr(k), _ptr(q), _ptr(hT), _ptr(out),
                                      _ptr(ws) if ws_bytes else None, ws_bytes)
        _lib.check("gla_recurrent_fwd_ws", rc)
        return hT, out

    @staticmethod
    def setup_context(ctx, inputs, output):
        h0, g, v, k, q, reverse, out_fp32 = inputs
        ctx.save_for_backward(h0, g, v, k, q, output[0])          # residuals of gla.py:169
        ctx.reverse = bool(reverse)
        ctx.out_fp32 = bool(out_fp32)

    @staticmethod
    def backward(ctx, dhT, dout):
        h0, g, v, k, q, hT = ctx.saved_tensors
        o_torch = torch.float32 if ctx.out_fp32 else v.dtype
        dhT = torch.zeros_like(h0) if dhT is None else dhT
        dout = torch.zeros(v.shape, dtype=o_torch, device=v.device) if dout is None else dout
        return _apply(_RecurrentGLABwd, h0, g, v, k, q, hT, dhT, dout, ctx.reverse, ctx.out_fp32) + (None, None)

    @staticmethod
    def vmap(info, in_dims, *args):
        outs = _RecurrentGLA.apply(*_merge_mapped(info, in_dims[:5], args[:5]), args[5], args[6])
        return _split_mapped(info, outs), (0, 0)


class _RecurrentGLABwd(torch.autograd.Function):
    """The backward rule of recurrent_gla as a function of its own (see _ChunkGLABwd)."""

    @staticmethod
    def forward(h0, g, v, k, q, hT, dhT, dout, reverse, out_fp32):
        h0, g, v, k, q = (t.contiguous() for t in (h0, g, v, k, q))
        B, T, H, DK = k.shape
        DV = v.shape[-1]
        lib = _lib.load()
        dt = _DT[v.dtype]
        odt = _lib.GLA_F32 if out_fp32 else dt
        dhT = dhT.to(h0.dtype).contiguous()                # the four state arrays share hidden_init's dtype
        dout = dout.to(torch.float32 if out_fp32 else v.dtype).contiguous()
        hTc = hT.to(h0.dtype).contiguous()
        dh0 = torch.empty_like(h0)
        dg = torch.empty_like(g)
        dv, dk, dq = torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)
        ws_bytes = lib.gla_recurrent_bwd_workspace_bytes(B, T, H, DK, DV, dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device) if ws_bytes else None
        rc = lib.gla_recurrent_bwd_ws(_stream(), B, T, H, DK, DV, dt, _DT[h0.dtype], odt, int(bool(reverse)), _ptr(h0),
                                      _ptr(g), _ptr(v), _ptr(k), _ptr(q), _ptr(hTc), _ptr(dhT), _ptr(dout),
                                      _ptr(dh0), _ptr(dg), _ptr(dv), _ptr(dk), _ptr(dq),
                                      _ptr(ws) if ws_bytes else None, ws_bytes)
        _lib.check("gla_recurrent_bwd_ws", rc)
        return dh0, dg, dv, dk, dq

    @staticmethod
    def setup_context(ctx, inputs, output):
        pass

    @staticmethod
    def backward(ctx, *grads):
        _no_double_backward("recurrent_gla")

    @staticmethod
    def vmap(info, in_dims, *args):
        outs = _RecurrentGLABwd.apply(*_merge_mapped(info, in_dims[:8], args[:8]), args[8], args[9])
        return _split_mapped(info, outs), (0,) * 5


def _recurrent(hidden_init, log_fgate, value, key, query, reverse, out_fp32):
    (h0, g, v, k, q), lead, (B, T, H, DK, DV) = _prep(hidden_init, log_fgate, value, key, query)
    if DK != DV:
        raise AssertionError("Not supported yet: key and value head dims differ")      # gla.py:120, 391
    pad = 16 - DK if DK < 16 else 0
    if pad:
        # Head dims below 16 (the reference packs several such heads into one tile, gla.py:60-62): the kernels' smallest
        # state is 16 x 16, so the rows are padded with zeros here (a zero key, query and value feature with gate 0
        # leaves the rest of the state and of the output untouched) and the results cut back.
        F = torch.nn.functional
        h0 = F.pad(h0, (0, pad, 0, pad))
        g, v, k, q = (F.pad(x, (0, pad)) for x in (g, v, k, q))
    hT, out = _apply(_RecurrentGLA, h0, g, v, k, q, bool(reverse), bool(out_fp32))
    if pad:
        hT, out = hT[..., :DK, :DV], out[..., :DV]
    return _as(hT, lead + (H, DK, DV), hidden_init.dtype), _as(out, lead + (T, H, DV), out.dtype)


def recurrent_gla(hidden_init, log_fgate, value, key, query, reverse: bool = False,
                  max_block_size: int = 64, num_warps: int = 1, num_stages: int = 1,
                  interpret: bool = False):
    """Recurrent form (gla.py:405-439): one rank-1 state update per timestep, the state never
    leaves registers.  `reverse` scans from the last timestep (gla.py:421-438).  `max_block_size`,
    `num_warps`, `num_stages`, `interpret` are the reference's Triton knobs: accepted, no effect."""
    if interpret:
        raise ValueError("interpret=True asks for the reference's CPU interpreter; this build has no CPU path")
    return _recurrent(hidden_init, log_fgate, value, key, query, reverse, False)


def recurrent_gla_naive(hidden, log_fgate, value, key, query, reverse):
    """The definition (gla.py:26-47): S_t = exp(g_t)*S_{t-1} + k_t v_t^T, o_t = S_t^T q_t with an fp32
    state.  `out` comes back in float32 (promotion at gla.py:37), `hidden` in its input dtype
    (gla.py:46).  On this build it runs the same per-timestep HIP kernel as `recurrent_gla`, writing
    fp32 outputs."""
    return _recurrent(hidden, log_fgate, value, key, query, reverse, True)


for _cls in (_ChunkGLA, _ChunkGLABwd, _RecurrentGLA, _RecurrentGLABwd):
    _cls._twin = _twin(_cls)
