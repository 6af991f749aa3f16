"""chunk_gla / recurrent_gla / recurrent_gla_naive and the ops.py scans for JAX-ROCm, on the gfx950 kernels of
libgla_hip.so through XLA FFI custom calls.  This is the module a maintainer of zhixuan-lin/gla-jax would put
in place of the Pallas/Triton bodies: same function names, argument order (hidden_init, log_fgate, value,
key, query), shapes, dtype rules and `jax.custom_vjp` structure as gla.py:405-441, 628-692 and ops.py:234-284,
396-456; batching through `jax.vmap` (the handlers are registered with vmap_method="broadcast_all", so mapped
axes become leading dimensions that the C ABI takes as its batch argument).

STATUS: source only.  Neither `jax` nor `jaxlib` (nor xla/ffi/api/ffi.h) exists on the machines this library
was built and tested on, so nothing in this file has run; importing it without jax raises ImportError.  The
tested front-end of the same C ABI is gla_jax_amd/gla.py (torch tensors, torch.autograd.Function).

Build the handler library first (gla_jax_amd/build.py::build_xla_ffi compiles gla_xla_ffi.cc against
jaxlib's headers and links it with libgla_hip.so).
"""
from __future__ import annotations

import ctypes
import functools
import os

try:
    import jax
    import jax.numpy as jnp
except ImportError as e:          # pragma: no cover - no jax on the build machines
    raise ImportError("gla_jax_amd.xla_ffi.gla_jax needs jax with a ROCm jaxlib; the torch front-end "
                      "gla_jax_amd.gla works without it") from e

_HERE = os.path.dirname(os.path.abspath(__file__))
_HIP = ctypes.CDLL(os.path.join(_HERE, "..", "libgla_hip.so"), mode=ctypes.RTLD_GLOBAL)
_FFI = ctypes.CDLL(os.path.join(_HERE, "libgla_xla_ffi.so"))
for _name in ("GlaChunkFwd", "GlaChunkBwd", "GlaRecurrentFwd", "GlaRecurrentBwd", "GlaCumsum", "GlaRnnScan"):
    jax.ffi.register_ffi_target(_name, jax.ffi.pycapsule(getattr(_FFI, _name)), platform="ROCM")

for _fn in ("gla_chunk_states_bytes", "gla_chunk_fwd_workspace_bytes", "gla_chunk_bwd_workspace_bytes"):
    getattr(_HIP, _fn).restype = ctypes.c_size_t
    getattr(_HIP, _fn).argtypes = [ctypes.c_int64] * 6 + [ctypes.c_int]

for _fn in ("gla_recurrent_fwd_workspace_bytes", "gla_recurrent_bwd_workspace_bytes"):
    getattr(_HIP, _fn).restype = ctypes.c_size_t
    getattr(_HIP, _fn).argtypes = [ctypes.c_int64] * 5 + [ctypes.c_int]

_GLA_F32, _GLA_BF16 = 0, 1


def _dt(dtype):
    if dtype == jnp.bfloat16:
        return _GLA_BF16
    if dtype == jnp.float32:
        return _GLA_F32
    raise TypeError(f"value, key, query must be float32 or bfloat16, got {dtype}")


def _sizes(key, value, chunk_size):
    """(states bytes, forward workspace bytes, backward workspace bytes) for arrays [..., T, H, D]."""
    *lead, T, H, DK = key.shape
    DV = value.shape[-1]
    B = 1
    for s in lead:
        B *= s
    args = (B, T, H, DK, DV, chunk_size, _dt(value.dtype))
    st, wf, wb = (getattr(_HIP, f)(*args) for f in
                  ("gla_chunk_states_bytes", "gla_chunk_fwd_workspace_bytes", "gla_chunk_bwd_workspace_bytes"))
    if st == 0 or wf == 0 or wb == 0:
        raise AssertionError(f"chunk_gla: unsupported shape/chunk_size {key.shape}, {chunk_size}")   # gla.py:499-500
    return st, wf, wb


def _like(x, dtype=None):
    return jax.ShapeDtypeStruct(x.shape, x.dtype if dtype is None else dtype)


def _state(hidden):
    """The state as the kernels take it: in its own dtype when that is float32 or bfloat16 (the reference loads
    hidden_init uncast into an fp32 state, gla.py:44, 89, and hands it uncast to the chunk scan, gla.py:711-716),
    through float32 otherwise."""
    return hidden if hidden.dtype in (jnp.float32, jnp.bfloat16) else hidden.astype(jnp.float32)


# ---------------------------------------------------------------------------------------------- chunk_gla
@functools.partial(jax.custom_vjp, nondiff_argnums=(5,))
def chunk_gla_forward_backward(hidden_init, log_fgate, value, key, query, chunk_size):      # gla.py:628-655
    return _chunk_fwd(hidden_init, log_fgate, value, key, query, chunk_size)[0]


def _chunk_fwd(hidden_init, log_fgate, value, key, query, chunk_size):
    st, wf, _ = _sizes(key, value, chunk_size)
    h0 = _state(hidden_init)
    g = log_fgate.astype(jnp.float32)
    hT, out, states, _ws = jax.ffi.ffi_call(
        "GlaChunkFwd",
        (_like(h0), _like(value), jax.ShapeDtypeStruct((st,), jnp.uint8), jax.ShapeDtypeStruct((wf,), jnp.uint8)),
        vmap_method="broadcast_all")(h0, g, value, key, query, chunk_size=int(chunk_size))
    return (hT.astype(hidden_init.dtype), out), (g, value, key, query, states, hidden_init.dtype, log_fgate.dtype)


def _chunk_bwd(chunk_size, res, cotangents):
    g, value, key, query, states, h_dtype, g_dtype = res
    dhT, dout = cotangents
    _, _, wb = _sizes(key, value, chunk_size)
    dh0, dg, dv, dk, dq, _ws = jax.ffi.ffi_call(
        "GlaChunkBwd",
        (_like(_state(dhT)), _like(g), _like(value), _like(key), _like(query),
         jax.ShapeDtypeStruct((wb,), jnp.uint8)),
        vmap_method="broadcast_all")(g, value, key, query, states, _state(dhT),
                                     dout.astype(value.dtype), chunk_size=int(chunk_size))
    return dh0.astype(h_dtype), dg.astype(g_dtype), dv, dk, dq                                 # gla.py:625


chunk_gla_forward_backward.defvjp(_chunk_fwd, _chunk_bwd)


def chunk_gla(hidden_init, log_fgate, value, key, query, chunk_size, block_size_t=64, block_size_d=64,
              interpret=False, num_warps=4, num_stages=2):
    """gla.py:657-692.  Unbatched [T,H,D] arrays or any leading batch axes; the Triton knobs are accepted
    and have no effect.  Note that under vmap the flat `states` residual is sized for the unbatched call
    and broadcast_all prepends the mapped axis to it as to every other result."""
    assert key.shape[-1] == value.shape[-1], "chunk_gla needs key and value head dims to be equal"   # gla.py:499
    assert chunk_size > 0 and chunk_size & (chunk_size - 1) == 0, \
        f"Chunk length must be power of 2, but got {chunk_size}"                                   # gla.py:500
    assert key.shape[-3] % chunk_size == 0                                                         # gla.py:674
    return chunk_gla_forward_backward(hidden_init, log_fgate, value, key, query, int(chunk_size))


# ------------------------------------------------------------------------------------------ recurrent_gla
@functools.partial(jax.custom_vjp, nondiff_argnums=(5, 6))
def recurrent_gla_forward_backward(hidden_init, log_fgate, value, key, query, reverse, out_fp32):   # gla.py:362-388
    return _rec_fwd(hidden_init, log_fgate, value, key, query, reverse, out_fp32)[0]


def _rec_workspace(key, value, which):
    """The workspace of a recurrent_gla call as a byte array (head dimension 256 and calls with few long sequences
    use one; elsewhere 16 bytes that nobody reads)."""
    *lead, T, H, DK = key.shape
    B = 1
    for s in lead:
        B *= s
    n = getattr(_HIP, f"gla_recurrent_{which}_workspace_bytes")(B, T, H, DK, value.shape[-1], _dt(value.dtype))
    return jax.ShapeDtypeStruct((max(int(n), 16),), jnp.uint8)


def _rec_fwd(hidden_init, log_fgate, value, key, query, reverse, out_fp32):
    h0 = _state(hidden_init)
    g = log_fgate.astype(jnp.float32)
    hT, out, _ws = jax.ffi.ffi_call(
        "GlaRecurrentFwd", (_like(h0), _like(value, jnp.float32 if out_fp32 else None),
                            _rec_workspace(key, value, "fwd")),
        vmap_method="broadcast_all")(h0, g, value, key, query, reverse=bool(reverse))
    res = (h0, g, value, key, query, hT, hidden_init.dtype, log_fgate.dtype)                     # gla.py:169
    return (hT.astype(hidden_init.dtype), out), res


def _rec_bwd(reverse, out_fp32, res, cotangents):
    h0, g, value, key, query, hT, h_dtype, g_dtype = res
    dhT, dout = cotangents
    dh0, dg, dv, dk, dq, _ws = jax.ffi.ffi_call(
        "GlaRecurrentBwd", (_like(h0), _like(g), _like(value), _like(key), _like(query),
                            _rec_workspace(key, value, "bwd")),
        vmap_method="broadcast_all")(h0, g, value, key, query, hT, dhT.astype(h0.dtype),
                                     dout.astype(jnp.float32 if out_fp32 else value.dtype),
                                     reverse=bool(reverse))
    return dh0.astype(h_dtype), dg.astype(g_dtype), dv, dk, dq                                   # gla.py:269


recurrent_gla_forward_backward.defvjp(_rec_fwd, _rec_bwd)


def recurrent_gla(hidden_init, log_fgate, value, key, query, reverse=False, max_block_size=64, num_warps=1,
                  num_stages=1, interpret=False):
    """gla.py:405-439; `max_block_size`, `num_warps`, `num_stages`, `interpret` are accepted and ignored."""
    assert key.shape[-1] == value.shape[-1], "Not supported yet"                                  # gla.py:120, 391
    return recurrent_gla_forward_backward(hidden_init, log_fgate, value, key, query, bool(reverse), False)


def recurrent_gla_naive(hidden, log_fgate, value, key, query, reverse):
    """gla.py:26-47: fp32 `out` (gla.py:37), `hidden` in its own dtype (gla.py:46)."""
    return recurrent_gla_forward_backward(hidden, log_fgate, value, key, query, bool(reverse), True)


# --------------------------------------------------------------------------------------------- ops.py scans
def cumsum_recursive(src, axis, init=None, reverse=False, block_size_t=2048):
    """ops.py:234-284: fp32 inclusive cumulative sum along `axis` plus `init` (shape of src without that
    axis); `block_size_t` is the reference's recursion knob and has no effect."""
    src32 = src.astype(jnp.float32)
    axis = axis % src.ndim
    init32 = (jnp.zeros(src.shape[:axis] + src.shape[axis + 1:], jnp.float32) if init is None
              else jnp.broadcast_to(init, src.shape[:axis] + src.shape[axis + 1:]).astype(jnp.float32))
    out = jax.ffi.ffi_call("GlaCumsum", _like(src32), vmap_method="sequential")(
        src32, init32, axis=int(axis), reverse=bool(reverse))
    return out.astype(src.dtype)


def rnn_recursive(log_fgate, kv, init_log_fgate=None, init_kv=None, block_size_t=256, reverse=False):
    """ops.py:396-456: x_n = exp(a_n)[:,None] * x_{n-1} + b_n with an optional initial pair (reverse: from the
    far end); returns (running sum of a including its init, states).  fp32 arithmetic, results in the input
    dtypes.  `block_size_t` is the reference's recursion knob and has no effect."""
    assert (init_log_fgate is None) == (init_kv is None), "init_log_fgate and init_kv go together"   # ops.py:407
    a, b = log_fgate.astype(jnp.float32), kv.astype(jnp.float32)
    if init_kv is None:                      # the reference starts from a zero gate sum and a zero state
        ia = jnp.zeros(a.shape[:-2] + a.shape[-1:], jnp.float32)
        ib = jnp.zeros(b.shape[:-3] + b.shape[-2:], jnp.float32)
    else:
        ia, ib = init_log_fgate.astype(jnp.float32), init_kv.astype(jnp.float32)
    oa, ob = jax.ffi.ffi_call("GlaRnnScan", (_like(a), _like(b)), vmap_method="broadcast_all")(
        a, b, ia, ib, reverse=bool(reverse))
    return oa.astype(log_fgate.dtype), ob.astype(kv.dtype)
