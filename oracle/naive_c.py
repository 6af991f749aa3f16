"""ctypes front-end of oracle/libgla_naive.so (the C restatement of recurrent_gla_naive).

TEST INFRASTRUCTURE ONLY: used by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile libgla_naive.so with the Makefile beside this file."""
    so = os.path.join(_HERE, "libgla_naive.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libgla_naive.so")
        if not os.path.exists(so):
            build()
        _LIB = ctypes.CDLL(so)
        for sfx in ("f32", "f64"):
            getattr(_LIB, "gla_naive_fwd_" + sfx).restype = ctypes.c_int
            getattr(_LIB, "gla_naive_bwd_" + sfx).restype = ctypes.c_int
    return _LIB


def _prep(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def naive_fwd(h0, g, v, k, q, reverse=False, dtype=np.float32, nthreads=None):
    """[B,T,H,D] inputs, [B,H,DK,DV] hidden -> (hidden_final, out) in `dtype`."""
    dt = np.dtype(dtype)
    sfx = "f32" if dt == np.float32 else "f64"
    h0, g, v, k, q = (_prep(a, dt) for a in (h0, g, v, k, q))
    B, T, H, DK = k.shape
    DV = v.shape[-1]
    assert h0.shape == (B, H, DK, DV) and g.shape == k.shape == q.shape and v.shape == (B, T, H, DV)
    hT = np.empty_like(h0)
    out = np.empty_like(v)
    nt = nthreads or os.cpu_count() or 1
    rc = getattr(lib(), "gla_naive_fwd_" + sfx)(B, T, H, DK, DV, _ptr(h0), _ptr(g), _ptr(v), _ptr(k),
                                                 _ptr(q), int(bool(reverse)), _ptr(hT), _ptr(out), int(nt))
    if rc != 0:
        raise RuntimeError(f"gla_naive_fwd_{sfx} failed: {rc}")
    return hT, out


def naive_bwd(h0, g, v, k, q, dhT, dout, dtype=np.float32, nthreads=None):
    """Returns (dh0, dg, dv, dk, dq, hidden_final, out) in `dtype` (forward time direction)."""
    dt = np.dtype(dtype)
    sfx = "f32" if dt == np.float32 else "f64"
    h0, g, v, k, q, dhT, dout = (_prep(a, dt) for a in (h0, g, v, k, q, dhT, dout))
    B, T, H, DK = k.shape
    DV = v.shape[-1]
    assert h0.shape == dhT.shape == (B, H, DK, DV) and dout.shape == v.shape
    dh0, hT = np.empty_like(h0), np.empty_like(h0)
    dg, dk, dq = np.empty_like(g), np.empty_like(k), np.empty_like(q)
    dv, out = np.empty_like(v), np.empty_like(v)
    nt = nthreads or os.cpu_count() or 1
    rc = getattr(lib(), "gla_naive_bwd_" + sfx)(B, T, H, DK, DV, _ptr(h0), _ptr(g), _ptr(v), _ptr(k),
                                                 _ptr(q), _ptr(dhT), _ptr(dout), _ptr(dh0), _ptr(dg),
                                                 _ptr(dv), _ptr(dk), _ptr(dq), _ptr(hT), _ptr(out), int(nt))
    if rc != 0:
        raise RuntimeError(f"gla_naive_bwd_{sfx} failed: {rc}")
    return dh0, dg, dv, dk, dq, hT, out
