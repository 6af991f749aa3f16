"""ctypes binding of libgla_hip.so (see include/gla_hip.h for the contract of every symbol).

There is no fallback: if the library is missing or a symbol is absent the import fails, and every
wrapper raises on a non-zero status."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgla_hip.so")

GLA_F32, GLA_BF16 = 0, 1
ABI_VERSION = 3                             # GLA_HIP_ABI_VERSION of include/gla_hip.h
GLA_CHUNK_FWD_STATIC_BYTES = 80 << 20      # capacity of gla_chunk_fwd_static's workspace (gla_hip.h)

_i64, _int, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol declared in include/gla_hip.h
SIGNATURES = {
    "gla_abi_version": (_int, []),
    "gla_status_string": (ctypes.c_char_p, [_int]),
    "gla_cumsum_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int]),
    "gla_rnn_scan_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int]),
    "gla_recurrent_fwd": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _int] + [_vp] * 7),
    "gla_recurrent_bwd": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _int] + [_vp] * 13),
    "gla_recurrent_fwd_workspace_bytes": (_sz, [_i64] * 5 + [_int]),
    "gla_recurrent_bwd_workspace_bytes": (_sz, [_i64] * 5 + [_int]),
    "gla_recurrent_fwd_ws": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _int] + [_vp] * 8 + [_sz]),
    "gla_recurrent_bwd_ws": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _int] + [_vp] * 14 + [_sz]),
    "gla_chunk_states_bytes": (_sz, [_i64] * 6 + [_int]),
    "gla_chunk_fwd_workspace_bytes": (_sz, [_i64] * 6 + [_int]),
    "gla_chunk_bwd_workspace_bytes": (_sz, [_i64] * 6 + [_int]),
    "gla_chunk_fwd": (_int, [_vp] + [_i64] * 6 + [_int, _int] + [_vp] * 9 + [_sz]),
    "gla_chunk_bwd": (_int, [_vp] + [_i64] * 6 + [_int, _int] + [_vp] * 13 + [_sz]),
    "gla_chunk_fwd_static": (_int, [_vp] + [_i64] * 6 + [_int, _int] + [_vp] * 8),
    "gla_chunk_fwd_stages": (_int, [_vp, _int] + [_i64] * 6 + [_int, _int] + [_vp] * 9 + [_sz]),
    "gla_chunk_bwd_stages": (_int, [_vp, _int] + [_i64] * 6 + [_int, _int] + [_vp] * 13 + [_sz]),
}

_lib = None


class GlaError(RuntimeError):
    def __init__(self, fn, status, text):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


def load():
    """Loads the library once and types every entry point.  Raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m gla_jax_amd.build` "
            "(hipcc, gfx950).  There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if lib.gla_abi_version() != ABI_VERSION:
        raise ImportError(f"libgla_hip.so ABI {lib.gla_abi_version()} != {ABI_VERSION}: rebuild it "
                          "(`python -m gla_jax_amd.build`)")
    _lib = lib
    return lib


def status_string(status: int) -> str:
    return load().gla_status_string(int(status)).decode()


def check(fn: str, status: int):
    if status != 0:
        raise GlaError(fn, status, status_string(status))
