"""CPU-side checks of the drop-in boundary: libgla_hip.so loads, exports every symbol that
include/gla_hip.h declares, rejects bad arguments on the host before any launch, and the Python
front-end refuses to run without the GPU path (there is no CPU fallback)."""
import ctypes
import os
import re

import pytest
import torch

from gla_jax_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gla_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gla_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_typed():
    names = declared_symbols()
    assert len(names) >= 13
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in gla_hip.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature in gla_jax_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == names
    header = open(os.path.join(ROOT, "include", "gla_hip.h")).read()
    assert _lib.load().gla_abi_version() == _lib.ABI_VERSION == int(
        re.search(r"#define GLA_HIP_ABI_VERSION (\d+)", header).group(1))
    # every ctypes signature lists as many arguments as the header declares
    from tests.test_xla_ffi_shim import declared
    for n, count in declared().items():
        assert len(_lib.SIGNATURES[n][1]) == count, f"{n}: {len(_lib.SIGNATURES[n][1])} ctypes arguments, {count} declared"


def test_status_strings():
    for code in range(-7, 1):
        assert len(_lib.status_string(code)) > 1
    assert "chunk" in _lib.status_string(-4)


def test_chunk_plan_and_sizes():
    lib = _lib.load()
    B, T, H, D = 4, 4096, 6, 128
    n_chunks = T // 128
    st = lib.gla_chunk_states_bytes(B, T, H, D, D, 128, _lib.GLA_BF16)
    assert st == B * H * (n_chunks + 1) * D * D * 2      # states before every chunk + the final one
    ws = lib.gla_chunk_fwd_workspace_bytes(B, T, H, D, D, 128, _lib.GLA_BF16)
    # per chunk: the products (16-bit mantissas for bf16 data), the decays, an exponent byte per 16 products, the
    # chunk-start state in the orientation the output kernel reads
    per_chunk = D * D * 2 + D * 4 + D * D // 16 + D * D * 2
    assert B * H * n_chunks * per_chunk <= ws <= B * H * n_chunks * per_chunk + 3 * 256
    assert lib.gla_chunk_fwd_workspace_bytes(B, T, H, D, D, 128, _lib.GLA_F32) >= B * H * 4 * n_chunks * (
        D * D * 4 + D * 4 + D * D * 4)                       # fp32 data: float products, 32-token tiles
    # the tile is the largest one built that divides T, whatever chunk_size says; unsupported combinations report 0
    assert lib.gla_chunk_states_bytes(B, T, H, D, D, 256, _lib.GLA_BF16) == st
    assert lib.gla_chunk_states_bytes(B, T, H, D, D, 32, _lib.GLA_BF16) == st
    assert lib.gla_chunk_states_bytes(B, 64 * 65, H, D, D, 32, _lib.GLA_BF16) == B * H * (65 + 1) * D * D * 2
    assert lib.gla_chunk_states_bytes(B, T, H, D, D, 16, _lib.GLA_BF16) == 0      # below the reference's own minimum
    assert lib.gla_chunk_states_bytes(B, T, H, D, D, 96, _lib.GLA_BF16) == 0      # not a power of two
    assert lib.gla_chunk_states_bytes(B, 100, H, D, D, 64, _lib.GLA_BF16) == 0    # does not divide T
    assert lib.gla_chunk_states_bytes(B, T, H, 128, 64, 128, _lib.GLA_BF16) == 0  # DK != DV
    # fp32 at D=128 runs on the 32-token tile: 4x as many chunks, 4-byte elements
    assert lib.gla_chunk_states_bytes(B, T, H, D, D, 128, _lib.GLA_F32) == B * H * (4 * n_chunks + 1) * D * D * 4
    # head dims built: 32, 64, 128; 256 runs as two passes of the 128-feature kernels over twice the heads
    assert lib.gla_chunk_states_bytes(B, T, H, 32, 32, 128, _lib.GLA_BF16) == B * H * (n_chunks + 1) * 32 * 32 * 2
    assert lib.gla_chunk_states_bytes(B, T, H, 32, 32, 128, _lib.GLA_F32) == B * H * (2 * n_chunks + 1) * 32 * 32 * 4
    # head dim 16 runs on the 32-feature kernels: the library's own buffers are sized for 32 x 32 states
    assert lib.gla_chunk_states_bytes(B, T, H, 16, 16, 128, _lib.GLA_BF16) == B * H * (n_chunks + 1) * 32 * 32 * 2
    assert lib.gla_chunk_states_bytes(B, T, H, 8, 8, 128, _lib.GLA_BF16) == 0
    assert lib.gla_chunk_states_bytes(B, T, H, 256, 256, 128, _lib.GLA_BF16) == 2 * lib.gla_chunk_states_bytes(
        B, T, 2 * H, 128, 128, 128, _lib.GLA_BF16) == B * H * (n_chunks + 1) * 256 * 256 * 2
    assert lib.gla_chunk_states_bytes(B, T, H, 256, 256, 128, _lib.GLA_F32) == B * H * (4 * n_chunks + 1) * 256 * 256 * 4
    # its workspace: one pass's, the value-side arrays with their halves exchanged, both passes' results in fp32
    # (out; dq, dk, dv, and the second pass's d(log_fgate)) and the states cut into blocks
    rows = B * T * H * 256 * 2
    hid = 4 * B * H * 256 * 256 * 2
    sub = lib.gla_chunk_fwd_workspace_bytes(B, T, 2 * H, 128, 128, 128, _lib.GLA_BF16)
    assert sub + 5 * rows + hid <= lib.gla_chunk_fwd_workspace_bytes(B, T, H, 256, 256, 128, _lib.GLA_BF16) <= (
        sub + 5 * rows + hid + 8 * 256)
    sub = lib.gla_chunk_bwd_workspace_bytes(B, T, 2 * H, 128, 128, 128, _lib.GLA_BF16)
    assert sub + 16 * rows + hid <= lib.gla_chunk_bwd_workspace_bytes(B, T, H, 256, 256, 128, _lib.GLA_BF16) <= (
        sub + 16 * rows + hid + 12 * 256)
    assert lib.gla_chunk_states_bytes(B, T, H, 512, 512, 128, _lib.GLA_BF16) == 0
    # recurrent_gla: a workspace at head dimension 256 (both passes' results in fp32 and the exchanged rows) and, at
    # every head dimension, where the sequences are few enough to run as S >= 4 segments of >= 128 steps side by
    # side (B*H*S <= 256 workgroups; S = 2 already for bf16 data at head dimensions 64 and more): the segments'
    # states in fp32, twice (backward: four times), and their gate sums
    r256 = lambda x: (x + 255) & ~255
    for D in (16, 32, 64, 128):
        assert lib.gla_recurrent_fwd_workspace_bytes(16, 2048, 16, D, D, _lib.GLA_BF16) == 0    # 256 sequences
        assert lib.gla_recurrent_bwd_workspace_bytes(16, 2048, 8, D, D, _lib.GLA_F32) == 0      # 128: S would be 2
        assert lib.gla_recurrent_fwd_workspace_bytes(1, 200, 2, D, D, _lib.GLA_BF16) == 0       # segments below 128 steps
        # (bf16 data at head dimension 128: the first pass takes every segment in F = 2 pieces, so its array of
        # contributions and the gate sums count twice)
        F = 2 if D == 128 else 1
        two = lib.gla_recurrent_fwd_workspace_bytes(16, 2048, 8, D, D, _lib.GLA_BF16)           # 128 sequences: S = 2
        assert two == ((1 + F) * r256(16 * 2 * 8 * D * D * 4) + r256(16 * 2 * F * 8 * D * 4) if D >= 64 else 0)
        S = 8                                                                                   # 24 sequences of 4096 steps
        hid, sums = r256(B * S * H * D * D * 4), r256(B * S * H * D * 4)
        assert lib.gla_recurrent_fwd_workspace_bytes(B, T, H, D, D, _lib.GLA_BF16) == (1 + F) * hid + F * sums
        assert lib.gla_recurrent_bwd_workspace_bytes(B, T, H, D, D, _lib.GLA_BF16) == (2 + 2 * F) * hid + F * sums
        assert lib.gla_recurrent_bwd_workspace_bytes(B, T, H, D, D, _lib.GLA_F32) == 4 * hid + sums
    assert lib.gla_recurrent_fwd_workspace_bytes(1, 1024, 64, 64, 64, _lib.GLA_BF16) == 2 * r256(4 * 64 * 64 * 64 * 4) + (
        r256(4 * 64 * 64 * 4))                                                                  # S = 4, the smallest
    rows32 = B * T * H * 256 * 4
    assert lib.gla_recurrent_fwd_workspace_bytes(B, T, H, 256, 128, _lib.GLA_BF16) == 0      # DK != DV: unsupported


def test_entry_points_reject_bad_arguments_without_touching_the_gpu():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    a = (ctypes.addressof(buf) + 15) & ~15          # a 16-byte aligned, non-null host address (never dereferenced)
    # NULL pointers
    assert lib.gla_cumsum_f32(None, None, None, a, 1, 8, 8, 0) == -1
    assert lib.gla_recurrent_fwd(None, 1, 8, 1, 64, 64, 1, 1, 1, 0, None, a, a, a, a, a, a) == -1
    # shapes / dtypes
    assert lib.gla_cumsum_f32(None, a, None, a, 0, 8, 8, 0) == -2
    assert lib.gla_recurrent_fwd(None, 1, 8, 1, 48, 48, 1, 1, 1, 0, a, a, a, a, a, a, a) == -2
    assert lib.gla_recurrent_fwd(None, 1, 8, 1, 64, 32, 1, 1, 1, 0, a, a, a, a, a, a, a) == -2   # DK != DV
    assert lib.gla_recurrent_fwd(None, 1, 8, 1, 64, 64, 5, 1, 1, 0, a, a, a, a, a, a, a) == -3
    assert lib.gla_recurrent_fwd(None, 1, 8, 1, 64, 64, 1, 7, 1, 0, a, a, a, a, a, a, a) == -3   # hidden dtype
    assert lib.gla_rnn_scan_f32(None, a, a, None, None, None, a, 1, 4, 4, 0, 0) == -2
    assert lib.gla_rnn_scan_f32(None, a, a + 4, None, None, None, a, 1, 4, 4, 8, 0) == -6      # 16-byte rows
    # misaligned
    assert lib.gla_recurrent_fwd(None, 1, 8, 1, 64, 64, 1, 1, 1, 0, a + 2, a, a, a, a, a, a) == -6
    # the workspace variants: ignored where none is needed, checked at head dimension 256
    rec = lambda D, ws, n: lib.gla_recurrent_fwd_ws(None, 1, 8, 1, D, D, 1, 1, 1, 0, a, a, a, a, a, a, a, ws, n)
    assert rec(48, None, 0) == -2
    assert rec(256, None, 0) == -5
    assert rec(256, a, 64) == -5
    # ... and where few long sequences run as segments (one sequence of 1024 steps: four segments)
    seg = lambda ws, n: lib.gla_recurrent_fwd_ws(None, 1, 1024, 1, 64, 64, 1, 1, 1, 0, a, a, a, a, a, a, a, ws, n)
    assert lib.gla_recurrent_fwd_workspace_bytes(1, 1024, 1, 64, 64, 1) > 64
    assert seg(None, 0) == -5 and seg(a, 64) == -5 and seg(a + 4, 1 << 30) == -6
    assert lib.gla_recurrent_bwd_ws(None, 1, 8, 1, 256, 256, 1, 1, 1, 0, a, a, a, a, a, a, a, a, a, a, a, a, a,
                                    a, 64) == -5
    assert lib.gla_recurrent_bwd_ws(None, 1, 8, 1, 256, 256, 1, 1, 1, 0, a, a, a, a, a, a, a, a, a, a, a, a, None,
                                    a, 1 << 40) == -1
    # chunk: not a power of two / not dividing T / unsupported head dim / missing workspace
    args = lambda T, D, C, hd=0: (None, 1, T, 1, D, D, C, 1, hd, a, a, a, a, a, a, a, a)
    assert lib.gla_chunk_fwd(*args(256, 64, 48), a, 1 << 30) == -4
    assert lib.gla_chunk_fwd(*args(200, 64, 64), a, 1 << 30) == -4
    assert lib.gla_chunk_fwd(*args(256, 96, 64), a, 1 << 30) == -7
    assert lib.gla_chunk_fwd(*args(256, 64, 64), None, 0) == -5
    assert lib.gla_chunk_fwd(*args(256, 64, 64), a, 16) == -5
    assert lib.gla_chunk_fwd(*args(256, 64, 64, hd=3), a, 1 << 30) == -3
    assert lib.gla_chunk_bwd(None, 1, 256, 1, 64, 64, 64, 1, 1, a, a, a, a, None, a, a, a, a, a, a, a, a, 1 << 30) == -1


def test_front_end_has_no_cpu_path():
    from gla_jax_amd import chunk_gla, cumsum_recursive, recurrent_gla
    T, H, D = 64, 1, 64
    h0 = torch.zeros(H, D, D)
    x = torch.zeros(T, H, D)
    with pytest.raises(ValueError, match="GPU"):
        chunk_gla(h0, x, x, x, x, 64)
    with pytest.raises(ValueError, match="GPU"):
        recurrent_gla(h0, x, x, x, x)
    with pytest.raises(ValueError, match="GPU"):
        cumsum_recursive(x, 0)


def test_oracle_is_not_imported_by_the_product():
    import glob
    for f in glob.glob(os.path.join(ROOT, "gla_jax_amd", "*.py")):
        src = open(f).read()
        assert "oracle" not in src, f"{f} mentions the oracle: the product path must not depend on it"


def test_canonical_arrays_pass_through_untouched():
    """The host layer adds no op (and no autograd node) for an array that is already dense, shaped and typed as the
    kernels take it, and converts everything else differentiably."""
    import torch
    from gla_jax_amd import gla
    t = torch.randn(2, 5, 3, 4, requires_grad=True)
    assert gla._as(t, (2, 5, 3, 4), torch.float32) is t
    u = gla._as(t, (10, 3, 4), torch.float32)                    # other shape: a view with a node
    assert u.shape == (10, 3, 4) and u.grad_fn is not None
    w = gla._as(t.transpose(0, 1), (5, 2, 3, 4), torch.float32)  # not dense: a copy
    assert w.is_contiguous() and w.grad_fn is not None
    b = gla._as(t, (2, 5, 3, 4), torch.bfloat16)
    assert b.dtype == torch.bfloat16 and b.grad_fn is not None
    # every Function has a twin in the older style that shares its forward, context and backward
    for cls in (gla._ChunkGLA, gla._ChunkGLABwd, gla._RecurrentGLA, gla._RecurrentGLABwd):
        assert issubclass(cls._twin, torch.autograd.Function) and cls._twin.backward is cls.backward
