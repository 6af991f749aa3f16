"""gla_chunk_fwd_static, the forward entry point that allocates nothing (its workspace is a static device
array inside the library), through the C ABI against gla_chunk_fwd with a caller-allocated workspace: bit-equal
outputs on two calls in a row, the second on a smaller input, then on the largest shape that fits; shapes
beyond the static array are rejected before any launch."""
import pytest
import torch

from tests.util import gpu_inputs

pytestmark = pytest.mark.gpu


def _run_pair(lib, _lib, B, T, H, D, chunk, seed, dtype=torch.bfloat16):
    _, dev = gpu_inputs(B, T, H, D, 2.0, seed=seed, dtype=dtype)
    h0, g, v, k, q = dev
    dt = _lib.GLA_BF16 if dtype == torch.bfloat16 else _lib.GLA_F32
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    wsb = lib.gla_chunk_fwd_workspace_bytes(B, T, H, D, D, chunk, dt)
    stb = lib.gla_chunk_states_bytes(B, T, H, D, D, chunk, dt)
    assert 0 < wsb <= _lib.GLA_CHUNK_FWD_STATIC_BYTES
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    outs = []
    for static in (False, True):
        hT, out = torch.full_like(h0, float("nan")), torch.full_like(v, float("nan"))
        states = torch.zeros(stb, dtype=torch.uint8, device="cuda")
        if static:
            rc = lib.gla_chunk_fwd_static(st, B, T, H, D, D, chunk, dt, dt, p(h0), p(g), p(v), p(k), p(q), p(hT), p(out),
                                          p(states))
        else:
            rc = lib.gla_chunk_fwd(st, B, T, H, D, D, chunk, dt, dt, p(h0), p(g), p(v), p(k), p(q), p(hT), p(out),
                                   p(states), p(ws), wsb)
        _lib.check("gla_chunk_fwd_static" if static else "gla_chunk_fwd", rc)
        outs.append((hT, out, states))
    torch.cuda.synchronize()
    for name, a, b in zip(("hidden_final", "out", "states"), outs[0], outs[1]):
        assert torch.isfinite(a.float()).all() if a.dtype != torch.uint8 else True
        assert torch.equal(a, b), f"{name} of gla_chunk_fwd_static differs from gla_chunk_fwd at {(B, T, H, D)}"


def test_static_entry_point_matches_the_workspace_one():
    from gla_jax_amd import _lib
    lib = _lib.load()
    _run_pair(lib, _lib, 2, 512, 3, 128, 128, seed=21)           # first call on this device: looks the array up
    _run_pair(lib, _lib, 1, 128, 2, 64, 64, seed=22)             # a smaller input right after: stale contents around it
    _run_pair(lib, _lib, 2, 96, 1, 64, 32, seed=23, dtype=torch.float32)
    _run_pair(lib, _lib, 4, 4096, 6, 128, 128, seed=24)          # the headline shape: 49.1 of the 80 MiB
    _run_pair(lib, _lib, 1, 256, 2, 256, 128, seed=25)           # head dimension 256: two passes inside the same array


def test_static_entry_point_rejects_what_does_not_fit():
    from gla_jax_amd import _lib
    lib = _lib.load()
    B, T, H, D = 8, 4096, 6, 128                                  # needs 98.25 MiB
    assert lib.gla_chunk_fwd_workspace_bytes(B, T, H, D, D, 128, _lib.GLA_BF16) > _lib.GLA_CHUNK_FWD_STATIC_BYTES
    x = torch.zeros(16, device="cuda")                             # never touched: the call is refused on the host
    rc = lib.gla_chunk_fwd_static(torch.cuda.current_stream().cuda_stream, B, T, H, D, D, 128, _lib.GLA_BF16,
                                  _lib.GLA_BF16,
                                  *([x.data_ptr()] * 8))
    assert rc == -5
    with pytest.raises(_lib.GlaError, match="workspace"):
        _lib.check("gla_chunk_fwd_static", rc)


def test_static_entry_point_allocates_nothing_and_replays_from_a_graph():
    """After a first call on the device (which looks up the array's address), a call of gla_chunk_fwd_static
    leaves the free device memory and torch's allocator untouched, and it can be recorded into a HIP graph:
    every replay, on new inputs copied into the same buffers and with eager work in between, equals
    gla_chunk_fwd on those inputs bit for bit."""
    from gla_jax_amd import _lib
    lib = _lib.load()
    B, T, H, D, chunk = 2, 512, 2, 128, 128
    dt = _lib.GLA_BF16
    p = lambda t: t.data_ptr()
    _, dev = gpu_inputs(B, T, H, D, 2.0, seed=31, dtype=torch.bfloat16)
    h0, g, v, k, q = dev
    hT, out = torch.empty_like(h0), torch.empty_like(v)
    wsb = lib.gla_chunk_fwd_workspace_bytes(B, T, H, D, D, chunk, dt)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    hT_e, out_e = torch.empty_like(h0), torch.empty_like(v)

    def static(stream):
        _lib.check("gla_chunk_fwd_static", lib.gla_chunk_fwd_static(stream, B, T, H, D, D, chunk, dt, dt, p(h0), p(g),
                                                                    p(v), p(k), p(q), p(hT), p(out), None))

    def eager():
        _lib.check("gla_chunk_fwd", lib.gla_chunk_fwd(torch.cuda.current_stream().cuda_stream, B, T, H, D, D, chunk,
                                                      dt, dt, p(h0), p(g), p(v), p(k), p(q), p(hT_e), p(out_e), None,
                                                      p(ws), wsb))

    static(torch.cuda.current_stream().cuda_stream)           # warm-up outside any capture
    torch.cuda.synchronize()
    free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    static(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the call changed the free device memory"
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static(torch.cuda.current_stream().cuda_stream)
    for it in range(3):
        _, fresh = gpu_inputs(B, T, H, D, 2.0, seed=40 + it, dtype=torch.bfloat16)
        for dst, src in zip(dev, fresh):
            dst.copy_(src)                                    # eager work between the replays
        hT.fill_(float("nan"))
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        eager()
        torch.cuda.synchronize()
        assert torch.equal(hT, hT_e) and torch.equal(out, out_e), f"replay {it} differs from gla_chunk_fwd"
