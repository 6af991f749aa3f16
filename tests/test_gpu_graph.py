"""The C ABI under HIP graph capture: the entry points only enqueue kernels on the given stream (no
allocation, no synchronisation, no memset nodes), so a caller may record a forward + backward step into a
graph and replay it.  Every replay is checked against the eager result, with eager work and
synchronisations between the replays."""
import pytest
import torch

from tests.util import gpu_inputs, to_dev, cotangents

pytestmark = pytest.mark.gpu


def _buffers(B, T, H, D, chunk, dtype):
    from gla_jax_amd import _lib
    lib = _lib.load()
    dt = _lib.GLA_BF16
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, 3.0, seed=77, dtype=dtype)
    dhT, dout = cotangents(h0, v, 9, dtype)
    dev += [to_dev(dhT, dtype), to_dev(dout, dtype)]
    u8 = lambda n: torch.empty(n, dtype=torch.uint8, device="cuda")
    ws_f = u8(lib.gla_chunk_fwd_workspace_bytes(B, T, H, D, D, chunk, dt))
    ws_b = u8(lib.gla_chunk_bwd_workspace_bytes(B, T, H, D, D, chunk, dt))
    states = u8(lib.gla_chunk_states_bytes(B, T, H, D, D, chunk, dt))
    return lib, dt, dev, ws_f, ws_b, states


@pytest.mark.parametrize("D", [128, 256])
def test_chunk_step_replays_from_a_graph(D):
    """D=256 runs as two passes of the 128-feature kernels with copies and sums between them: all of them are
    kernels on the caller's stream, so the whole sequence records and replays like a single pass."""
    from gla_jax_amd import _lib
    B, T, H, chunk = 2, 512, 2, 128
    dtype = torch.bfloat16
    lib, dt, (h0, g, v, k, q, dhT, dout), ws_f, ws_b, states = _buffers(B, T, H, D, chunk, dtype)
    outs = lambda: [torch.empty_like(h0), torch.empty_like(v), torch.empty_like(h0), torch.empty_like(g),
                    torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)]
    p = lambda t: t.data_ptr()

    def step(stream, o):
        hT, out, dh0, dg, dv, dk, dq = o
        _lib.check("gla_chunk_fwd", lib.gla_chunk_fwd(stream, B, T, H, D, D, chunk, dt, dt, p(h0), p(g), p(v), p(k),
                                                      p(q), p(hT), p(out), p(states), p(ws_f), ws_f.numel()))
        _lib.check("gla_chunk_bwd", lib.gla_chunk_bwd(stream, B, T, H, D, D, chunk, dt, dt, p(g), p(v), p(k), p(q),
                                                      p(states), p(dhT), p(dout), p(dh0), p(dg), p(dv), p(dk),
                                                      p(dq), p(ws_b), ws_b.numel()))

    eager = outs()
    step(torch.cuda.current_stream().cuda_stream, eager)      # also sets the kernels' LDS limits before capture
    torch.cuda.synchronize()

    replayed = outs()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream().cuda_stream, replayed)
    for it in range(3):
        for t in replayed:
            t.fill_(float("nan"))                             # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("hidden_final", "out", "dh0", "dg", "dv", "dk", "dq"), eager, replayed):
            assert torch.equal(a, b), f"replay {it}: {name} differs from the eager result"


@pytest.mark.parametrize("D", [32, 64])
def test_recurrent_step_replays_from_a_graph(D):
    """Both recurrent paths (vector kernels at D=32, matrix-core kernels at D=64): the backward keeps its
    scratch inside its own outputs, so a replay needs nothing but the recorded kernels."""
    from gla_jax_amd import _lib
    lib = _lib.load()
    B, T, H = 2, 150, 3
    dtype, dt = torch.bfloat16, _lib.GLA_BF16
    (h0n, gn, vn, kn, qn), (h0, g, v, k, q) = gpu_inputs(B, T, H, D, 3.0, seed=78, dtype=dtype)
    dhTn, doutn = cotangents(h0n, vn, 10, dtype)
    dhT, dout = to_dev(dhTn, dtype), to_dev(doutn, dtype)
    outs = lambda: [torch.empty_like(h0), torch.empty_like(v), torch.empty_like(h0), torch.empty_like(g),
                    torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)]
    p = lambda t: t.data_ptr()

    def step(stream, o):
        hT, out, dh0, dg, dv, dk, dq = o
        _lib.check("gla_recurrent_fwd", lib.gla_recurrent_fwd(stream, B, T, H, D, D, dt, dt, dt, 0, p(h0), p(g), p(v),
                                                              p(k), p(q), p(hT), p(out)))
        _lib.check("gla_recurrent_bwd", lib.gla_recurrent_bwd(stream, B, T, H, D, D, dt, dt, dt, 0, p(h0), p(g), p(v),
                                                              p(k), p(q), p(hT), p(dhT), p(dout), p(dh0), p(dg),
                                                              p(dv), p(dk), p(dq)))

    eager = outs()
    step(torch.cuda.current_stream().cuda_stream, eager)
    torch.cuda.synchronize()
    replayed = outs()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream().cuda_stream, replayed)
    for it in range(3):
        for t in replayed:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("hidden_final", "out", "dh0", "dg", "dv", "dk", "dq"), eager, replayed):
            assert torch.equal(a, b), f"replay {it}: {name} differs from the eager result"


@pytest.mark.parametrize("B,T,H,D", [(2, 150, 2, 256), (1, 1024, 2, 64), (1, 1024, 1, 256)])
def test_recurrent_step_with_a_workspace_replays_from_a_graph(B, T, H, D):
    """gla_recurrent_fwd_ws / gla_recurrent_bwd_ws: head dimension 256 (two passes of the D=128 matrix-core kernels,
    their partial results in the caller's workspace), few long sequences (segments side by side: a dozen kernels
    per call, the states between them in the workspace), and both at once."""
    from gla_jax_amd import _lib
    lib = _lib.load()
    dtype, dt = torch.bfloat16, _lib.GLA_BF16
    (h0n, gn, vn, kn, qn), (h0, g, v, k, q) = gpu_inputs(B, T, H, D, 3.0, seed=79, dtype=dtype)
    dhTn, doutn = cotangents(h0n, vn, 11, dtype)
    dhT, dout = to_dev(dhTn, dtype), to_dev(doutn, dtype)
    u8 = lambda n: torch.empty(n, dtype=torch.uint8, device="cuda")
    ws_f = u8(lib.gla_recurrent_fwd_workspace_bytes(B, T, H, D, D, dt))
    ws_b = u8(lib.gla_recurrent_bwd_workspace_bytes(B, T, H, D, D, dt))
    assert ws_f.numel() > 0 and ws_b.numel() > 0
    outs = lambda: [torch.empty_like(h0), torch.empty_like(v), torch.empty_like(h0), torch.empty_like(g),
                    torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)]
    p = lambda t: t.data_ptr()

    def step(stream, o):
        hT, out, dh0, dg, dv, dk, dq = o
        _lib.check("gla_recurrent_fwd_ws", lib.gla_recurrent_fwd_ws(stream, B, T, H, D, D, dt, dt, dt, 0, p(h0), p(g),
                                                                    p(v), p(k), p(q), p(hT), p(out), p(ws_f),
                                                                    ws_f.numel()))
        _lib.check("gla_recurrent_bwd_ws", lib.gla_recurrent_bwd_ws(stream, B, T, H, D, D, dt, dt, dt, 0, p(h0), p(g),
                                                                    p(v), p(k), p(q), p(hT), p(dhT), p(dout), p(dh0),
                                                                    p(dg), p(dv), p(dk), p(dq), p(ws_b), ws_b.numel()))

    eager = outs()
    step(torch.cuda.current_stream().cuda_stream, eager)
    torch.cuda.synchronize()
    replayed = outs()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream().cuda_stream, replayed)
    for it in range(3):
        for t in replayed:
            t.fill_(float("nan"))
        ws_f.fill_(255)                                       # the workspace holds nothing a replay relies on
        ws_b.fill_(255)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("hidden_final", "out", "dh0", "dg", "dv", "dk", "dq"), eager, replayed):
            assert torch.equal(a, b), f"replay {it}: {name} differs from the eager result"
