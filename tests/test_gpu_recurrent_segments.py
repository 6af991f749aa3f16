"""recurrent_gla on few sequences: with a workspace the C entry points run every sequence as S segments side by
side (a pass from zero states, a scan over the segments, the real pass; the backward likewise for the states'
cotangents).  Checked against the oracle like every other recurrent_gla case, and against the same call without a
workspace (the sequences run whole): the two may differ by the order of fp32 sums only."""
import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from tests.util import check_recurrent_outputs, cotangents, fmt_log, gpu_inputs, to_dev, to_np

pytestmark = pytest.mark.gpu

# dtype, B, T, H, D, reverse, gate shift: shapes at which gla_recurrent_*_workspace_bytes ask for segments
CASES = [
    (torch.bfloat16, 1, 1024, 2, 64, False, 3.0),
    (torch.bfloat16, 1, 1024, 2, 64, True, 3.0),
    (torch.bfloat16, 2, 2048, 1, 128, False, 5.0),
    (torch.bfloat16, 1, 2048, 1, 128, True, 0.0),
    (torch.float32, 1, 1024, 2, 32, False, 3.0),
    (torch.float32, 1, 1024, 1, 64, True, 1.0),
    (torch.bfloat16, 1, 1024, 3, 16, False, 3.0),
    (torch.bfloat16, 2, 1024, 1, 256, False, 3.0),
    (torch.bfloat16, 1, 1024, 1, 256, True, 3.0),
    (torch.bfloat16, 1, 1200, 2, 64, False, 3.0),       # 8 segments of 150 steps: not a multiple of the kernels' blocks
    (torch.bfloat16, 1, 1280, 3, 64, True, 3.0),        # 10 segments of 128 steps
    (torch.bfloat16, 1, 256, 2, 128, False, 3.0),       # two segments (bf16 at head dimensions 64 and more only)
    (torch.bfloat16, 2, 256, 1, 128, True, 1.0),
    (torch.bfloat16, 1, 256, 1, 256, False, 3.0),
    (torch.bfloat16, 2, 256, 1, 64, True, 3.0),
    (torch.bfloat16, 1, 384, 2, 64, False, 1.0),        # three
    (torch.bfloat16, 1, 2048, 64, 128, False, 3.0),     # 4 segments of 512 steps, the lean passes in pieces of 256
    (torch.bfloat16, 2, 2048, 16, 256, True, 3.0),
]


def _sizes(B, T, H, D, dtype):
    from gla_jax_amd import _lib
    lib = _lib.load()
    dt = _lib.GLA_BF16 if dtype == torch.bfloat16 else _lib.GLA_F32
    return (lib.gla_recurrent_fwd_workspace_bytes(B, T, H, D, D, dt),
            lib.gla_recurrent_bwd_workspace_bytes(B, T, H, D, D, dt))


@pytest.mark.parametrize("dtype,B,T,H,D,reverse,shift", CASES)
def test_segmented_recurrent_gla_matches_oracle(dtype, B, T, H, D, reverse, shift):
    from gla_jax_amd import recurrent_gla
    assert min(_sizes(B, T, H, D, dtype)) > 0, "the case is meant to run in segments"
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, shift, seed=T + D, dtype=dtype)
    g = g.copy()
    g[:, 300::411] = -200.0                    # resets, one of them right behind a segment boundary or two
    g[:, 255] = -30.0
    dev[1] = to_dev(g, torch.float32)
    dhT, dout = cotangents(h0, v, 5, dtype)
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = recurrent_gla(*dev, reverse=reverse)
    loss = (hT.float() * to_dev(dhT, dtype).float()).sum() + (out.float() * to_dev(dout, dtype).float()).sum()
    grads = torch.autograd.grad(loss, dev)
    if B * H >= 32:         # many sequences: the C restatement on all host threads (fp64); it walks forward in time,
        from oracle import naive_c                     # and the reversed scan is that of the flipped sequence
        fl = (lambda a: np.ascontiguousarray(a[:, ::-1])) if reverse else (lambda a: a)
        dh0_, dg_, dv_, dk_, dq_, hT_, out_ = naive_c.naive_bwd(h0, fl(g), fl(v), fl(k), fl(q), dhT, fl(dout),
                                                                dtype=np.float64, nthreads=16)
        exp = (dh0_, fl(dg_), fl(dv_), fl(dk_), fl(dq_), hT_, fl(out_))
    else:
        exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads)))


@pytest.mark.parametrize("dtype,B,T,H,D,reverse", [(torch.bfloat16, 1, 1024, 2, 64, False),
                                                    (torch.bfloat16, 1, 1024, 1, 128, True),
                                                    (torch.bfloat16, 2, 4096, 8, 64, False),
                                                    (torch.float32, 1, 1024, 2, 32, False)])
def test_segments_agree_with_whole_sequences(dtype, B, T, H, D, reverse):
    """The same call through gla_recurrent_fwd / _bwd (no workspace: whole sequences) and through the _ws entry
    points (segments).  fp32 state hand-over, so the results differ by fp32 summation order: a rounding step of the
    stored type at most on a few elements, far below the parity bound."""
    from gla_jax_amd import _lib
    lib = _lib.load()
    dt = _lib.GLA_BF16 if dtype == torch.bfloat16 else _lib.GLA_F32
    (h0n, gn, vn, kn, qn), (h0, g, v, k, q) = gpu_inputs(B, T, H, D, 3.0, seed=91, dtype=dtype)
    dhTn, doutn = cotangents(h0n, vn, 12, dtype)
    dhT, dout = to_dev(dhTn, dtype), to_dev(doutn, dtype)
    p = lambda t: t.data_ptr()
    u8 = lambda n: torch.empty(n, dtype=torch.uint8, device="cuda")
    nf, nb = _sizes(B, T, H, D, dtype)
    assert nf > 0 and nb > 0
    ws_f, ws_b = u8(nf), u8(nb)
    outs = lambda: [torch.empty_like(h0), torch.empty_like(v), torch.empty_like(h0), torch.empty_like(g),
                    torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)]
    st = torch.cuda.current_stream().cuda_stream
    rv = int(reverse)
    whole, seg = outs(), outs()
    hT, out, dh0, dg, dv, dk, dq = whole
    _lib.check("gla_recurrent_fwd", lib.gla_recurrent_fwd(st, B, T, H, D, D, dt, dt, dt, rv, p(h0), p(g), p(v), p(k), p(q),
                                                          p(hT), p(out)))
    _lib.check("gla_recurrent_bwd", lib.gla_recurrent_bwd(st, B, T, H, D, D, dt, dt, dt, rv, p(h0), p(g), p(v), p(k), p(q),
                                                          p(hT), p(dhT), p(dout), p(dh0), p(dg), p(dv), p(dk), p(dq)))
    hT, out, dh0, dg, dv, dk, dq = seg
    _lib.check("gla_recurrent_fwd_ws", lib.gla_recurrent_fwd_ws(st, B, T, H, D, D, dt, dt, dt, rv, p(h0), p(g), p(v), p(k),
                                                                p(q), p(hT), p(out), p(ws_f), nf))
    _lib.check("gla_recurrent_bwd_ws", lib.gla_recurrent_bwd_ws(st, B, T, H, D, D, dt, dt, dt, rv, p(h0), p(g), p(v), p(k),
                                                                p(q), p(hT), p(dhT), p(dout), p(dh0), p(dg), p(dv), p(dk),
                                                                p(dq), p(ws_b), nb))
    # the same call again: the same bits (no result depends on the order in which workgroups or waves finish)
    again = outs()
    hT, out, dh0, dg, dv, dk, dq = again
    ws_f.fill_(1)
    ws_b.fill_(2)
    _lib.check("gla_recurrent_fwd_ws", lib.gla_recurrent_fwd_ws(st, B, T, H, D, D, dt, dt, dt, rv, p(h0), p(g), p(v), p(k),
                                                                p(q), p(hT), p(out), p(ws_f), nf))
    _lib.check("gla_recurrent_bwd_ws", lib.gla_recurrent_bwd_ws(st, B, T, H, D, D, dt, dt, dt, rv, p(h0), p(g), p(v), p(k),
                                                                p(q), p(hT), p(dhT), p(dout), p(dh0), p(dg), p(dv), p(dk),
                                                                p(dq), p(ws_b), nb))
    torch.cuda.synchronize()
    for name, a, b in zip(("hidden_final", "out", "dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery"), seg, again):
        assert torch.equal(a, b), f"{name} differs between two runs of the same call"
    for name, a, b in zip(("hidden_final", "out", "dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery"), whole, seg):
        a, b = to_np(a), to_np(b)
        rms = float(np.sqrt(np.mean(a ** 2)))
        worst = float(np.abs(a - b).max()) / rms
        frac = float(np.mean(a != b))
        print(f"{name}: max difference {worst:.2e} of an RMS, {100 * frac:.2f} % of the elements differ")
        # bf16 results: one rounding step of a value of 8 RMS is 3.1e-2 RMS, on few elements.  d(log_fgate) (fp32)
        # of bf16 data: the running sum over the later steps starts from sum_v d(state) * state at a segment's end
        # where the whole sequence carries the sum of its terms, two forms whose own errors are 1e-4 each (as
        # against the oracle).  fp32 data: summation order only.
        if dtype == torch.float32:
            assert worst <= 2e-5, name
        elif name == "dlog_fgate":
            assert worst <= 1e-3, name
        else:
            assert worst <= 4e-2 and frac <= 0.02, name


@pytest.mark.parametrize("B,T,H,D,reverse", [(1, 1024, 2, 64, False), (1, 2048, 1, 128, True), (1, 1024, 1, 256, False),
                                             (1, 1024, 2, 32, False)])
def test_segmented_recurrent_gla_naive_flavour(B, T, H, D, reverse):
    """bf16 data with an fp32 `out` and an fp32 cotangent for it (gla.py:37): the forward runs in segments like
    recurrent_gla's; in the backward the pass for the states' cotangents takes dout as two bf16 arrays, head and
    remainder, whose states add (D = 32 has no such pass and runs its backward on whole sequences)."""
    from gla_jax_amd import recurrent_gla_naive
    from tests.util import assert_plain
    dtype = torch.bfloat16
    assert min(_sizes(B, T, H, D, dtype)) > 0
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, 3.0, seed=T + D + 1, dtype=dtype)
    dhT, dout = cotangents(h0, v, 6, torch.float32)
    dhT = O.bf16_round(dhT)
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = recurrent_gla_naive(*dev, reverse=reverse)
    assert out.dtype == torch.float32 and hT.dtype == dtype
    loss = (hT.float() * to_dev(dhT, dtype).float()).sum() + (out * to_dev(dout, torch.float32)).sum()
    grads = torch.autograd.grad(loss, dev)
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
    assert_plain("out", to_np(out), exp[6], 1e-4)
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads, out_fp32=True)))


def test_random_shapes_in_segments_agree_with_whole_sequences():
    """A fixed-seed draw of shapes that run in segments (both element types, fp32 states beside bf16 data, the
    recurrent_gla_naive flavour, every head dimension, lengths that are odd multiples of 256, both directions,
    scattered resets), each through the entry points with a workspace and through those without.  The case is
    printed before it runs."""
    from gla_jax_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(20240611)
    p = lambda t: t.data_ptr()
    done = 0
    for it in range(40):
        dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float32
        dt = _lib.GLA_BF16 if dtype == torch.bfloat16 else _lib.GLA_F32
        hd = torch.float32 if rng.random() < 0.3 else dtype
        hdt = _lib.GLA_BF16 if hd == torch.bfloat16 else _lib.GLA_F32
        D = int(rng.choice([16, 32, 64, 64, 128, 128, 256]))
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        T = int(rng.choice([512, 1024, 1280, 1536, 2048, 2560, 3072]))
        if D == 256 or dtype == torch.float32:
            T = min(T, 1536)                       # the whole-sequence vector kernels are slow
        rev = int(rng.integers(0, 2))
        naive = dtype == torch.bfloat16 and rng.random() < 0.25
        odt, otype = (_lib.GLA_F32, torch.float32) if naive else (dt, dtype)
        shift = float(rng.choice([0.0, 1.0, 3.0, 5.0]))
        nf, nb = _sizes(B, T, H, D, dtype)
        print(f"case {it}: {dtype} states {hd} fp32-out {naive} B{B} T{T} H{H} D{D} reverse {rev} shift {shift} "
              f"workspace {nf} {nb}", flush=True)
        if nf == 0:
            continue
        gen = torch.Generator(device="cuda").manual_seed(1000 + it)
        rand = lambda *s, t=dtype: torch.randn(*s, device="cuda", generator=gen).to(t)
        g = torch.nn.functional.logsigmoid(shift + rand(B, T, H, D, t=torch.float32))
        if rng.random() < 0.5:
            g[:, torch.as_tensor(rng.integers(0, T, size=5), device="cuda")] = float(rng.choice([-200.0, -30.0]))
        h0, dhT = rand(B, H, D, D, t=hd), rand(B, H, D, D, t=hd)
        v, k, q, dout = rand(B, T, H, D), rand(B, T, H, D), rand(B, T, H, D), rand(B, T, H, D, t=otype)
        outs = lambda: [torch.empty_like(h0), torch.empty_like(dout), torch.empty_like(h0), torch.empty_like(g),
                        torch.empty_like(v), torch.empty_like(k), torch.empty_like(q)]
        ws_f = torch.full((nf,), 77, dtype=torch.uint8, device="cuda")
        ws_b = torch.full((nb,), 77, dtype=torch.uint8, device="cuda")
        st = torch.cuda.current_stream().cuda_stream
        whole, seg = outs(), outs()
        hT, out, dh0, dg, dv, dk, dq = whole
        _lib.check("gla_recurrent_fwd", lib.gla_recurrent_fwd(st, B, T, H, D, D, dt, hdt, odt, rev, p(h0), p(g), p(v), p(k),
                                                              p(q), p(hT), p(out)))
        _lib.check("gla_recurrent_bwd", lib.gla_recurrent_bwd(st, B, T, H, D, D, dt, hdt, odt, rev, p(h0), p(g), p(v), p(k),
                                                              p(q), p(hT), p(dhT), p(dout), p(dh0), p(dg), p(dv), p(dk),
                                                              p(dq)))
        hT, out, dh0, dg, dv, dk, dq = seg
        _lib.check("gla_recurrent_fwd_ws", lib.gla_recurrent_fwd_ws(st, B, T, H, D, D, dt, hdt, odt, rev, p(h0), p(g), p(v),
                                                                    p(k), p(q), p(hT), p(out), p(ws_f), nf))
        _lib.check("gla_recurrent_bwd_ws", lib.gla_recurrent_bwd_ws(st, B, T, H, D, D, dt, hdt, odt, rev, p(h0), p(g), p(v),
                                                                    p(k), p(q), p(hT), p(dhT), p(dout), p(dh0), p(dg), p(dv),
                                                                    p(dk), p(dq), p(ws_b), nb))
        torch.cuda.synchronize()
        for name, a, b in zip(("hidden_final", "out", "dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery"), whole, seg):
            x, y = a.double(), b.double()
            worst = float((x - y).abs().max()) / float(x.pow(2).mean().sqrt())
            # a float result: the order of fp32 sums (d(log_fgate) of bf16 data: two forms of the carried sum, 1e-4
            # each); a bf16 result: a rounding step of a value of up to 16 RMS
            bound = 2e-3 if a.dtype == torch.float32 else 6.3e-2
            assert worst <= bound, f"case {it} {name}: {worst:.3e}"
        done += 1
    assert done >= 25
