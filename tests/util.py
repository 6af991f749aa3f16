"""Shared helpers of the parity tests.

Tolerance model.  north_star states: max|err| / RMS(expected) <= 2e-2 for bf16 inputs, <= 1e-4 for fp32.
  * fp32 inputs: exactly that (`assert_parity` with no emulation).
  * bf16 inputs: the plain bound holds where bf16 arithmetic can meet it and is asserted there.  Where it
    cannot (rounding the EXACT fp64 output of BASELINE configs[4] to bf16 already costs 2.24e-2 RMS, because
    |out| reaches 7 RMS), the yardstick is the reference itself: the oracle's restatement of chunk_gla with
    every rounding point of the reference switched on (rescaled q/k, stored scores, per-chunk products,
    chunk states, intra/inter and their sum: gla.py:463-477, 719, 816-822, 851, 991-992), run on the SAME
    inputs, its outputs stored in the input dtype.  A tensor passes when
        max|hip - exact| / RMS  <=  max(2e-2, K_REF * max|emulated reference - exact| / RMS),  K_REF = 1.5.
    For recurrent_gla the reference computes in fp32 and rounds only what it stores (gla.py:89, 140), so
    its emulation is the exact result rounded to bf16.
"""
import concurrent.futures
import os

import numpy as np
import torch

from oracle import gla_oracle as O

TOL = {torch.bfloat16: 2e-2, torch.float32: 1e-4}   # max-abs error / RMS of the oracle (north_star)
K_REF = 1.5                                          # allowance over the emulated reference's own error
GRAD_NAMES = ("dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery")


def to_dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to("cuda").to(dtype)


def to_np(t):
    return t.detach().to(torch.float32).cpu().numpy().astype(np.float64)


def err_over_rms(got, exp):
    exp = np.asarray(exp, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    rms = np.sqrt((exp ** 2).mean())
    return float(np.abs(got - exp).max() / max(rms, 1e-30))


def assert_parity(name, got, exact, tol, emu=None, k_ref=K_REF, log=None):
    """max|got - exact| / RMS(exact) <= max(tol, k_ref * max|emu - exact| / RMS(exact)).

    `emu` is the emulated reference result on the same inputs (None: the plain north_star bound).
    Returns (hip error, reference error or None), both over RMS; `log`, a dict, receives them by name."""
    got = np.asarray(got, dtype=np.float64)
    exact = np.asarray(exact, dtype=np.float64)
    assert got.shape == exact.shape, f"{name}: shape {got.shape} != {exact.shape}"
    assert np.isfinite(got).all(), f"{name}: non-finite values"
    rms = max(float(np.sqrt((exact ** 2).mean())), 1e-30)
    e_hip = float(np.abs(got - exact).max() / rms)
    e_ref = None
    bound = tol
    if emu is not None:
        emu = np.asarray(emu, dtype=np.float64)
        assert emu.shape == exact.shape
        e_ref = float(np.abs(emu - exact).max() / rms)
        bound = max(tol, k_ref * e_ref)
    if log is not None:
        log[name] = (e_hip, e_ref)
    ref_txt = "" if e_ref is None else f", emulated reference {e_ref:.3e}"
    assert e_hip <= bound, (f"{name}: max|err|/rms = {e_hip:.3e} > bound {bound:.3e} "
                            f"(north_star {tol:.1e}{ref_txt}, rms {rms:.3e})")
    return e_hip, e_ref


def assert_plain(name, got, exact, tol, log=None):
    """The north_star bound itself: max|got - exact| <= tol * RMS(exact)."""
    return assert_parity(name, got, exact, tol, None, log=log)


def _emulate_one(args):
    h0, g, v, k, q, chunk, dhT, dout = args
    hf, out, res = O.chunk_gla_forward(h0, g, v, k, q, chunk, rnd=O.bf16_round)
    r = {"hidden_final": O.bf16_round(hf), "out": out}
    if dhT is not None:
        grads = O.chunk_gla_backward(g, v, k, q, res, dhT, dout, chunk, rnd=O.bf16_round)
        for n, a in zip(GRAD_NAMES, grads):
            # gradients come back in the dtype of their primal (gla.py:1216-1220, 753): bf16, the gates' fp32
            r[n] = a if n == "dlog_fgate" else O.bf16_round(a)
    return r


def reference_emulation(h0, g, v, k, q, chunk, dhT=None, dout=None, workers=None):
    """What the reference's chunk_gla would return on bf16 inputs: the oracle's restatement with the
    reference's own bf16 rounding points (see the module docstring), per batch element and head.  Arrays carry
    one leading batch axis.  Returns a dict name -> float array (`out`, `hidden_final` and, with cotangents,
    the five gradients)."""
    B, T, H, D = g.shape
    jobs = []
    for b in range(B):
        for h in range(H):
            s = slice(h, h + 1)
            jobs.append((h0[b, s], g[b, :, s], v[b, :, s], k[b, :, s], q[b, :, s], chunk,
                         None if dhT is None else dhT[b, s], None if dout is None else dout[b, :, s]))
    workers = workers or min(16, len(jobs), os.cpu_count() or 1)
    if workers > 1:
        with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as ex:
            parts = list(ex.map(_emulate_one, jobs))
    else:
        parts = [_emulate_one(j) for j in jobs]
    out = {}
    for name in parts[0]:
        per_b = []
        for b in range(B):
            hs = [parts[b * H + h][name] for h in range(H)]
            axis = 0 if name in ("hidden_final", "dhidden_init") else 1
            per_b.append(np.concatenate(hs, axis=axis))
        out[name] = np.stack(per_b)
    return out


def stored_emulation(exact):
    """The emulated result of a reference path that computes in fp32 and rounds only what it stores
    (recurrent_gla, gla.py:89, 140, 265-268): the exact values rounded to bf16."""
    return O.bf16_round(np.asarray(exact, dtype=np.float32)).astype(np.float64)


def check_chunk_outputs(dtype, arrs, chunk, hT, out, grads=None, dhT=None, dout=None, exact=None, log=None,
                        plain=()):
    """Forward (and gradients when given) of a chunk_gla call against the exact oracle, under the tolerance
    model of this module.  `arrs` = (h0, g, v, k, q) numpy with a leading batch axis; `exact` may carry the
    oracle's result (dh0, dg, dv, dk, dq, hidden_final, out) when the caller computed it already.  Names in
    `plain` are held to the plain north_star bound even for bf16."""
    h0, g, v, k, q = arrs
    tol = TOL[dtype]
    if exact is None:
        if grads is None:
            eh, eo = O.recurrent_gla_naive(h0, g, v, k, q)
            exact = (None,) * 5 + (eh, eo)
        else:
            exact = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)
    emu = {}
    if dtype == torch.bfloat16:
        emu = reference_emulation(h0, g, v, k, q, chunk, dhT if grads is not None else None,
                                  dout if grads is not None else None)
    log = {} if log is None else log
    pick = lambda n: None if n in plain else emu.get(n)
    assert_parity("out", to_np(out), exact[6], tol, pick("out"), log=log)
    assert_parity("hidden_final", to_np(hT), exact[5], tol, pick("hidden_final"), log=log)
    if grads is not None:
        for n, got, e in zip(GRAD_NAMES, grads, exact[:5]):
            assert_parity(n, to_np(got), e, tol, pick(n), log=log)
    return log


def check_recurrent_outputs(dtype, exact, hT, out, grads=None, out_fp32=False, log=None):
    """The same for recurrent_gla / recurrent_gla_naive: the reference computes in fp32 (gla.py:89), so its
    emulated error is the rounding of what it stores in bf16."""
    tol = TOL[dtype]
    bf = dtype == torch.bfloat16
    log = {} if log is None else log
    st = (lambda e: stored_emulation(e)) if bf else (lambda e: None)
    assert_parity("out", to_np(out), exact[6], tol, None if out_fp32 else st(exact[6]), log=log)
    assert_parity("hidden_final", to_np(hT), exact[5], tol, st(exact[5]), log=log)
    if grads is not None:
        for n, got, e in zip(GRAD_NAMES, grads, exact[:5]):
            assert_parity(n, to_np(got), e, tol, None if n == "dlog_fgate" else st(e), log=log)
    return log


def fmt_log(log):
    return {n: (f"{a:.2e}" if b is None else f"{a:.2e} (ref {b:.2e})") for n, (a, b) in log.items()}


def gpu_inputs(B, T, H, D, shift, seed, dtype, batch_dims=True):
    """Oracle inputs (numpy, bf16-representable when dtype is bf16) and their device copies."""
    arrs = O.make_inputs(B, T, H, D, shift, seed=seed, low_precision=(dtype == torch.bfloat16),
                         batch_dims=batch_dims)
    h0, g, v, k, q = arrs
    dev = [to_dev(h0, dtype), to_dev(g, torch.float32), to_dev(v, dtype), to_dev(k, dtype), to_dev(q, dtype)]
    return arrs, dev


def cotangents(h0, v, seed, dtype):
    rng = np.random.default_rng(7000 + seed)
    dhT = rng.standard_normal(h0.shape, dtype=np.float32)
    dout = rng.standard_normal(v.shape, dtype=np.float32)
    if dtype == torch.bfloat16:
        dhT, dout = O.bf16_round(dhT), O.bf16_round(dout)
    return dhT, dout


def loss_of(hT, out, dhT, dout):
    return (hT.float() * to_dev(dhT, torch.float32)).sum() + (out.float() * to_dev(dout, torch.float32)).sum()
