"""The tolerance model of tests/util.py on the CPU: the emulated reference (the oracle's chunk_gla with the
reference's bf16 rounding points) is assembled per batch entry and head exactly as a direct call gives it, and
`assert_parity` bounds an error by max(north_star, 1.5 x the emulated reference's error)."""
import numpy as np
import pytest

from oracle import gla_oracle as O
from tests import util


def test_reference_emulation_matches_direct_calls():
    B, T, H, D, C = 2, 64, 3, 16, 32
    h0, g, v, k, q = O.make_inputs(B, T, H, D, 1.0, seed=2)
    dhT, dout = util.cotangents(h0, v, 1, __import__("torch").bfloat16)
    emu = util.reference_emulation(h0, g, v, k, q, C, dhT, dout, workers=2)
    for b in range(B):
        hf, out, res = O.chunk_gla_forward(h0[b], g[b], v[b], k[b], q[b], C, rnd=O.bf16_round)
        grads = O.chunk_gla_backward(g[b], v[b], k[b], q[b], res, dhT[b], dout[b], C, rnd=O.bf16_round)
        np.testing.assert_array_equal(emu["out"][b], out)
        np.testing.assert_array_equal(emu["hidden_final"][b], O.bf16_round(hf))
        for n, a in zip(util.GRAD_NAMES, grads):
            np.testing.assert_array_equal(emu[n][b], a if n == "dlog_fgate" else O.bf16_round(a))
    # and it is close to, but not equal to, the exact result
    exact = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)
    e = util.err_over_rms(emu["out"], exact[6])
    assert 1e-4 < e < 1e-1


def test_assert_parity_bounds():
    rng = np.random.default_rng(0)
    exact = rng.standard_normal(1000)
    rms = np.sqrt((exact ** 2).mean())
    off = np.zeros(1000)
    off[3] = 1.0
    util.assert_parity("x", exact + 0.019 * rms * off, exact, 2e-2)                  # inside the plain bound
    with pytest.raises(AssertionError):
        util.assert_parity("x", exact + 0.021 * rms * off, exact, 2e-2)              # outside it
    emu = exact + 0.03 * rms * off                                                   # reference error 3e-2
    util.assert_parity("x", exact + 0.044 * rms * off, exact, 2e-2, emu)             # <= 1.5 x 3e-2
    with pytest.raises(AssertionError):
        util.assert_parity("x", exact + 0.046 * rms * off, exact, 2e-2, emu)
    with pytest.raises(AssertionError):
        util.assert_parity("x", np.where(off > 0, np.nan, exact), exact, 2e-2)       # non-finite values
