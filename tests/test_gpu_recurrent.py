"""GPU parity of recurrent_gla / recurrent_gla_naive (forward, all five gradients) through the C ABI
against the oracle.  Tolerance (north_star): max|err| / RMS(oracle) <= 2e-2 for bf16 inputs,
<= 1e-4 for fp32."""
import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from oracle import naive_c
from tests.util import (TOL, assert_plain, check_recurrent_outputs, cotangents, fmt_log, gpu_inputs, to_dev, to_np)

pytestmark = pytest.mark.gpu


def run_fwd_bwd(fn, dev, dhT, dout, out_dtype, **kw):
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = fn(*dev, **kw)
    loss = (hT.float() * dhT.float()).sum() + (out.float() * dout.float()).sum()
    grads = torch.autograd.grad(loss, dev)
    return hT, out, grads


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,T,H,D", [(2, 67, 3, 64), (1, 32, 2, 16), (1, 40, 1, 128), (2, 24, 2, 32), (3, 1, 5, 64),
                                     (1, 17, 1, 64), (2, 45, 2, 256), (2, 37, 3, 8), (1, 20, 2, 4)])
@pytest.mark.parametrize("reverse", [False, True])
def test_recurrent_gla_matches_oracle(dtype, B, T, H, D, reverse):
    from gla_jax_amd import recurrent_gla
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, 3.0, seed=B * 100 + T, dtype=dtype)
    dhT, dout = cotangents(h0, v, 1, dtype)
    hT, out, grads = run_fwd_bwd(recurrent_gla, dev, to_dev(dhT, dtype), to_dev(dout, dtype), dtype,
                                 reverse=reverse)
    assert out.dtype == dtype and hT.dtype == dtype
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads)))


@pytest.mark.parametrize("D", [32, 64])
@pytest.mark.parametrize("reverse", [False, True])
def test_recurrent_gate_gradient_of_a_short_sequence(D, reverse):
    """d(log_fgate) ends in sum_v dhidden_final * hidden_final (gla.py:263), the same for every step.  On a
    short sequence with a large final state it dominates; it must come from the fp32 state of the backward's
    first sweep (with the stored bf16 hidden_final it is off by 2^-9 of |dh.h|, 1.6e-2 of the gradient's norm
    on this input).  Both the vector kernels (D=32) and the matrix-core kernels (D=64)."""
    from gla_jax_amd import recurrent_gla
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(1, 13, 1, D, -2.0, seed=603, dtype=dtype)
    dhT, dout = cotangents(h0, v, 103, dtype)
    _, _, grads = run_fwd_bwd(recurrent_gla, dev, to_dev(dhT, dtype), to_dev(dout, dtype), dtype, reverse=reverse)
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
    err = to_np(grads[1]) - exp[1]
    assert np.linalg.norm(err) <= 1e-3 * np.linalg.norm(exp[1])


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("T", [64, 200, 333])
def test_recurrent_matrix_core_path_over_gate_regimes(T, reverse, D):
    """bf16 at D=64 and D=128 runs 64 steps per iteration on the matrix cores: sequences that are not a
    multiple of 64 (padded steps), mild gates (one anchor per 16 steps) and hard ones (resets, the dyadic
    levels) in the same sequence, both directions, forward and all gradients."""
    from gla_jax_amd import recurrent_gla
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(2, T, 2, D, 1.0, seed=T + 7, dtype=dtype)
    g = g.copy()
    g[:, 5::37] = -200.0                       # hard resets at scattered positions
    g[:, T // 2:T // 2 + 4, :, ::2] = -60.0    # a hard stretch on every other feature
    dev[1] = to_dev(g, torch.float32)
    dhT, dout = cotangents(h0, v, 2, dtype)
    hT, out, grads = run_fwd_bwd(recurrent_gla, dev, to_dev(dhT, dtype), to_dev(dout, dtype), dtype,
                                 reverse=reverse)
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads)))


@pytest.mark.parametrize("T,D", [(50, 64), (300, 64), (150, 128), (40, 32), (90, 256)])
def test_recurrent_gla_naive_returns_fp32_out(T, D):
    """The naive flavour (gla.py:26-47): fp32 `out` (promotion at gla.py:37) to fp32 accuracy although the inputs
    are bf16, and an fp32 cotangent for it in the backward.  D=64 and 128 run on the matrix-core kernels (the
    fp32 accumulators stored unrounded; sequences longer than one block of steps), D=32 on the vector kernels."""
    from gla_jax_amd import recurrent_gla_naive
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(2, T, 2, D, 5.0, seed=9, dtype=dtype)
    dhT, dout = cotangents(h0, v, 2, torch.float32)
    dhT = O.bf16_round(dhT)
    hT, out, grads = run_fwd_bwd(recurrent_gla_naive, dev, to_dev(dhT, dtype), to_dev(dout, torch.float32),
                                 torch.float32, reverse=False)
    assert out.dtype == torch.float32 and hT.dtype == dtype            # gla.py:37, 46
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)
    assert_plain("out", to_np(out), exp[6], 1e-4)                      # fp32 state and output
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads, out_fp32=True)))


def test_recurrent_gla_naive_reverse():
    """recurrent_gla_naive(reverse=True) (gla.py:45): the scan runs from the last step down, outputs stay in
    place; forward and all gradients."""
    from gla_jax_amd import recurrent_gla_naive
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(2, 77, 3, 64, 2.0, seed=19, dtype=dtype)
    dhT, dout = cotangents(h0, v, 4, torch.float32)
    dhT = O.bf16_round(dhT)
    hT, out, grads = run_fwd_bwd(recurrent_gla_naive, dev, to_dev(dhT, dtype), to_dev(dout, torch.float32),
                                 torch.float32, reverse=True)
    assert out.dtype == torch.float32 and hT.dtype == dtype
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=True)
    assert_plain("out", to_np(out), exp[6], 1e-4)
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads, out_fp32=True)))
    # the reversed scan is the forward scan of the flipped sequence (gla.py:421-438)
    fl = lambda t: t.flip(1).contiguous()
    hT2, out2 = recurrent_gla_naive(dev[0], fl(dev[1]), fl(dev[2]), fl(dev[3]), fl(dev[4]), False)
    assert torch.equal(hT2, hT) and torch.equal(fl(out2), out)


def test_recurrent_unbatched_and_vmap_agree():
    from gla_jax_amd import recurrent_gla
    (h0, g, v, k, q), dev = gpu_inputs(3, 33, 2, 64, 3.0, seed=4, dtype=torch.bfloat16)
    hT_b, out_b = recurrent_gla(*dev)
    hT_v, out_v = torch.func.vmap(recurrent_gla)(*dev)
    assert torch.equal(hT_b, hT_v) and torch.equal(out_b, out_v)
    for b in range(3):
        hT_1, out_1 = recurrent_gla(*[t[b] for t in dev])
        assert torch.equal(hT_1, hT_b[b]) and torch.equal(out_1, out_b[b])


def test_recurrent_full_benchmark_shape_against_c_oracle():
    """BASELINE configs[4]: B16,T2048,H16,D64 bf16, gates log_sigmoid(3+N(0,1)); forward and all
    gradients against the C restatement in fp64 on every (b,h) pair."""
    from gla_jax_amd import recurrent_gla
    dtype = torch.bfloat16
    B, T, H, D = 16, 2048, 16, 64
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, 3.0, seed=44, dtype=dtype)
    dhT, dout = cotangents(h0, v, 3, dtype)
    hT, out, grads = run_fwd_bwd(recurrent_gla, dev, to_dev(dhT, dtype), to_dev(dout, dtype), dtype)
    exp = naive_c.naive_bwd(h0, g, v, k, q, dhT, dout, dtype=np.float64, nthreads=16)
    print(fmt_log(check_recurrent_outputs(dtype, exp, hT, out, grads)))


def test_recurrent_rejects_bad_arguments():
    from gla_jax_amd import _lib, recurrent_gla
    (h0, g, v, k, q), dev = gpu_inputs(1, 8, 1, 48, 3.0, seed=5, dtype=torch.bfloat16)
    with pytest.raises(_lib.GlaError):
        recurrent_gla(*dev)                       # head dim 48 is not built
    with pytest.raises(AssertionError):
        recurrent_gla(dev[0], dev[1], dev[2][..., :32], dev[3], dev[4])
