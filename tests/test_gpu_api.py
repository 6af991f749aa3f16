"""Dtype and differentiation rules of the public entry points that the parity files do not exercise:
hidden_init in a dtype of its own (it enters the fp32 state uncast and hidden_final comes back in that dtype,
gla.py:44-46, 89-97, 711-716, 727) and the refusal of second-order gradients (the reference defines
first-order custom_vjp rules only, gla.py:441, 655)."""
import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from tests.util import assert_plain, cotangents, err_over_rms, gpu_inputs, loss_of, to_dev, to_np

pytestmark = pytest.mark.gpu


def _bind(name):
    from gla_jax_amd import chunk_gla, recurrent_gla, recurrent_gla_naive
    return {"chunk_gla": lambda *a: chunk_gla(*a, 64), "recurrent_gla": lambda *a: recurrent_gla(*a),
            "recurrent_gla_naive": lambda *a: recurrent_gla_naive(*a, False)}[name]


@pytest.mark.parametrize("name", ["recurrent_gla", "recurrent_gla_naive"])
@pytest.mark.parametrize("D", [64, 32, 256])
def test_fp32_state_beside_bf16_arrays_is_not_rounded(name, D):
    """A float32 hidden_init whose values bf16 does NOT hold, beside bf16 value/key/query: the recurrent paths
    load it into their fp32 state as it is and store hidden_final in float32 (gla.py:44-46, 89-97), so the
    final state and the gradient of the initial one match the fp64 oracle to float32 accuracy (1e-4 RMS), far
    below the 2^-9 a cast of the state to bf16 would leave.  D=64 runs on the matrix-core kernels, D=32 on the
    vector kernels, D=256 as two passes of the 128-feature matrix-core kernels with the states cut into blocks."""
    fn = _bind(name)
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(2, 200, 2, D, 4.0, seed=21, dtype=dtype)
    rng = np.random.default_rng(99)
    h0 = rng.standard_normal(h0.shape).astype(np.float32)          # not representable in bf16
    dhT = rng.standard_normal(h0.shape).astype(np.float32)
    _, dout = cotangents(h0, v, 21, dtype)
    assert np.abs(O.bf16_round(h0) - h0).max() > 1e-3
    args = [to_dev(h0, torch.float32)] + [t.clone() for t in dev[1:]]
    args = [t.requires_grad_(True) for t in args]
    hT, out = fn(*args)
    assert hT.dtype == torch.float32
    grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), args)
    assert grads[0].dtype == torch.float32
    exact = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)
    assert_plain("hidden_final", to_np(hT), exact[5], 1e-4)
    assert_plain("dhidden_init", to_np(grads[0]), exact[0], 1e-4)
    # and the same call with the state cast to bf16 first is measurably worse: the test would see a cast
    hT16, _ = fn(args[0].detach().to(dtype), *[t.detach() for t in args[1:]])
    assert err_over_rms(to_np(hT16), exact[5]) > 1e-3


@pytest.mark.parametrize("D", [64, 256])
def test_chunk_fp32_state_beside_bf16_arrays_enters_the_scan_unrounded(D):
    """chunk_gla hands hidden_init to the chunk scan uncast (gla.py:711-716): with keys of zero the final state
    is exactly hidden_init times the total decay, and a float32 hidden_init that bf16 does not hold must come
    back to float32 accuracy.  Only the copy used as the first chunk's incoming state is rounded (gla.py:720).
    Head dimension 256 cuts the states into four blocks on the way in and puts them together on the way out."""
    from gla_jax_amd import chunk_gla
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(2, 256, 2, D, 4.0, seed=22, dtype=dtype)
    rng = np.random.default_rng(98)
    h0 = rng.standard_normal(h0.shape).astype(np.float32)
    dhT = rng.standard_normal(h0.shape).astype(np.float32)
    args = [to_dev(h0, torch.float32), dev[1], dev[2], torch.zeros_like(dev[3]), dev[4]]
    args = [t.clone().requires_grad_(True) for t in args]
    hT, out = chunk_gla(*args, 64)
    assert hT.dtype == torch.float32 and out.dtype == dtype
    decay = np.exp(g.astype(np.float64).sum(axis=1))                      # [B,H,DK]
    assert_plain("hidden_final", to_np(hT), h0 * decay[..., None], 1e-5)
    # d(hidden_init) = total decay * d(hidden_final) + (what `out` contributes: none with a zero cotangent)
    (dh0,) = torch.autograd.grad((hT * to_dev(dhT, torch.float32)).sum(), args[:1])
    assert dh0.dtype == torch.float32
    assert_plain("dhidden_init", to_np(dh0), dhT * decay[..., None], 1e-5)
    # general keys: the bf16 bound against the oracle, float32 state in and out
    args = [to_dev(h0, torch.float32)] + [t.clone() for t in dev[1:]]
    hT, out = chunk_gla(*args, 64)
    eh, eo = O.recurrent_gla_naive(h0, g, v, k, q)
    assert_plain("hidden_final", to_np(hT), eh, 2e-2)
    assert_plain("out", to_np(out), eo, 3e-2)


@pytest.mark.parametrize("name", ["chunk_gla", "recurrent_gla"])
def test_bf16_hidden_init_with_fp32_arrays(name):
    """The other way round: a bf16 hidden_init beside float32 arrays computes in float32 and hands
    hidden_final back in bf16."""
    fn = _bind(name)
    (h0, g, v, k, q), dev = gpu_inputs(1, 128, 2, 64, 3.0, seed=13, dtype=torch.float32)
    h16 = dev[0].to(torch.bfloat16)
    hT_s, out_s = fn(h16.float(), *dev[1:])
    hT_m, out_m = fn(h16, *dev[1:])
    assert hT_m.dtype == torch.bfloat16 and out_m.dtype == torch.float32
    assert torch.equal(hT_m, hT_s.to(torch.bfloat16)) and torch.equal(out_m, out_s)


@pytest.mark.parametrize("name", ["chunk_gla", "recurrent_gla", "recurrent_gla_naive"])
def test_second_order_gradients_raise(name):
    fn = _bind(name)
    (h0, g, v, k, q), dev = gpu_inputs(1, 64, 1, 64, 3.0, seed=14, dtype=torch.float32)
    args = [t.clone().requires_grad_(True) for t in dev]
    hT, out = fn(*args)
    first = torch.autograd.grad(hT.sum() + out.sum(), args, create_graph=True)
    assert all(t.requires_grad for t in first)
    with pytest.raises(NotImplementedError, match="second-order"):
        torch.autograd.grad(sum(t.sum() for t in first), args)


def test_chunk_forward_without_gradients_keeps_no_residual():
    """Under no_grad (or with no argument that requires a gradient) chunk_gla skips the chunk-state residual; the
    results are those of the differentiable call, bit for bit."""
    from gla_jax_amd import chunk_gla
    (h0, g, v, k, q), dev = gpu_inputs(2, 256, 2, 128, 3.0, seed=15, dtype=torch.bfloat16)
    hT_a, out_a = chunk_gla(*[t.clone().requires_grad_(True) for t in dev], 128)
    with torch.no_grad():
        hT_b, out_b = chunk_gla(*dev, 128)
    hT_c, out_c = chunk_gla(*dev, 128)
    assert not hT_b.requires_grad and not out_c.requires_grad
    assert torch.equal(hT_a, hT_b) and torch.equal(out_a, out_b)
    assert torch.equal(hT_a, hT_c) and torch.equal(out_a, out_c)


@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
def test_chunk_values_that_are_not_finite_reach_the_state(bad):
    """The per-chunk products travel from one kernel to the next as 16-bit mantissas with shared exponents; a
    product that is not finite must still arrive as such, so that a NaN or an overflow in the inputs shows in
    hidden_final instead of being swallowed on the way."""
    from gla_jax_amd import chunk_gla
    _, dev = gpu_inputs(1, 256, 1, 64, 4.0, seed=17, dtype=torch.bfloat16)
    dev[2][0, 130, 0, 5] = bad                      # one value of `value`, in the second chunk
    hT, out = chunk_gla(*dev, 128)
    assert not torch.isfinite(hT.float()[0, 0, :, 5]).any()          # that value feature of the final state
    assert torch.isfinite(hT.float()[0, 0, :, 40:]).all()            # value features of other product tiles are untouched
    assert not torch.isfinite(out.float()[0, 130, 0, 5])
