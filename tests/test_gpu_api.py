"""Dtype and differentiation rules of the public entry points that the parity files do not exercise:
hidden_init in a dtype of its own (hidden_final comes back in that dtype, gla.py:46, 727; the state enters the
chunk kernels in the value dtype, gla.py:720) and the refusal of second-order gradients (the reference defines
first-order custom_vjp rules only, gla.py:441, 655)."""
import pytest
import torch

from tests.util import cotangents, gpu_inputs, loss_of

pytestmark = pytest.mark.gpu


def _bind(name):
    from gla_jax_amd import chunk_gla, recurrent_gla, recurrent_gla_naive
    return {"chunk_gla": lambda *a: chunk_gla(*a, 64), "recurrent_gla": lambda *a: recurrent_gla(*a),
            "recurrent_gla_naive": lambda *a: recurrent_gla_naive(*a, False)}[name]


@pytest.mark.parametrize("name", ["chunk_gla", "recurrent_gla", "recurrent_gla_naive"])
def test_fp32_hidden_init_with_bf16_arrays(name):
    """hidden_init float32 (values that bf16 holds exactly) beside bf16 value/key/query: hidden_final and the
    gradient of hidden_init are float32 and equal, bit for bit, what the all-bf16 call returns; `out` and the
    other gradients do not change at all."""
    fn = _bind(name)
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(2, 128, 2, 64, 3.0, seed=12, dtype=dtype)
    dhT, dout = cotangents(h0, v, 12, dtype)
    same = [t.clone().requires_grad_(True) for t in dev]
    hT_s, out_s = fn(*same)
    g_s = torch.autograd.grad(loss_of(hT_s, out_s, dhT, dout), same)
    mixed = [dev[0].float()] + [t.clone() for t in dev[1:]]
    mixed = [t.requires_grad_(True) for t in mixed]
    hT_m, out_m = fn(*mixed)
    assert hT_s.dtype == dtype and hT_m.dtype == torch.float32
    assert out_m.dtype == out_s.dtype
    assert torch.equal(hT_m, hT_s.float()) and torch.equal(out_m, out_s)
    g_m = torch.autograd.grad(loss_of(hT_m, out_m, dhT, dout), mixed)
    assert g_m[0].dtype == torch.float32 and torch.equal(g_m[0], g_s[0].float())
    for a, b in zip(g_m[1:], g_s[1:]):
        assert a.dtype == b.dtype and torch.equal(a, b)


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
