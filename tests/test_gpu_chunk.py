"""GPU parity of chunk_gla (forward and all five gradients) through the C ABI against the oracle's
naive recurrence.  Tolerance (north_star): max|err| / RMS(oracle) <= 2e-2 for bf16, <= 1e-4 for fp32; for
bf16 the bound widens to 1.5 x the error of the emulated reference on the same inputs where that is
larger (tests/util.py)."""
import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from oracle import naive_c
from tests.util import (GRAD_NAMES, TOL, assert_parity, assert_plain, check_chunk_outputs, cotangents, err_over_rms,
                        fmt_log, gpu_inputs, loss_of, reference_emulation, to_dev, to_np)

pytestmark = pytest.mark.gpu

# The kernels run with the largest tile built (128, 64, 32 tokens; fp32: 64, 32 at D=64 and 32 at D=128) that
# divides T, whatever chunk_size asks for: T picks the tile here.
CASES = [
    # dtype, B, T, H, D, chunk, gate shift
    (torch.bfloat16, 2, 256, 2, 128, 128, 5.0),
    (torch.bfloat16, 1, 448, 3, 64, 64, 5.0),       # 64-token tiles
    (torch.bfloat16, 2, 192, 1, 128, 64, 1.0),      # 64-token tiles
    (torch.bfloat16, 1, 256, 2, 64, 128, 0.0),
    (torch.bfloat16, 1, 96, 2, 64, 32, 3.0),        # 32-token tiles
    (torch.bfloat16, 1, 512, 1, 128, 256, 5.0),     # chunk above the largest tile: same result
    (torch.bfloat16, 1, 256, 2, 64, 32, 3.0),       # chunk below the tile that is used: same result
    (torch.float32, 1, 512, 2, 64, 64, 5.0),        # BASELINE configs[0]
    (torch.float32, 2, 96, 1, 64, 32, 0.0),         # fp32, 32-token tiles
    (torch.bfloat16, 1, 160, 2, 128, 32, 2.0),      # the smallest tile at D=128
    (torch.float32, 1, 256, 2, 128, 128, 4.0),      # fp32 at D=128 runs on the 32-token tile
    (torch.bfloat16, 3, 128, 5, 128, 128, 3.0),     # a single chunk per sequence, odd batch and head counts
    (torch.bfloat16, 1, 64, 1, 64, 64, 3.0),
    (torch.bfloat16, 2, 160, 2, 256, 32, 4.0),      # head dimension 256: four problems of head dimension 128
    (torch.bfloat16, 1, 256, 1, 256, 128, 0.0),     # the same under strong decay
    (torch.bfloat16, 2, 384, 3, 256, 128, 2.0),
    (torch.float32, 2, 96, 2, 256, 32, 3.0),        # ... and in fp32
    (torch.bfloat16, 2, 256, 3, 32, 128, 3.0),      # head dimension 32: one k-step per feature contraction
    (torch.bfloat16, 1, 192, 2, 32, 64, 0.0),       # ... 64-token tiles, strong decay
    (torch.bfloat16, 1, 96, 1, 32, 32, 5.0),        # ... 32-token tiles
    (torch.float32, 2, 192, 2, 32, 64, 2.0),        # ... fp32
    (torch.float32, 1, 96, 2, 32, 32, 0.0),
    (torch.bfloat16, 2, 256, 3, 16, 128, 3.0),      # head dimension 16: the 32-feature kernels, rows padded by zeros
    (torch.bfloat16, 1, 192, 5, 16, 64, 0.0),
    (torch.bfloat16, 3, 32, 1, 16, 32, 5.0),
    (torch.float32, 2, 192, 2, 16, 64, 1.0),
    (torch.float32, 1, 96, 3, 16, 32, 4.0),
]


@pytest.mark.parametrize("dtype,B,T,H,D,chunk,shift", CASES)
def test_chunk_forward_matches_oracle(dtype, B, T, H, D, chunk, shift):
    from gla_jax_amd import chunk_gla
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, shift, seed=T + D + chunk, dtype=dtype)
    hT, out = chunk_gla(*dev, chunk)
    assert out.dtype == dtype and hT.dtype == dtype and out.shape == dev[2].shape
    print(fmt_log(check_chunk_outputs(dtype, (h0, g, v, k, q), chunk, hT, out)))


@pytest.mark.parametrize("dtype,B,T,H,D,chunk,shift", CASES)
def test_chunk_backward_matches_oracle(dtype, B, T, H, D, chunk, shift):
    from gla_jax_amd import chunk_gla
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, shift, seed=T + D + chunk + 1, dtype=dtype)
    dhT, dout = cotangents(h0, v, 5, dtype)
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = chunk_gla(*dev, chunk)
    grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), dev)
    print(fmt_log(check_chunk_outputs(dtype, (h0, g, v, k, q), chunk, hT, out, grads, dhT, dout)))


def test_chunk_strong_decay_and_hard_resets():
    """Gates far below log_sigmoid(N(0,1)): every rescaling factor must stay <= 1 (no overflow), also
    when a gate closes completely inside a 16-token sub-block."""
    from gla_jax_amd import chunk_gla
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(1, 256, 2, 128, -2.0, seed=77, dtype=dtype)
    g = g.copy()
    g[:, 5::37] = -200.0           # hard resets at scattered positions
    g[:, 100:104] = -90.0
    dev[1] = to_dev(g, torch.float32)
    hT, out = chunk_gla(*dev, 128)
    print(fmt_log(check_chunk_outputs(dtype, (h0, g, v, k, q), 128, hT, out)))


def test_chunk_fp32_closed_gates_do_not_cost_precision():
    """fp32 inputs, strong decay and gates that close completely: the decay of a key towards the end of its
    chunk must come from the later gates alone, not from a difference of two prefix sums that both carry
    the closed gate (-200 leaves 3e-5 of absolute error in every later prefix, 1e-4 x RMS in the state)."""
    from gla_jax_amd import chunk_gla
    dtype = torch.float32
    (h0, g, v, k, q), dev = gpu_inputs(3, 64, 4, 64, -2.0, seed=538, dtype=dtype)
    g = g.copy()
    g[:, [9, 15, 50]] = -200.0
    dev[1] = to_dev(g, torch.float32)
    eh, eo = O.recurrent_gla_naive(h0, g, v, k, q)
    for chunk in (32, 64):
        hT, out = chunk_gla(*dev, chunk)
        assert_plain("out", to_np(out), eo, 2e-5)
        assert_plain("hidden_final", to_np(hT), eh, 2e-5)


@pytest.mark.parametrize("regime", ["mild", "mixed", "resets"])
def test_chunk_backward_over_gate_regimes(regime):
    """Sub-blocks whose gates are mild take the single-anchor path, the others the dyadic recursion; a chunk
    may hold both kinds.  All five gradients against the oracle in every regime."""
    from gla_jax_amd import chunk_gla
    dtype = torch.bfloat16
    shift = {"mild": 4.0, "mixed": -1.5, "resets": -1.5}[regime]
    (h0, g, v, k, q), dev = gpu_inputs(1, 256, 2, 128, shift, seed=91, dtype=dtype)
    g = g.copy()
    if regime == "resets":
        g[:, 5::37] = -200.0
        g[:, 100:104, :, ::2] = -90.0          # only every other feature: the sub-block still takes the recursion
    dev[1] = to_dev(g, torch.float32)
    dhT, dout = cotangents(h0, v, 6, dtype)
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = chunk_gla(*dev, 128)
    grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), dev)
    print(fmt_log(check_chunk_outputs(dtype, (h0, g, v, k, q), 128, hT, out, grads, dhT, dout)))


def test_chunk_size_and_concatenation_invariance():
    from gla_jax_amd import chunk_gla
    dtype = torch.float32
    (h0, g, v, k, q), dev = gpu_inputs(1, 256, 2, 64, 2.0, seed=31, dtype=dtype)
    hA, oA = chunk_gla(*dev, 64)            # 256 tokens: 64-token tiles
    hB, oB = chunk_gla(*dev, 32)            # the same tiles, whatever chunk_size says
    scale = oA.abs().max().item()
    assert torch.equal(oA, oB) and torch.equal(hA, hB)
    # the sequence cut at token 96: both pieces (96 and 160 tokens) run on 32-token tiles
    h1, o1 = chunk_gla(dev[0], *[t[:, :96] for t in dev[1:]], 32)
    h2, o2 = chunk_gla(h1, *[t[:, 96:] for t in dev[1:]], 32)
    assert (torch.cat([o1, o2], 1) - oA).abs().max().item() < 1e-4 * scale
    assert (h2 - hA).abs().max().item() < 1e-4 * hA.abs().max().item()


def test_chunk_rejects_what_the_reference_rejects():
    from gla_jax_amd import _lib, chunk_gla
    (_, _, _, _, _), dev = gpu_inputs(1, 96, 1, 64, 2.0, seed=3, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        chunk_gla(*dev, 48)                 # not a power of two (gla.py:500)
    with pytest.raises(AssertionError):
        chunk_gla(*dev, 64)                 # 96 % 64 != 0 (einops rearrange, gla.py:674)
    with pytest.raises(_lib.GlaError):
        chunk_gla(*dev, 8)                  # below the smallest tile built here
    (_, _, _, _, _), dev = gpu_inputs(1, 64, 1, 512, 2.0, seed=3, dtype=torch.float32)
    with pytest.raises(_lib.GlaError):
        chunk_gla(*dev, 32)                 # head dimensions above 256 are not built


def _full_shape_check(B, T, H, D, chunk, shift, seed, plain=()):
    """Forward + all gradients at a BASELINE shape, EVERY batch entry and head, against the C restatement of
    the naive recurrence (fp64) and the emulated reference on the same inputs."""
    from gla_jax_amd import chunk_gla
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, shift, seed=seed, dtype=dtype)
    dhT, dout = cotangents(h0, v, seed, dtype)
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = chunk_gla(*dev, chunk)
    grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), dev)
    exact = naive_c.naive_bwd(h0, g, v, k, q, dhT, dout, dtype=np.float64, nthreads=16)
    log = check_chunk_outputs(dtype, (h0, g, v, k, q), chunk, hT, out, grads, dhT, dout, exact=exact, plain=plain)
    print("max|err|/rms:", fmt_log(log))
    # what storing the EXACT result in the tensor's own dtype costs: the floor under any implementation's error
    # (d(log_fgate) is float32: no floor to speak of)
    names = ("dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery", "hidden_final", "out")
    floor = {n: err_over_rms(O.bf16_round(np.asarray(e, dtype=np.float32)), e) for n, e in zip(names, exact)
             if n != "dlog_fgate"}
    print("storage floor:", {n: f"{x:.2e}" for n, x in floor.items()})
    return log, dev, (hT, out) + tuple(grads), (dhT, dout)


def test_chunk_baseline_config_fwd_bwd_full_shape():
    """BASELINE configs[1]/[2]: B4,T4096,H6,D128, chunk 128, gates log_sigmoid(5+N(0,1)), every batch entry and
    head.  The final state, the gradient of the initial one and d(log_fgate) meet the plain north_star bound
    (2e-2 RMS, no allowance).  out, dvalue, dkey and dquery do not: storing the exact result in bf16 costs
    1.3-1.5e-2 there, and eight operand roundings of about 1e-3 RMS each (rescaled q and k, the score blocks, the
    chunk states) bring the maximum over 12.6 M elements to 2.3-2.5e-2, where the emulated reference sits at
    3.7-4.1e-2.  They are held to 2.6e-2, a stated gap to the plain bound, not to a blanket allowance."""
    log, _, _, _ = _full_shape_check(4, 4096, 6, 128, 128, 5.0, seed=12,
                                     plain=("hidden_final", "dhidden_init", "dlog_fgate"))
    for name in ("out", "dvalue", "dkey", "dquery"):
        assert log[name][0] <= 2.6e-2, f"{name}: {log[name][0]:.3e}"
        assert log[name][0] <= 0.7 * log[name][1], f"{name}: no longer well below the emulated reference"


def test_chunk_long_context_strong_decay_full_shape():
    """BASELINE configs[3]: B1,T32768,H8,D128, chunk 128, gates log_sigmoid(N(0,1)): all eight heads against
    the oracle, and every head run alone equals, bit for bit, the same head of the full run."""
    from gla_jax_amd import chunk_gla
    log, dev, full, (dhT, dout) = _full_shape_check(1, 32768, 8, 128, 128, 0.0, seed=13)
    for h in (0, 3, 7):
        one = [(t.detach()[:, h:h + 1] if i == 0 else t.detach()[:, :, h:h + 1]).contiguous().requires_grad_(True)
               for i, t in enumerate(dev)]          # dev[0] is hidden_init [B,H,D,D], the rest are [B,T,H,D]
        hT1, out1 = chunk_gla(*one, 128)
        g1 = torch.autograd.grad(loss_of(hT1, out1, dhT[:, h:h + 1], dout[:, :, h:h + 1]), one)
        for name, a, b in zip(("hidden_final", "out") + GRAD_NAMES, (hT1, out1) + tuple(g1), full):
            b = b[:, h:h + 1] if name in ("hidden_final", "dhidden_init") else b[:, :, h:h + 1]
            assert torch.equal(a, b), f"head {h} alone differs from the full run in {name}"


def test_chunk_vmap_forward_and_gradient():
    """Batching as the reference does it (jax.vmap over a leading axis of all five arrays, then the gradient
    of a scalar loss, gla.py:1331-1344): torch.func.vmap(chunk_gla) equals the batched call bit for bit, in
    the outputs and in every gradient taken through it; a mapped axis other than 0 and an unmapped
    hidden_init work too."""
    from gla_jax_amd import chunk_gla
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(3, 128, 2, 64, 3.0, seed=8, dtype=dtype)
    dhT, dout = cotangents(h0, v, 8, dtype)
    one = lambda *a: chunk_gla(*a, 64)
    ref = [t.clone().requires_grad_(True) for t in dev]
    hT_b, out_b = chunk_gla(*ref, 64)
    g_b = torch.autograd.grad(loss_of(hT_b, out_b, dhT, dout), ref)
    mapped = [t.clone().requires_grad_(True) for t in dev]
    hT_v, out_v = torch.func.vmap(one)(*mapped)
    assert torch.equal(hT_v, hT_b) and torch.equal(out_v, out_b)
    g_v = torch.autograd.grad(loss_of(hT_v, out_v, dhT, dout), mapped)
    for a, b in zip(g_v, g_b):
        assert torch.equal(a, b)
    # functional form: grad of (loss of vmap), all five arguments
    wdh, wdo = to_dev(dhT, torch.float32), to_dev(dout, torch.float32)

    def loss(*a):
        hT, out = torch.func.vmap(one)(*a)
        return (hT.float() * wdh).sum() + (out.float() * wdo).sum()
    g_f = torch.func.grad(loss, argnums=(0, 1, 2, 3, 4))(*dev)
    for a, b in zip(g_f, g_b):
        assert torch.equal(a, b)
    # the sequence arrays mapped over axis 1, one hidden_init shared by the whole batch
    moved = [dev[0][0]] + [t.movedim(0, 1).contiguous() for t in dev[1:]]
    hT_m, out_m = torch.func.vmap(one, in_dims=(None, 1, 1, 1, 1))(*moved)
    hT_s, out_s = chunk_gla(dev[0][0].expand(3, -1, -1, -1).contiguous(), *dev[1:], 64)
    assert torch.equal(hT_m, hT_s) and torch.equal(out_m, out_s)
