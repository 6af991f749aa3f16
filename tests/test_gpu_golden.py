"""The HIP path, through the C ABI, against the committed golden vectors (tests/golden/*.npz): chunk_gla at
every tile size, recurrent_gla in both directions and both element types, and the two stand-alone scans.
Tolerance as everywhere (north_star): max|err| / RMS <= 2e-2 for bf16, <= 1e-4 for fp32."""
import numpy as np
import pytest
import torch

from tests.test_golden import GRADS, INPUTS, load
from tests.util import GRAD_NAMES, TOL, check_chunk_outputs, check_recurrent_outputs, err_over_rms, to_dev, to_np

pytestmark = pytest.mark.gpu


def device_inputs(d, dtype):
    return [to_dev(d[k], torch.float32 if k == "log_fgate" else dtype) for k in INPUTS]


def golden(d, tag):
    """(dh0, dg, dv, dk, dq, hidden_final, out) of the fixture, in the oracle's order."""
    assert tuple(GRADS) == GRAD_NAMES
    return tuple(d[f"{tag}_{n}"] for n in GRADS) + (d[f"{tag}_hidden_final"], d[f"{tag}_out"])


def fwd_bwd(fn, d, dtype, **kw):
    dev = [t.requires_grad_(True) for t in device_inputs(d, dtype)]
    hT, out = fn(*dev, **kw)
    loss = (hT.float() * to_dev(d["dhidden_final"], torch.float32)).sum() + \
           (out.float() * to_dev(d["dout"], torch.float32)).sum()
    return hT, out, torch.autograd.grad(loss, dev)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("chunk", [32, 64])
def test_chunk_gla_against_golden(dtype, chunk):
    from gla_jax_amd import chunk_gla
    d = load("gla_T64_H1_D64.npz")
    hT, out, grads = fwd_bwd(chunk_gla, d, dtype, chunk_size=chunk)
    arrs = tuple(np.asarray(d[k_], dtype=np.float32)[None] for k_ in INPUTS)
    lead = lambda a: np.asarray(a)[None]
    check_chunk_outputs(dtype, arrs, chunk, hT[None], out[None], [t[None] for t in grads],
                        lead(d["dhidden_final"]), lead(d["dout"]), exact=tuple(lead(a) for a in golden(d, "fwd")))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("reverse", [False, True])
def test_recurrent_gla_against_golden(dtype, reverse):
    from gla_jax_amd import recurrent_gla
    d = load("gla_T64_H1_D64.npz")
    hT, out, grads = fwd_bwd(recurrent_gla, d, dtype, reverse=reverse)
    check_recurrent_outputs(dtype, golden(d, "rev" if reverse else "fwd"), hT, out, grads)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("reverse", [False, True])
def test_recurrent_gla_small_head_dim_against_golden(dtype, reverse):
    """Head dim 8 is below the kernels' smallest state: the front-end pads the rows to 16 and cuts the results back."""
    from gla_jax_amd import recurrent_gla
    d = load("gla_T12_H2_D8.npz")
    hT, out, grads = fwd_bwd(recurrent_gla, d, dtype, reverse=reverse)
    assert out.shape[-1] == 8 and hT.shape[-2:] == (8, 8)
    check_recurrent_outputs(dtype, golden(d, "rev" if reverse else "fwd"), hT, out, grads)


def test_scans_against_golden():
    from gla_jax_amd import cumsum_recursive, rnn_recursive
    d = load("scans.npz")
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
    for reverse in (False, True):
        for with_init in (False, True):
            tag = f"{'rev' if reverse else 'fwd'}_{'init' if with_init else 'noinit'}"
            got = cumsum_recursive(dev(d["cumsum_src"]), 1, init=dev(d["cumsum_init"]) if with_init else None,
                                   reverse=reverse)
            assert err_over_rms(to_np(got), d[f"cumsum_{tag}"]) < 1e-5, tag
            ga, gx = rnn_recursive(dev(d["rnn_log_fgate"]), dev(d["rnn_kv"]),
                                   dev(d["rnn_init_log_fgate"]) if with_init else None,
                                   dev(d["rnn_init_kv"]) if with_init else None, reverse=reverse)
            assert err_over_rms(to_np(ga), d[f"rnn_a_{tag}"]) < 1e-5, tag
            assert err_over_rms(to_np(gx), d[f"rnn_x_{tag}"]) < 1e-5, tag
