"""The committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from the fp64
oracle) against three independent routes on the CPU: the NumPy oracle as it is now, the C restatement, and
torch.autograd through a separately written torch loop.  A change that moves the oracle's results fails
here; the GPU tests compare the HIP path with the same files (tests/test_gpu_golden.py)."""
import os

import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from oracle import naive_c
from tests.test_oracle import autograd_reference

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GRADS = ("dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery")
INPUTS = ("hidden_init", "log_fgate", "value", "key", "query")


def load(name):
    with np.load(os.path.join(GOLDEN, name)) as z:      # plain arrays only: no pickle is involved
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("name,rtol", [("gla_T12_H2_D8.npz", 1e-12), ("gla_T64_H1_D64.npz", 2e-6)])
def test_oracle_reproduces_the_golden_recurrence(name, rtol):
    d = load(name)
    ins = [d[k] for k in INPUTS]
    for tag, reverse in (("fwd", False), ("rev", True)):
        hT, out = O.recurrent_gla_naive(*ins, reverse=reverse)
        grads = O.recurrent_gla_naive_grad(*ins, d["dhidden_final"], d["dout"], reverse=reverse)
        scale = lambda a: rtol * max(1.0, float(np.abs(a).max()))
        np.testing.assert_allclose(hT, d[f"{tag}_hidden_final"], rtol=rtol, atol=scale(hT))
        np.testing.assert_allclose(out, d[f"{tag}_out"], rtol=rtol, atol=scale(out))
        for gname, gval in zip(GRADS, grads):
            np.testing.assert_allclose(gval, d[f"{tag}_{gname}"], rtol=rtol, atol=scale(gval), err_msg=gname)


def test_golden_gradients_are_what_autograd_gives():
    """Not the oracle's two-sweep formula: torch.autograd (fp64) through an independent loop."""
    d = load("gla_T12_H2_D8.npz")
    ins = [d[k].astype(np.float64) for k in INPUTS]
    grads, hT, out = autograd_reference(*ins, d["dhidden_final"].astype(np.float64), d["dout"].astype(np.float64))
    np.testing.assert_allclose(hT, d["fwd_hidden_final"], rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(out, d["fwd_out"], rtol=1e-10, atol=1e-11)
    for gname, gval in zip(GRADS, grads):
        np.testing.assert_allclose(gval, d[f"fwd_{gname}"], rtol=1e-10, atol=1e-10, err_msg=gname)


def test_chunked_oracle_reproduces_the_golden_forward_and_gradients():
    d = load("gla_T64_H1_D64.npz")
    ins = [d[k] for k in INPUTS]
    for chunk in (32, 64):
        hT, out, res = O.chunk_gla_forward(*ins, chunk, block_size_t=16)
        grads = O.chunk_gla_backward(*ins[1:], res, d["dhidden_final"], d["dout"], chunk, block_size_t=16)
        for got, key in ((hT, "fwd_hidden_final"), (out, "fwd_out")):
            assert np.abs(got - d[key]).max() <= 1e-5 * np.abs(d[key]).max(), (chunk, key)
        for gname, gval in zip(GRADS, grads):
            assert np.abs(gval - d[f"fwd_{gname}"]).max() <= 1e-5 * np.abs(d[f"fwd_{gname}"]).max(), (chunk, gname)


def test_c_restatement_reproduces_the_golden_recurrence():
    d = load("gla_T64_H1_D64.npz")
    ins = [d[k][None] for k in INPUTS]                 # the C side takes a batch axis
    hT, out = naive_c.naive_fwd(*ins, dtype=np.float64)
    np.testing.assert_allclose(hT[0], d["fwd_hidden_final"], rtol=2e-6, atol=2e-6 * np.abs(hT).max())
    np.testing.assert_allclose(out[0], d["fwd_out"], rtol=2e-6, atol=2e-6 * np.abs(out).max())
    hT, out = naive_c.naive_fwd(*ins, reverse=True, dtype=np.float64)
    np.testing.assert_allclose(out[0], d["rev_out"], rtol=2e-6, atol=2e-6 * np.abs(out).max())
    res = naive_c.naive_bwd(*ins, d["dhidden_final"][None], d["dout"][None], dtype=np.float64)
    for gname, gval in zip(GRADS, res[:5]):
        ref = d[f"fwd_{gname}"]
        np.testing.assert_allclose(gval[0], ref, rtol=2e-6, atol=2e-6 * np.abs(ref).max(), err_msg=gname)


def test_golden_scans():
    d = load("scans.npz")
    src, init = d["cumsum_src"].astype(np.float64), d["cumsum_init"].astype(np.float64)
    # cumsum: np.cumsum on flipped data, written out here rather than through the oracle
    for reverse in (False, True):
        x = src[:, ::-1] if reverse else src
        y = np.cumsum(x, axis=1)
        y = y[:, ::-1] if reverse else y
        tag = "rev" if reverse else "fwd"
        np.testing.assert_allclose(d[f"cumsum_{tag}_noinit"], y, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(d[f"cumsum_{tag}_init"], y + init[:, None, :], rtol=1e-12, atol=1e-12)
    # diagonal recurrence: explicit loop over the steps
    a, b = d["rnn_log_fgate"].astype(np.float64), d["rnn_kv"].astype(np.float64)
    ia, ib = d["rnn_init_log_fgate"].astype(np.float64), d["rnn_init_kv"].astype(np.float64)
    for reverse in (False, True):
        for with_init in (False, True):
            tag = f"{'rev' if reverse else 'fwd'}_{'init' if with_init else 'noinit'}"
            x = ib.copy() if with_init else np.zeros_like(ib)
            ca = ia.copy() if with_init else np.zeros_like(ia)
            steps = range(a.shape[0] - 1, -1, -1) if reverse else range(a.shape[0])
            for n in steps:
                x = np.exp(a[n])[:, None] * x + b[n]
                ca = ca + a[n]
                np.testing.assert_allclose(d[f"rnn_x_{tag}"][n], x, rtol=1e-12, atol=1e-12)
                np.testing.assert_allclose(d[f"rnn_a_{tag}"][n], ca, rtol=1e-12, atol=1e-12)
