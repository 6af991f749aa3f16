"""Writes the golden vectors of the parity tests (tests/golden/*.npz) from the fp64 oracle.

    python -m tests.golden.make_golden          (from the repository root)

The reference holds no golden vectors, known-answer tests or fixtures for this path and cannot be imported
(jax is absent), so these files are not reference outputs: they freeze what the oracle computes today, after
the oracle itself was pinned by closed forms, autograd and brute force (tests/test_oracle.py).  They serve
two purposes: a later change of the oracle that moves its results is caught on the CPU
(tests/test_golden.py), and the HIP path is compared against data that does not depend on the oracle's
code at test time (tests/test_gpu_golden.py).

Every file holds its inputs, so the tests never regenerate them.  q, k, v, the initial state and the
cotangents are bf16-representable: the same file feeds the bf16 and the fp32 kernels.  Outputs are stored
in float64, except where noted.
"""
import os

import numpy as np

from oracle import gla_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


def _draw(rng, shape, bf16=True):
    x = rng.standard_normal(shape, dtype=np.float32)
    return O.bf16_round(x) if bf16 else x


def gla_case(name, T, H, D, shift, seed, resets=(), out_dtype=np.float64):
    """One sequence [T,H,D] (no batch axis): forward and all five gradients of the recurrence
    (gla.py:26-47, 297-359, 263) in both scan directions; chunk_gla must reproduce the forward direction."""
    rng = np.random.default_rng(seed)
    h0 = _draw(rng, (H, D, D))
    g = O.log_sigmoid(shift + rng.standard_normal((T, H, D))).astype(np.float32)
    for t, val in resets:
        g[t] = val
    v, k, q = (_draw(rng, (T, H, D)) for _ in range(3))
    dhT = _draw(rng, (H, D, D))
    dout = _draw(rng, (T, H, D))
    data = dict(hidden_init=h0, log_fgate=g, value=v, key=k, query=q, dhidden_final=dhT, dout=dout)
    for tag, reverse in (("fwd", False), ("rev", True)):
        hT, out = O.recurrent_gla_naive(h0, g, v, k, q, reverse=reverse)
        grads = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
        data[f"{tag}_hidden_final"] = hT.astype(out_dtype)
        data[f"{tag}_out"] = out.astype(out_dtype)
        for gname, gval in zip(("dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery"), grads[:5]):
            data[f"{tag}_{gname}"] = np.asarray(gval).astype(out_dtype)
    np.savez_compressed(os.path.join(HERE, name), **data)


def scan_case(name, seed):
    """cumsum (ops.py:234-284) and the diagonal RNN scan (ops.py:286-456), with and without init, both directions."""
    rng = np.random.default_rng(seed)
    src = rng.standard_normal((3, 37, 5), dtype=np.float32)
    cinit = rng.standard_normal((3, 5), dtype=np.float32)
    a = -np.abs(rng.standard_normal((6, 8), dtype=np.float32))
    b = rng.standard_normal((6, 8, 4), dtype=np.float32)
    ia = -np.abs(rng.standard_normal((8,), dtype=np.float32))
    ib = rng.standard_normal((8, 4), dtype=np.float32)
    data = dict(cumsum_src=src, cumsum_init=cinit, rnn_log_fgate=a, rnn_kv=b, rnn_init_log_fgate=ia, rnn_init_kv=ib)
    for reverse in (False, True):
        for with_init in (False, True):
            tag = f"{'rev' if reverse else 'fwd'}_{'init' if with_init else 'noinit'}"
            data[f"cumsum_{tag}"] = O.cumsum(src, 1, init=cinit if with_init else None, reverse=reverse)
            ca, cx = O.rnn_scan(a, b, ia if with_init else None, ib if with_init else None, reverse=reverse)
            data[f"rnn_a_{tag}"] = ca
            data[f"rnn_x_{tag}"] = cx
    np.savez_compressed(os.path.join(HERE, name), **data)


def main():
    # tiny: pins the oracle to 1e-12 (and the C restatement beside it)
    gla_case("gla_T12_H2_D8.npz", T=12, H=2, D=8, shift=1.0, seed=11)
    # the smallest shape every HIP path accepts (head dim 64; chunk sizes 32 and 64): mixed gates with
    # one full reset and one strong decay inside a 16-token sub-block.  Outputs in float32 (file size).
    gla_case("gla_T64_H1_D64.npz", T=64, H=1, D=64, shift=1.0, seed=12, resets=((21, -200.0), (40, -30.0)),
             out_dtype=np.float32)
    scan_case("scans.npz", seed=13)


if __name__ == "__main__":
    main()
