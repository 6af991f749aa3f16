"""A randomized parity sweep inside the suite: small random cases of chunk_gla and recurrent_gla (both element
types, every head dimension and tile, both directions, gate shifts -2..5, scattered hard resets), each held to the
tolerance model of tests/util.py in all seven results.  The cases follow from SWEEP_SEED alone, so a failure
names a reproducible case (its index, shape, shift, seeds and resets are printed before anything is launched)
and another seed is one constant away.  The cases that earlier sweeps found are the named regression tests of
tests/test_gpu_chunk_regress.py; a case of THIS sweep that is out of bounds and not fixed is listed there as an
expected failure and here in KNOWN_OPEN: the sweep still runs it and fails if it has started to pass."""
import os
import time

import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from tests.util import (check_chunk_outputs, check_recurrent_outputs, cotangents, fmt_log, gpu_inputs, loss_of,
                        to_dev)

pytestmark = pytest.mark.gpu

# GLA_SWEEP_SEED / GLA_SWEEP_CASES in the environment run another or a longer sweep without editing this file
SWEEP_SEED = int(os.environ.get("GLA_SWEEP_SEED", "31337"))
SWEEP_CASES = int(os.environ.get("GLA_SWEEP_CASES", "150"))
SWEEP_SECONDS = 60.0 if "GLA_SWEEP_CASES" not in os.environ else 1e9   # stop drawing new cases after this long
SWEEP_MIN = min(60, SWEEP_CASES)                                       # ... but not before this many have run
# (seed, case index) -> its name in OPEN_CASES of tests/test_gpu_chunk_regress.py
KNOWN_OPEN = {(31337, 43): "s31337_c43"}


def draw_case(rng, it):
    kind = "chunk" if it % 3 != 2 else "recurrent"
    dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float32
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    shift = float(rng.choice([-2.0, 0.0, 1.0, 3.0, 5.0]))
    if kind == "chunk":
        D = int(rng.choice([16, 32, 64, 128, 128, 256])) if dtype == torch.bfloat16 else int(rng.choice([16, 32, 64, 128, 256]))
        chunk = int(rng.choice([32, 64, 128]))
        T = chunk * int(rng.integers(1, 5))
        reverse = False
    else:
        D = int(rng.choice([16, 32, 64, 64, 128]))
        T, chunk = int(rng.integers(1, 150)), 0
        reverse = bool(rng.integers(0, 2))
    resets = None
    if rng.random() < 0.4 and T > 8:
        resets = (rng.integers(0, T, size=max(1, T // 20)).tolist(), float(rng.choice([-200.0, -60.0, -25.0])))
    return dict(kind=kind, dtype=dtype, B=B, T=T, H=H, D=D, chunk=chunk, shift=shift, reverse=reverse,
                resets=resets, seed=900 + it + 1000 * SWEEP_SEED, cseed=it)


def run_case(c):
    from gla_jax_amd import chunk_gla, recurrent_gla
    dtype = c["dtype"]
    (h0, g, v, k, q), dev = gpu_inputs(c["B"], c["T"], c["H"], c["D"], c["shift"], seed=c["seed"], dtype=dtype)
    if c["resets"] is not None:
        g = g.copy()
        g[:, np.asarray(c["resets"][0])] = c["resets"][1]
        dev[1] = to_dev(g, torch.float32)
    dhT, dout = cotangents(h0, v, c["cseed"], dtype)
    dev = [t.clone().requires_grad_(True) for t in dev]
    if c["kind"] == "chunk":
        hT, out = chunk_gla(*dev, c["chunk"])
        grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), dev)
        return check_chunk_outputs(dtype, (h0, g, v, k, q), c["chunk"], hT, out, grads, dhT, dout)
    hT, out = recurrent_gla(*dev, reverse=c["reverse"])
    grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), dev)
    exact = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=c["reverse"])
    return check_recurrent_outputs(dtype, exact, hT, out, grads)


def test_randomized_sweep():
    rng = np.random.default_rng(SWEEP_SEED)
    t0 = time.time()
    worst = {}
    done = 0
    for it in range(SWEEP_CASES):
        c = draw_case(rng, it)
        if done >= SWEEP_MIN and time.time() - t0 > SWEEP_SECONDS:
            break
        print(f"sweep seed {SWEEP_SEED} case {it}: {c}", flush=True)
        if (SWEEP_SEED, it) in KNOWN_OPEN:
            with pytest.raises(AssertionError):
                run_case(c)
            print(f"  known open case {KNOWN_OPEN[(SWEEP_SEED, it)]}: still out of bounds")
            done += 1
            continue
        log = run_case(c)                    # raises on the first tensor out of bounds: the line above names the case
        done += 1
        for name, (a, b) in log.items():
            if b:
                ratio = a / max(b, 1e-30)
                if ratio > worst.get((c["kind"], name), (0.0,))[0]:
                    worst[(c["kind"], name)] = (ratio, a, b, it)
    print(f"{done} cases in {time.time() - t0:.1f} s; worst ratio to the emulated reference per tensor:")
    for key, (ratio, a, b, it) in sorted(worst.items()):
        print(f"  {key[0]:9s} {key[1]:13s} {ratio:.2f} (hip {a:.2e}, reference {b:.2e}, case {it})")
    assert done >= SWEEP_MIN
