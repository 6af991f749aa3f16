"""Benchmark and three-way self-check of the public entry points, the counterpart of `python gla.py`
(test_speed, gla.py:1275-1499) of zhixuan-lin/gla-jax:

    python -m gla_jax_amd.selfcheck [--batch 4 --seq-len 4096 --key-dim 2048 --head-dim 128]
                                    [--dtype bf16|fp32] [--reverse] [--methods a,b,c] [--no-grad] [--json]

Every method of {recurrent_gla_naive, recurrent_gla, chunk_gla} (gla.py:1308-1312) runs on the same seeded
inputs, batched over the leading axis, with the loss hidden_final.sum() + out.sum() (all-ones cotangents,
gla.py:1336-1338) and gradients with respect to all five arrays (gla.py:1340).  For each method the first call
is timed apart from the steady state (the reference prints it as compilation time, gla.py:1404-1424; here it is
the loading of the kernels), and the steady state is timed the way timeit's autorange does it
(gla.py:1430-1434): repeat counts 1, 2, 5, 10, ... until a batch of calls takes at least 0.2 s, every output
complete before the clock stops (gla.py:1397).  Then every pair of methods is compared on each of the seven
results (hidden_final, out, dhidden_init, dlog_fgate, dvalue, dkey, dquery): whether they agree to
allclose's defaults (rtol 1e-5, atol 1e-8), the largest absolute difference and the relative L2 difference
||a - b|| / ||a|| (gla.py:1452-1465).  Like the reference, the script reports and does not judge: it exits 0
unless a result is not finite.

Defaults follow the reference's script: batch 4, 4096 tokens, key_dim 2048 split into heads of 128
(16 heads), chunk_size = head_dim, bf16, gates log_sigmoid(5 + N(0,1)) in fp32 (gla.py:1288-1299, 1386-1392).
One difference on purpose: the reference draws every array from the same PRNG key (value == key == query);
here each array has its own stream.  `reverse` applies to the two recurrent methods only, as in the reference
(chunk_gla has no such argument, gla.py:657-669), so with it the pairs that involve chunk_gla are skipped.
"""
from __future__ import annotations

import argparse
import itertools
import json
import sys
import time

import torch

METHODS = ("recurrent_gla_naive", "recurrent_gla", "chunk_gla")
RESULTS = ("hidden_final", "out", "dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery")


def make_inputs(batch, seq_len, heads, head_dim, dtype, gate_shift=5.0, seed=0, device="cuda"):
    """hidden_init [B,H,D,D], log_fgate/value/key/query [B,T,H,D] (gla.py:1386-1392), one generator per array."""
    def rn(i, *shape):
        g = torch.Generator(device=device).manual_seed(1000 * seed + i)
        return torch.randn(*shape, generator=g, device=device, dtype=torch.float32)
    hidden_init = rn(0, batch, heads, head_dim, head_dim).to(dtype)
    log_fgate = torch.nn.functional.logsigmoid(gate_shift + rn(1, batch, seq_len, heads, head_dim))
    value, key, query = (rn(i, batch, seq_len, heads, head_dim).to(dtype) for i in (2, 3, 4))
    return hidden_init, log_fgate, value, key, query


def _bind(name, chunk_size, reverse):
    from . import chunk_gla, recurrent_gla, recurrent_gla_naive
    if name == "chunk_gla":
        return lambda *a: chunk_gla(*a, chunk_size)
    if name == "recurrent_gla":
        return lambda *a: recurrent_gla(*a, reverse=reverse)
    if name == "recurrent_gla_naive":
        return lambda *a: recurrent_gla_naive(*a, reverse)
    raise ValueError(f"unknown method {name!r}; choose from {METHODS}")


def run_method(name, inputs, chunk_size, reverse=False, grad=True):
    """One forward (+ backward) of `name`; returns the dict of results of gla.py:1406-1420."""
    fn = _bind(name, chunk_size, reverse)
    if not grad:
        with torch.no_grad():
            hidden_final, out = fn(*inputs)
        return {"hidden_final": hidden_final, "out": out}
    args = [t.detach().requires_grad_(True) for t in inputs]
    hidden_final, out = fn(*args)
    loss = hidden_final.float().sum() + out.float().sum()          # gla.py:1336-1338
    grads = torch.autograd.grad(loss, args)
    res = {"hidden_final": hidden_final.detach(), "out": out.detach()}
    res.update(zip(RESULTS[2:], grads))
    return res


def autorange(stmt, min_time=0.2):
    """timeit.Timer.autorange with a device synchronisation inside the clock: returns (calls, seconds)."""
    i = 1
    while True:
        for j in (1, 2, 5):
            number = i * j
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(number):
                stmt()
            torch.cuda.synchronize()
            taken = time.perf_counter() - t0
            if taken >= min_time:
                return number, taken
        i *= 10


def compare(a, b):
    """allclose at jnp.allclose's defaults, max |a - b| and ||a - b|| / ||a|| in fp32 (gla.py:1452-1465)."""
    af, bf = a.float(), b.float()
    diff = af - bf
    return {
        "allclose": bool(torch.allclose(af, bf, rtol=1e-5, atol=1e-8)),
        "max_abs": float(diff.abs().max()),
        "rel_l2": float(torch.linalg.vector_norm(diff) / torch.linalg.vector_norm(af).clamp_min(1e-30)),
    }


def selfcheck(batch=4, seq_len=4096, key_dim=2048, head_dim=128, dtype=torch.bfloat16, reverse=False,
              methods=METHODS, grad=True, check=True, time_it=True, gate_shift=5.0, seed=0, out="stdout"):
    """Runs the methods, prints the reference's report to `out` (a file object; "stdout": sys.stdout as it is
    when the call is made; None: silent) and returns it as a dict."""
    if isinstance(out, str):
        out = sys.stdout
    if key_dim % head_dim:
        raise ValueError(f"key_dim {key_dim} is not a multiple of head_dim {head_dim}")
    heads = key_dim // head_dim                                    # gla.py:1317
    chunk_size = head_dim                                          # gla.py:1319
    say = (lambda *a: print(*a, file=out)) if out is not None else (lambda *a: None)
    inputs = make_inputs(batch, seq_len, heads, head_dim, dtype, gate_shift, seed)
    report = {"config": {"batch_size": batch, "seq_len": seq_len, "key_dim": key_dim, "head_dim": head_dim,
                         "num_heads": heads, "chunk_size": chunk_size, "dtype": str(dtype).split(".")[-1],
                         "reverse": bool(reverse), "grad": bool(grad)},
              "methods": {}, "pairs": {}}
    results = {}
    for name in methods:
        say("=" * 80)
        say(f"seq_len: {seq_len}")
        say(f"head_dim: {head_dim}")
        say(f"batch_size: {batch}")
        say(name)
        stmt = lambda: run_method(name, inputs, chunk_size, reverse, grad)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        results[name] = stmt()
        torch.cuda.synchronize()
        first = time.perf_counter() - t0
        say(f"First call (kernel loading): {first}s")
        entry = {"first_call_s": first}
        if time_it:
            number, taken = autorange(stmt)
            entry.update(iterations=number, time_ms=taken / number * 1e3,
                         mtokens_per_s=batch * seq_len * number / taken / 1e6)
            say(f"Length: {seq_len}")
            say(f"Iterations: {number}")
            say(f"Time: {taken / number * 1e3}ms")
        for key, val in results[name].items():
            if not bool(torch.isfinite(val.float()).all()):
                entry.setdefault("non_finite", []).append(key)
        report["methods"][name] = entry
        say("=" * 80)
    if check and len(results) >= 2:
        for a, b in itertools.combinations(results, 2):
            if reverse and "chunk_gla" in (a, b):
                say(f"Skipping {a} and {b}: chunk_gla has no reverse argument")
                continue
            say(f"Verifying {a} and {b}")
            pair = {}
            for key in results[a]:
                c = compare(results[a][key], results[b][key])
                pair[key] = c
                if not c["allclose"]:
                    say(f"  {a}->{key} and {b}->{key} do not match")
                    say(f"    Max abs error {c['max_abs']}")
                    say(f"    Rel error {c['rel_l2']}")
            report["pairs"][f"{a} vs {b}"] = pair
    return report


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m gla_jax_amd.selfcheck", description=__doc__.split("\n\n")[0])
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--seq-len", type=int, default=4096)
    ap.add_argument("--key-dim", type=int, default=2048)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--dtype", choices=("bf16", "fp32"), default="bf16")
    ap.add_argument("--gate-shift", type=float, default=5.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--reverse", action="store_true")
    ap.add_argument("--methods", default=",".join(METHODS))
    ap.add_argument("--no-grad", action="store_true", help="forward only (GRAD = False in the reference)")
    ap.add_argument("--no-check", action="store_true", help="skip the pairwise comparison (CHECK = False)")
    ap.add_argument("--no-time", action="store_true", help="skip the steady-state timing")
    ap.add_argument("--json", action="store_true", help="print the report as one JSON line at the end")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("gla_jax_amd.selfcheck needs a GPU: the library has no CPU path")
    rep = selfcheck(args.batch, args.seq_len, args.key_dim, args.head_dim,
                    torch.bfloat16 if args.dtype == "bf16" else torch.float32, args.reverse,
                    tuple(m for m in args.methods.split(",") if m), not args.no_grad, not args.no_check,
                    not args.no_time, args.gate_shift, args.seed)
    if args.json:
        print(json.dumps(rep))
    bad = {m: e["non_finite"] for m, e in rep["methods"].items() if e.get("non_finite")}
    if bad:
        sys.exit(f"non-finite results: {bad}")


if __name__ == "__main__":
    main()
