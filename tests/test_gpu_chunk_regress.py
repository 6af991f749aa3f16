"""bf16 chunk_gla cases that randomized sweeps (small shapes, gate shifts -2..5, scattered resets) found out of
bounds, kept as named cases and held to the tolerance model of tests/util.py (north_star's 2e-2 RMS, or 1.5 x
the emulated reference's own error on the same inputs).

Two families.  The first nine sat 0.1-20 % above an earlier, hand-set tolerance (`2e-2 RMS + one bf16 ulp of the
element`) in one gradient tensor each.  The other eleven failed the present model in d(log_fgate) only, all under
strong decay (gate shift 0 or 1): with ONE anchor per 16-token sub-block and plain bf16 operands the gate
gradient came out up to 2.2 x less accurate than the reference's dyadic anchors give it; the gradient kernel
now takes the operands of a sub-block's own products as bf16 head + remainder (gla_chunk_bwd.hip), and a
repeat of both sweeps (330 cases) finds every tensor within the model, the worst ratio to the emulated
reference being 1.47 (d(log_fgate), at 2.3e-2 RMS).

A third pair came from later sweeps (some 1 300 cases with other seeds): d(log_fgate) 1.56 x and 1.73 x the
emulated reference's error, one with mild and one with strong gates.  Both were the chunk-level term of
gla.py:782, which the gradient kernel formed as sum_v dS' * S_{n+1} from the STORED state after the chunk: that
carries the bf16 rounding of a whole state, where the reference's two terms carry the rounding of a decayed
state and of single key rows.  The kernel now forms the two terms as the reference does (gla_chunk_bwd.hip).

A last one (of a further 300) had dvalue at 1.505 x the emulated reference's error (bound 1.5 x): the bf16
rounding of the score blocks as the operand of dv = A^T dO, under strong decay, where the own sub-block's scores
carry most of dv.  Those now enter that product (and out = A V in the forward) as bf16 head + remainder.

OPEN_CASES lists cases that are known to fail and not fixed; they are expected failures (strict: a case that
starts to pass must be moved to SWEEP_CASES).  Three cases.  Two are of five further sweeps of 400 cases each (the suite's
own sweep with other seeds).  The first: d(log_fgate) of a head-dimension-32 case (one 64-token chunk, three hard
resets) at 2.35e-2 RMS = 1.63 x the emulated reference (bound 1.5 x).  Per token the gate-cumsum gradient of the
kernel and of the emulated reference are off by the same amounts (0.1-0.5 in values of 5-150: the bf16 rounding
of the operands of the dq / dk products); d(log_fgate) is their reverse running sum, a random walk that on these
inputs ends at +1.1 for the kernel and +0.6 for the reference at the worst token.  With 32 features a sum has a
quarter of the terms it has at D=128 and the ratio of the two maxima scatters accordingly.  Taking the dyadic
levels' operand as head + remainder (like the one-anchor path's) changes nothing here and costs the gradient
kernel spills: not kept.

The second: dvalue of a head-dimension-16 case (one 128-token chunk, six resets to -25) at 4.42e-2 RMS = 1.57 x the
emulated reference.  It is ONE element, ten RMS large: the exact value is 140.389, its bf16 neighbours are 140 and
141, the emulated reference stores 140 (off by 0.389 = 2.8e-2 RMS, the storage rounding of the exact value) and the
kernel 141 (off by 0.611): an error of 0.11 before rounding, 0.8e-2 RMS, put the kernel's value past the midpoint.
Both are neighbours of the exact value; over the whole tensor the kernel's L2 error is 0.85 x the emulated
reference's (2.99e-3 against 3.51e-3 of an RMS) and with five other cotangents for the same inputs the ratio of the
maxima is 0.5-0.9.  A bound of 1.5 x the reference's maximum cannot hold against a rounding that falls to the other
neighbour where the reference's own error on that element is below 0.4 of a spacing; the bound is left as it is and
the case is listed.

The third is case 43 of the suite's own sweep (tests/test_gpu_sweep.py, which runs it as a known open case), a
head-dimension-256 case with three resets to -25 in one 64-token chunk.  It passed (0.88 x) while head dimension
256 had kernels of its own on 32-token tiles and is at 1.63 x in d(log_fgate) since it runs as four problems of head
dimension 128 (gla_split.hip): the error is one pair term, rows 11 and 17 of a key feature whose gate
gradient is nine RMS large (657 where the RMS is 76), off by 0.5 % where the emulated reference is off by 0.26 %.
dA = dO V^T of that pair is now the sum of two halves over the value features, each rounded to bf16 on its own; on
average that costs nothing (40 random head-dimension-256 cases: median 0.90, largest 1.21, against 0.90 and 1.17
before; every other tensor at 0.70 as before) and a single large term can come out either way."""
import numpy as np
import pytest
import torch

from tests.util import check_chunk_outputs, cotangents, fmt_log, gpu_inputs, loss_of, to_dev

pytestmark = pytest.mark.gpu

# name: (B, T, H, D, chunk, gate shift, input seed, cotangent seed, reset rows or None, reset value, tensor that failed)
SWEEP_CASES = {
    "s77_c10": (3, 128, 4, 128, 32, 1.0, 510, 10, None, 0.0, "dvalue"),
    "s77_c88": (3, 256, 4, 64, 128, 3.0, 588, 88, None, 0.0, "dvalue"),
    "s77_c98": (2, 192, 2, 128, 64, 5.0, 598, 98, [172, 59, 86, 150, 4, 54, 185, 60, 157], -25.0, "dvalue"),
    "s77_c204": (2, 128, 3, 64, 128, 1.0, 704, 204, None, 0.0, "dquery"),
    "s51_c90": (3, 640, 2, 64, 128, 5.0, 590, 90,
                [257, 394, 477, 383, 551, 80, 634, 197, 173, 614, 186, 278, 93, 205, 604, 473, 453, 259, 131, 396,
                 540, 325, 263, 601, 497, 67, 508, 247, 528, 67, 631, 510], -200.0, "dkey"),
    "s51_c94": (1, 960, 2, 64, 64, 5.0, 594, 94,
                [816, 912, 775, 718, 859, 527, 359, 583, 427, 250, 433, 283, 805, 710, 928, 821, 197, 20, 238, 907,
                 738, 869, 480, 264, 236, 127, 100, 419, 220, 930, 219, 293, 838, 586, 499, 873, 765, 166, 869, 333,
                 693, 262, 724, 40, 551, 400, 44, 846], -60.0, "dvalue"),
    "s43_c60": (3, 384, 4, 128, 128, 5.0, 560, 60,
                [335, 286, 56, 27, 235, 293, 356, 117, 85, 377, 334, 107, 362, 116, 370, 335, 244, 100, 249], -25.0,
                "dvalue"),
    "s43_c178": (3, 384, 4, 128, 128, 0.0, 678, 178, None, 0.0, "dhidden_init"),
    "s41_c212": (3, 128, 4, 128, 128, 3.0, 712, 212, None, 0.0, "dquery"),
    # second family: d(log_fgate) under strong decay
    "s101_c19": (1, 64, 3, 128, 32, 0.0, 101919, 19, [42, 2, 4], -60.0, "dlog_fgate"),
    "s101_c51": (2, 128, 4, 128, 32, 1.0, 101951, 51, None, 0.0, "dlog_fgate"),
    "s101_c94": (2, 128, 1, 128, 128, 1.0, 101994, 94, None, 0.0, "dlog_fgate"),
    "s101_c115": (1, 96, 2, 128, 32, 1.0, 102015, 115, None, 0.0, "dlog_fgate"),
    "s101_c123": (1, 64, 1, 64, 32, 1.0, 102023, 123, [2, 20, 22], -25.0, "dlog_fgate"),
    "s101_c136": (2, 32, 2, 64, 32, 0.0, 102036, 136, None, 0.0, "dlog_fgate"),
    "s101_c165": (1, 512, 4, 128, 128, 0.0, 102065, 165, None, 0.0, "dlog_fgate"),
    "s101_c180": (1, 64, 1, 64, 32, 0.0, 102080, 180, None, 0.0, "dlog_fgate"),
    "s202_c1": (2, 576, 2, 128, 64, 1.0, 202901, 1, None, 0.0, "dlog_fgate"),
    "s202_c6": (1, 768, 1, 64, 128, 0.0, 202906, 6, None, 0.0, "dlog_fgate"),
    "s202_c88": (2, 896, 4, 256, 128, 1.0, 202988, 88, None, 0.0, "dlog_fgate"),
    # third family: the chunk-level term of d(log_fgate)
    "s505_c115": (3, 384, 2, 128, 128, 5.0, 506015, 115, None, 0.0, "dlog_fgate"),
    "s606_c64": (1, 64, 1, 64, 32, -2.0, 606964, 64, None, 0.0, "dlog_fgate"),
    # dvalue under strong decay: the own sub-block's scores as the operand of dv = A^T dO
    "s707_c228": (2, 256, 1, 64, 128, 1.0, 708128, 228, None, 0.0, "dvalue"),
}


# found by a sweep, out of bounds, not fixed (see the module docstring)
OPEN_CASES = {
    "s202_c342": (1, 64, 4, 32, 32, 5.0, 203242, 342, [55, 13, 23], -200.0, "dlog_fgate"),
    "s404_c360": (2, 128, 2, 16, 32, 5.0, 405260, 360, [102, 57, 35, 46, 68, 56], -25.0, "dvalue"),
    "s31337_c43": (2, 64, 3, 256, 64, 3.0, 31337943, 43, [19, 34, 26], -25.0, "dlog_fgate"),
}
OPEN_REASONS = {
    "s202_c342": "d(log_fgate) 1.63 x the emulated reference (bound 1.5 x), see the module docstring",
    "s404_c360": "dvalue 1.57 x the emulated reference (bound 1.5 x): one element stored as the other bf16 neighbour "
                 "of the exact value, see the module docstring",
    "s31337_c43": "d(log_fgate) 1.63 x the emulated reference (bound 1.5 x): one pair term of a head-dimension-256 "
                  "case, see the module docstring",
}


@pytest.mark.parametrize("case", sorted(SWEEP_CASES) + [
    pytest.param(c, marks=pytest.mark.xfail(reason=OPEN_REASONS[c], strict=True, raises=AssertionError))
    for c in sorted(OPEN_CASES)])
def test_chunk_sweep_case(case):
    from gla_jax_amd import chunk_gla
    B, T, H, D, chunk, shift, seed, cseed, rows, val, _ = {**SWEEP_CASES, **OPEN_CASES}[case]
    dtype = torch.bfloat16
    (h0, g, v, k, q), dev = gpu_inputs(B, T, H, D, shift, seed=seed, dtype=dtype)
    if rows is not None:
        g = g.copy()
        g[:, np.asarray(rows)] = val
        dev[1] = to_dev(g, torch.float32)
    dhT, dout = cotangents(h0, v, cseed, dtype)
    dev = [t.clone().requires_grad_(True) for t in dev]
    hT, out = chunk_gla(*dev, chunk)
    grads = torch.autograd.grad(loss_of(hT, out, dhT, dout), dev)
    print(case, fmt_log(check_chunk_outputs(dtype, (h0, g, v, k, q), chunk, hT, out, grads, dhT, dout)))
