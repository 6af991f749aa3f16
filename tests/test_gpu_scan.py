"""GPU parity of the stand-alone scans (ops.py operators) against the oracle; bit-level agreement is
not expected for fp32 sums in a different order, so the bound is 1e-5 relative to the result's RMS."""
import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from tests.util import err_over_rms, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,axis", [((3, 128, 96), 1), ((2, 5, 37, 6, 64), 2), ((4096, 40), 0),
                                        ((7, 300), 1), ((24, 32, 128, 128), 2)])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
def test_cumsum_recursive(shape, axis, reverse, with_init):
    from gla_jax_amd import cumsum_recursive
    rng = np.random.default_rng(1)
    x = rng.standard_normal(shape, dtype=np.float32)
    ishape = shape[:axis] + shape[axis + 1:]
    init = rng.standard_normal(ishape, dtype=np.float32) if with_init else None
    got = cumsum_recursive(torch.from_numpy(x).cuda(), axis,
                           init=None if init is None else torch.from_numpy(init).cuda(), reverse=reverse)
    exp = O.cumsum(x, axis, init=init, reverse=reverse)
    assert err_over_rms(to_np(got), exp) < 1e-5


@pytest.mark.parametrize("T,K,V,batch", [(32, 128, 128, None), (256, 16, 64, 3), (5, 8, 4, None),
                                           (19, 5, 7, 2), (9, 3, 1, None), (33, 4, 6, None)])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
def test_rnn_recursive(T, K, V, batch, reverse, with_init):
    from gla_jax_amd import rnn_recursive
    rng = np.random.default_rng(2)
    lead = () if batch is None else (batch,)
    a = -np.abs(rng.standard_normal(lead + (T, K), dtype=np.float32))
    b = rng.standard_normal(lead + (T, K, V), dtype=np.float32)
    ia = -np.abs(rng.standard_normal(lead + (K,), dtype=np.float32)) if with_init else None
    ib = rng.standard_normal(lead + (K, V), dtype=np.float32) if with_init else None
    dev = lambda z: None if z is None else torch.from_numpy(z).cuda()
    ga, gx = rnn_recursive(dev(a), dev(b), dev(ia), dev(ib), reverse=reverse)
    for i in range(batch or 1):
        sel = (lambda z: z) if batch is None else (lambda z: None if z is None else z[i])
        ea, ex = O.rnn_scan(sel(a), sel(b), sel(ia), sel(ib), reverse=reverse)
        assert err_over_rms(to_np(sel(gx)), ex) < 1e-5
        assert err_over_rms(to_np(sel(ga)), ea) < 1e-5
