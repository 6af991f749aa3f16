"""Arrays past 2^31 elements (and 2^32 bytes): every offset the kernels form must be 64-bit.

No CPU restatement finishes at these sizes, so the check is a size-independent property: sequences are
independent of each other, hence the LAST batch entry of a large call (the one whose rows lie past element
2^31) must come out bit for bit as it does when it is the only entry of a small call; the small call's
own correctness is what the parity tests establish.  The scans are compared with torch's float64 cumsum and a closed form as well."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _need_gib(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * 2**30:
        pytest.skip(f"needs {gib} GiB of free device memory, {free / 2**30:.0f} GiB available")


def _inputs(B, T, H, D, shift, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    rn = lambda *s, dt=torch.bfloat16: torch.randn(*s, device="cuda", dtype=torch.float32, generator=gen).to(dt)
    h0 = rn(B, H, D, D)
    g = torch.nn.functional.logsigmoid(rn(B, T, H, D, dt=torch.float32) + shift)
    v, k, q = rn(B, T, H, D), rn(B, T, H, D), rn(B, T, H, D)
    return [h0, g, v, k, q]


def _fwd_bwd(fn, args, seed):
    args = [a.requires_grad_(True) for a in args]
    hT, out = fn(*args)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    dhT = torch.randn(hT.shape, device="cuda", generator=gen).to(hT.dtype)
    dout = torch.randn(out.shape, device="cuda", generator=gen).to(out.dtype)
    grads = torch.autograd.grad((hT, out), args, grad_outputs=(dhT, dout))
    return (hT.detach(), out.detach()) + tuple(grads), (dhT, dout)


def _last_entry_alone(fn, args, cots, b):
    args = [a.detach()[b:b + 1].clone().requires_grad_(True) for a in args]
    hT, out = fn(*args)
    grads = torch.autograd.grad((hT, out), args, grad_outputs=(cots[0][b:b + 1].clone(), cots[1][b:b + 1].clone()))
    return (hT.detach(), out.detach()) + tuple(grads)


NAMES = ("hidden_final", "out", "dhidden_init", "dlog_fgate", "dvalue", "dkey", "dquery")


def test_chunk_gla_past_2_31_elements():
    from gla_jax_amd import chunk_gla
    _need_gib(170)
    B, T, H, D = 5, 65536, 64, 128
    assert B * T * H * D > 2**31 and (B - 1) * T * H * D >= 2**31
    fn = lambda *a: chunk_gla(*a, 128)
    args = _inputs(B, T, H, D, 4.0, seed=1)
    big, cots = _fwd_bwd(fn, args, seed=2)
    for b in (B - 1, 0):
        small = _last_entry_alone(fn, args, cots, b)
        for name, x, y in zip(NAMES, big, small):
            assert torch.isfinite(y.float()).all(), name
            assert torch.equal(x[b:b + 1], y), f"{name}: batch entry {b} of {B} differs from the same entry run alone"


def test_recurrent_gla_past_2_31_elements():
    from gla_jax_amd import recurrent_gla
    _need_gib(110)
    B, T, H, D = 5, 32768, 256, 64
    assert (B - 1) * T * H * D >= 2**31
    args = _inputs(B, T, H, D, 3.0, seed=3)
    big, cots = _fwd_bwd(recurrent_gla, args, seed=4)
    for b in (B - 1, 0):
        small = _last_entry_alone(recurrent_gla, args, cots, b)
        for name, x, y in zip(NAMES, big, small):
            assert torch.isfinite(y.float()).all(), name
            assert torch.equal(x[b:b + 1], y), f"{name}: batch entry {b} of {B} differs from the same entry run alone"


@pytest.mark.parametrize("reverse", [False, True])
def test_scans_past_2_31_elements(reverse):
    from gla_jax_amd import cumsum_recursive, rnn_recursive
    _need_gib(60)
    gen = torch.Generator(device="cuda").manual_seed(5)
    # cumsum over the T axis of [B, T, H, D]: the last batch entry starts at element 2^31
    B, T, H, D = 5, 4096, 1024, 128
    x = torch.randn(B, T, H, D, device="cuda", generator=gen)
    y = cumsum_recursive(x, 1, reverse=reverse)
    for b in (B - 1, 0):
        xb = x[b]
        assert torch.equal(y[b], cumsum_recursive(xb.clone(), 0, reverse=reverse))
        xd = xb.double()
        ref = xd.flip(0).cumsum(0).flip(0) if reverse else xd.cumsum(0)
        # float32 running sums of 4096 unit normals reach ~200: a few float32 ulps of that
        torch.testing.assert_close(y[b].double(), ref, rtol=0, atol=1e-3)
        del xd, ref
    del x, y
    torch.cuda.empty_cache()
    # the chunk-state recurrence over N chunks of [B, N, K, V]
    Bn, N, K, V = 5, 2048, 512, 512
    a = -torch.rand(Bn, N, K, device="cuda", generator=gen)
    kv = torch.randn(Bn, N, K, V, device="cuda", generator=gen)
    ca, xs = rnn_recursive(a, kv, reverse=reverse)
    for b in (Bn - 1, 0):
        ca1, xs1 = rnn_recursive(a[b].clone(), kv[b].clone(), reverse=reverse)
        assert torch.equal(ca[b], ca1) and torch.equal(xs[b], xs1)
        # the state after the last step of the scan, by the closed form sum_n exp(sum of the later gates) * kv_n
        ab = a[b].double()
        later = (ab.flip(0).cumsum(0).flip(0) - ab) if not reverse else (ab.cumsum(0) - ab)
        last = (later.exp()[:, :, None] * kv[b, :, :, :8].double()).sum(0)
        got = xs[b, 0 if reverse else N - 1, :, :8].double()
        torch.testing.assert_close(got, last, rtol=1e-4, atol=1e-3)
