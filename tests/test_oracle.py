"""Pins the CPU oracle (oracle/gla_oracle.py, oracle/libgla_naive.so) by things the mathematics
fixes, none of which re-types the oracle's own formula:

  * closed forms of the recurrence (no decay -> causal linear attention via a tril matmul, zero keys,
    total decay, T=1, D=1 scalar loop, reverse = flip/flip),
  * torch.autograd in fp64 through an independently written torch loop, and central differences,
  * np.cumsum / explicit sums for the two scans, brute-force triple loops for the gated scores,
  * naive == chunked, chunk-size invariance, concatenation invariance.
The reference (zhixuan-lin/gla-jax) holds no golden vectors or tests of its own."""
import numpy as np
import pytest
import torch

from oracle import gla_oracle as O
from oracle import naive_c


def rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


def inputs(T=24, H=2, DK=5, DV=5, seed=0, shift=1.0):
    h0 = rand((H, DK, DV), seed)
    g = O.log_sigmoid(shift + rand((T, H, DK), seed + 1))
    v = rand((T, H, DV), seed + 2)
    k = rand((T, H, DK), seed + 3)
    q = rand((T, H, DK), seed + 4)
    return h0, g, v, k, q


# ---------------------------------------------------------------- naive: closed forms
def test_naive_no_decay_is_causal_linear_attention():
    h0, g, v, k, q = inputs()
    g = np.zeros_like(g)
    hT, out = O.recurrent_gla_naive(h0, g, v, k, q)
    T = g.shape[0]
    for h in range(g.shape[1]):
        A = np.tril(q[:, h] @ k[:, h].T)
        exp_out = A @ v[:, h] + q[:, h] @ h0[h]
        np.testing.assert_allclose(out[:, h], exp_out, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(hT[h], h0[h] + k[:, h].T @ v[:, h], rtol=1e-12, atol=1e-12)
    assert out.shape == (T, 2, 5)


def test_naive_zero_keys_only_decays_the_initial_state():
    h0, g, v, k, q = inputs()
    k = np.zeros_like(k)
    hT, out = O.recurrent_gla_naive(h0, g, v, k, q)
    lam = np.cumsum(g, axis=0)
    exp_out = np.einsum("thk,hkv->thv", q * np.exp(lam), h0)
    np.testing.assert_allclose(out, exp_out, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(hT, np.exp(lam[-1])[:, :, None] * h0, rtol=1e-12)


def test_naive_total_decay_keeps_only_the_current_token():
    h0, g, v, k, q = inputs()
    g = np.full_like(g, -1e4)           # exp -> 0 exactly
    _, out = O.recurrent_gla_naive(h0, g, v, k, q)
    exp_out = (q * k).sum(-1, keepdims=True) * v
    np.testing.assert_allclose(out, exp_out, rtol=1e-12, atol=1e-12)


def test_naive_single_step_and_scalar_recurrence():
    h0, g, v, k, q = inputs(T=1)
    hT, out = O.recurrent_gla_naive(h0, g, v, k, q)
    S = np.exp(g[0])[:, :, None] * h0 + k[0][:, :, None] * v[0][:, None, :]
    np.testing.assert_allclose(hT, S, rtol=1e-13)
    np.testing.assert_allclose(out[0], np.einsum("hk,hkv->hv", q[0], S), rtol=1e-12)
    # D = 1: a scalar recurrence written as a python loop
    h0, g, v, k, q = inputs(T=17, H=1, DK=1, DV=1, seed=5)
    _, out = O.recurrent_gla_naive(h0, g, v, k, q)
    s = float(h0[0, 0, 0])
    for t in range(17):
        s = np.exp(g[t, 0, 0]) * s + k[t, 0, 0] * v[t, 0, 0]
        assert abs(out[t, 0, 0] - q[t, 0, 0] * s) < 1e-12


def test_naive_reverse_is_flip_scan_flip():
    h0, g, v, k, q = inputs(seed=7)
    hT_r, out_r = O.recurrent_gla_naive(h0, g, v, k, q, reverse=True)
    fl = lambda a: a[::-1]
    hT_f, out_f = O.recurrent_gla_naive(h0, fl(g), fl(v), fl(k), fl(q))
    np.testing.assert_allclose(hT_r, hT_f, rtol=1e-13)
    np.testing.assert_allclose(out_r, fl(out_f), rtol=1e-13)


def test_naive_batch_dims_are_independent():
    parts = [inputs(seed=10 * b) for b in range(3)]
    stacked = [np.stack([p[i] for p in parts]) for i in range(5)]
    hT, out = O.recurrent_gla_naive(*stacked)
    for b, p in enumerate(parts):
        hb, ob = O.recurrent_gla_naive(*p)
        np.testing.assert_allclose(hT[b], hb, rtol=1e-13)
        np.testing.assert_allclose(out[b], ob, rtol=1e-13)


# ---------------------------------------------------------------- naive: gradients
def torch_loop(h0, g, v, k, q):
    """Independent torch restatement (per-step einsum on [H,..]) for autograd."""
    S = h0
    outs = []
    for t in range(g.shape[0]):
        S = torch.exp(g[t]).unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        outs.append((q[t].unsqueeze(-1) * S).sum(-2))
    return S, torch.stack(outs)


def autograd_reference(h0, g, v, k, q, dhT, dout):
    ts = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (h0, g, v, k, q)]
    hT, out = torch_loop(*ts)
    loss = (hT * torch.tensor(dhT)).sum() + (out * torch.tensor(dout)).sum()
    grads = torch.autograd.grad(loss, ts)
    return [x.numpy() for x in grads], hT.detach().numpy(), out.detach().numpy()


@pytest.mark.parametrize("reverse", [False, True])
def test_naive_grad_matches_autograd(reverse):
    h0, g, v, k, q = inputs(T=19, H=2, DK=4, DV=6, seed=3)
    dhT, dout = rand(h0.shape, 50), rand(v.shape, 51)
    got = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout, reverse=reverse)
    fl = (lambda a: a[::-1].copy()) if reverse else (lambda a: a)
    (dh0, dg, dv, dk, dq), hT, out = autograd_reference(h0, fl(g), fl(v), fl(k), fl(q), dhT, fl(dout))
    for a, b in zip(got, (dh0, fl(dg), fl(dv), fl(dk), fl(dq), hT, fl(out))):
        np.testing.assert_allclose(a, b, rtol=1e-10, atol=1e-11)


def test_naive_grad_matches_central_differences():
    h0, g, v, k, q = inputs(T=6, H=1, DK=3, DV=2, seed=11)
    dhT, dout = rand(h0.shape, 60), rand(v.shape, 61)
    grads = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)[:5]
    args = [h0, g, v, k, q]

    def loss(a):
        hT, out = O.recurrent_gla_naive(*a)
        return (hT * dhT).sum() + (out * dout).sum()

    eps = 1e-6
    for i in range(5):
        num = np.zeros_like(args[i])
        it = np.nditer(args[i], flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            ap = [a.copy() for a in args]; am = [a.copy() for a in args]
            ap[i][idx] += eps; am[i][idx] -= eps
            num[idx] = (loss(ap) - loss(am)) / (2 * eps)
        np.testing.assert_allclose(grads[i], num, rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------- scans
def test_cumsum_against_numpy_and_flips():
    x = rand((3, 16, 7), 1)
    init = rand((3, 7), 2)
    np.testing.assert_allclose(O.cumsum(x, 1), np.cumsum(x, 1), rtol=1e-14)
    np.testing.assert_allclose(O.cumsum(x, 1, init=init), np.cumsum(x, 1) + init[:, None], rtol=1e-14)
    rev = O.cumsum(x, 1, init=init, reverse=True)
    for t in range(16):
        np.testing.assert_allclose(rev[:, t], x[:, t:].sum(1) + init, rtol=1e-12, atol=1e-12)


def test_rnn_scan_closed_form_and_associativity():
    N, K, V = 9, 4, 3
    a = -np.abs(rand((N, K), 3)); b = rand((N, K, V), 4)
    ia = -np.abs(rand((K,), 5)); ib = rand((K, V), 6)
    ca, x = O.rnn_scan(a, b, ia, ib)
    cum = np.cumsum(a, 0)
    for n in range(N):
        exp_x = np.exp(cum[n])[:, None] * ib
        for m in range(n + 1):
            exp_x = exp_x + np.exp(cum[n] - cum[m])[:, None] * b[m]
        np.testing.assert_allclose(x[n], exp_x, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(ca[n], ia + cum[n], rtol=1e-13)
    # reverse: x_n = e^{a_n} x_{n+1} + b_n with x_N = init
    _, xr = O.rnn_scan(a, b, ia, ib, reverse=True)
    _, xf = O.rnn_scan(a[::-1], b[::-1], ia, ib)
    np.testing.assert_allclose(xr, xf[::-1], rtol=1e-13)
    # the combine op (A_i,b_i)o(A_j,b_j) = (A_i+A_j, e^{A_j} b_i + b_j) is associative (ops.py:286-297)
    op = lambda p, r: (p[0] + r[0], np.exp(r[0])[:, None] * p[1] + r[1])
    e = [(a[i], b[i]) for i in range(3)]
    l = op(op(e[0], e[1]), e[2]); r = op(e[0], op(e[1], e[2]))
    np.testing.assert_allclose(l[1], r[1], rtol=1e-13)


# ---------------------------------------------------------------- gated scores
def brute_scores(lam, k, q):
    L, D = lam.shape
    A = np.zeros((L, L))
    for i in range(L):
        for j in range(i + 1):
            A[i, j] = sum(q[i, d] * k[j, d] * np.exp(lam[i, d] - lam[j, d]) for d in range(D))
    return A


@pytest.mark.parametrize("L", [2, 8, 32, 64])
def test_compute_score_is_the_brute_force_sum(L):
    D = 3
    lam = np.cumsum(O.log_sigmoid(rand((L, D), 8)), 0)
    k, q = rand((L, D), 9), rand((L, D), 10)
    np.testing.assert_allclose(O.compute_score(lam, k, q), brute_scores(lam, k, q), rtol=1e-11, atol=1e-12)


def test_compute_score_backward_matches_autograd_of_the_brute_form():
    L, D = 16, 4
    lam = np.cumsum(O.log_sigmoid(rand((L, D), 12)), 0)
    k, q, dA = rand((L, D), 13), rand((L, D), 14), rand((L, L), 15)
    tl, tk, tq = (torch.tensor(a, requires_grad=True) for a in (lam, k, q))
    W = torch.exp(tl[:, None, :] - tl[None, :, :])
    A = torch.tril((tq[:, None, :] * tk[None, :, :] * W).sum(-1))
    gl, gk, gq = torch.autograd.grad((A * torch.tensor(dA)).sum(), (tl, tk, tq))
    dl, dk, dq = O.compute_score_backward(lam, k, q, dA)
    np.testing.assert_allclose(dl, gl.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dk, gk.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dq, gq.numpy(), rtol=1e-10, atol=1e-11)
    # every within-block anchor cancels: the gradient wrt log_lambda sums to 0 over rows
    np.testing.assert_allclose(dl.sum(0), 0, atol=1e-10)


# ---------------------------------------------------------------- chunked == naive
@pytest.mark.parametrize("C,bt", [(8, 4), (16, 16), (32, 8), (64, 64)])
def test_chunk_forward_equals_naive_for_every_chunk_size(C, bt):
    h0, g, v, k, q = inputs(T=64, H=2, DK=6, DV=6, seed=21)
    hT, out = O.recurrent_gla_naive(h0, g, v, k, q)
    hc, oc, _ = O.chunk_gla_forward(h0, g, v, k, q, C, block_size_t=bt)
    np.testing.assert_allclose(oc, out, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(hc, hT, rtol=1e-9, atol=1e-10)


def test_chunk_concatenation_invariance():
    h0, g, v, k, q = inputs(T=64, H=1, DK=4, DV=4, seed=22)
    hT, out = O.chunk_gla(h0, g, v, k, q, 16)
    h1, o1 = O.chunk_gla(h0, g[:32], v[:32], k[:32], q[:32], 16)
    h2, o2 = O.chunk_gla(h1, g[32:], v[32:], k[32:], q[32:], 16)
    np.testing.assert_allclose(np.concatenate([o1, o2]), out, rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(h2, hT, rtol=1e-10, atol=1e-11)


@pytest.mark.parametrize("C,bt", [(16, 4), (32, 32)])
def test_chunk_backward_equals_naive_gradients(C, bt):
    h0, g, v, k, q = inputs(T=64, H=2, DK=5, DV=5, seed=23)
    dhT, dout = rand(h0.shape, 70), rand(v.shape, 71)
    ref = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)[:5]
    _, _, res = O.chunk_gla_forward(h0, g, v, k, q, C, block_size_t=bt)
    got = O.chunk_gla_backward(g, v, k, q, res, dhT, dout, C, block_size_t=bt)
    for a, b in zip(got, ref):
        np.testing.assert_allclose(a, b, rtol=1e-8, atol=1e-9)


def test_chunk_with_bf16_rounding_points_of_the_reference():
    # configs[0] shape (B1,T512,H2,D64,C64) with every bf16 rounding point of the reference switched
    # on (rescaled q/k, scores, kv, chunk states, intra, inter and their sum).  The relative L2 error
    # stays ~1e-2, but the max-abs error reaches ~3e-2 of the output RMS: the reference's own
    # rounding scheme does not meet the 2e-2 max-abs bound that the HIP kernels are held to, which
    # is why those keep fp32 accumulators and round operands only.
    h0, g, v, k, q = O.make_inputs(1, 512, 2, 64, 5.0, seed=1, batch_dims=False)
    hT, out = O.recurrent_gla_naive(h0, g, v, k, q)
    hc, oc, _ = O.chunk_gla_forward(h0, g, v, k, q, 64, rnd=O.bf16_round)
    rms = np.sqrt((out ** 2).mean())
    assert np.abs(oc - out).max() / rms < 6e-2
    assert np.linalg.norm(oc - out) / np.linalg.norm(out) < 1e-2
    assert np.abs(hc - hT).max() / np.sqrt((hT ** 2).mean()) < 4e-2


def test_reference_rounding_points_gradients():
    """What the reference's own bf16 rounding points (rescaled q/k, stored scores, bf16 chunk states)
    cost in the gradients, on strong-decay gates: the plain max|err|/RMS of d(log_fgate) is already
    above 2e-2 while the relative L2 error stays small.  This is the yardstick for the tolerance
    model of tests/util.py::assert_close."""
    h0, g, v, k, q = O.make_inputs(1, 256, 2, 64, 0.0, seed=3, batch_dims=False)
    rng = np.random.default_rng(9)
    dhT = O.bf16_round(rng.standard_normal(h0.shape, dtype=np.float32))
    dout = O.bf16_round(rng.standard_normal(v.shape, dtype=np.float32))
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)
    _, _, res = O.chunk_gla_forward(h0, g, v, k, q, 64, rnd=O.bf16_round)
    got = O.chunk_gla_backward(g, v, k, q, res, dhT, dout, 64, rnd=O.bf16_round)
    raw = [np.abs(a - b).max() / np.sqrt((b ** 2).mean()) for a, b in zip(got, exp[:5])]
    l2 = [np.linalg.norm(a - b) / np.linalg.norm(b) for a, b in zip(got, exp[:5])]
    assert max(l2) < 1e-2
    assert 2e-2 < raw[1] < 8e-2          # d(log_fgate): 3.8e-2 with these seeds
    assert max(raw) < 8e-2


def test_bf16_round_is_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.140625, 1e-3], dtype=np.float32)
    r = O.bf16_round(x)
    t = torch.tensor(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(r, t)
    big = np.random.default_rng(0).standard_normal(10000).astype(np.float32)
    np.testing.assert_array_equal(O.bf16_round(big), torch.tensor(big).bfloat16().float().numpy())


# ---------------------------------------------------------------- C restatement
@pytest.mark.parametrize("dt,tol", [(np.float64, 1e-11), (np.float32, 2e-4)])
def test_c_naive_matches_numpy_oracle(dt, tol):
    B, T, H, D = 2, 48, 3, 8
    h0, g, v, k, q = O.make_inputs(B, T, H, D, 2.0, seed=3)
    dhT, dout = rand(h0.shape, 80), rand(v.shape, 81)
    for rev in (False, True):
        hT, out = naive_c.naive_fwd(h0, g, v, k, q, reverse=rev, dtype=dt, nthreads=2)
        eh, eo = O.recurrent_gla_naive(h0, g, v, k, q, reverse=rev)
        np.testing.assert_allclose(out, eo, rtol=tol, atol=tol)
        np.testing.assert_allclose(hT, eh, rtol=tol, atol=tol)
    got = naive_c.naive_bwd(h0, g, v, k, q, dhT, dout, dtype=dt, nthreads=3)
    exp = O.recurrent_gla_naive_grad(h0, g, v, k, q, dhT, dout)
    for a, b in zip(got, exp):
        scale = np.abs(b).max()
        np.testing.assert_allclose(a, b, rtol=tol, atol=tol * scale)
