"""CPU oracle for the Gated Linear Attention hot path.  TEST INFRASTRUCTURE ONLY.

This module is a checker: it may be imported by tests/, by __graft_entry__.smoke()
and by bench.py's cpu_baseline leg, and by nothing else.  The product path
(gla_jax_amd) never imports it and has no CPU fallback.

It restates, in NumPy, the algorithms of the reference (zhixuan-lin/gla-jax).
Each function cites the reference lines it follows.  The reference ships no
golden vectors and its only arithmetic dependency (jax 0.4.29 / jaxlib CUDA
wheels, README.md:20-22) is not present, so bit-level parity with the Pallas
kernels is "parity unpinned"; what IS pinned (tests/test_oracle.py):

  recurrent_gla_naive        closed forms: g==0 (causal linear attention),
                             k==0, T==1, D==1 scalar recurrence, f==0,
                             reverse == flip/flip
  recurrent_gla_naive_grad   torch.autograd (fp64) through an independent
                             torch restatement of the loop + central finite
                             differences
  cumsum / rnn_scan          np.cumsum, sequential loops, flips, associativity
  compute_score              brute-force A[i,j] over (i,j,d)
  chunk_gla_forward/backward equality with the naive recurrence and its
                             gradients, chunk-size invariance, concatenation
                             invariance

Conventions: arrays are [..., T, H, D] with any leading batch dims, hidden is
[..., H, DK, DV]; argument order is (hidden, log_fgate, value, key, query) as in
the reference (gla.py:26, 405, 657).
"""
from __future__ import annotations

import numpy as np

__all__ = [
    "bf16_round", "recurrent_gla_naive", "recurrent_gla_naive_grad", "cumsum", "rnn_scan",
    "compute_score", "compute_score_backward", "chunk_gla_forward", "chunk_gla_backward",
    "chunk_gla", "make_inputs",
]


# ----------------------------------------------------------------------------------------------
# helpers
# ----------------------------------------------------------------------------------------------
def bf16_round(x):
    """Round to bfloat16 (nearest even) and return the value widened back to float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    bias = ((u >> 16) & 1) + 0x7FFF
    u = ((u + bias) & 0xFFFF0000).astype(np.uint32)
    return u.view(np.float32).reshape(x.shape)


def _ident(x):
    return x


def log_sigmoid(x):
    x = np.asarray(x, dtype=np.float64)
    return -np.logaddexp(0.0, -x)


def make_inputs(B, T, H, D, gate_shift, seed=0, low_precision=True, batch_dims=True):
    """Seeded inputs in the shapes of BASELINE.json's configs: q,k,v,hidden_init ~ N(0,1),
    log_fgate = log_sigmoid(gate_shift + N(0,1)) in fp32.  Every tensor has its own stream
    (the reference's script reuses one PRNG key for all of them, gla.py:1386-1392, which makes
    value == key == query; BASELINE.json asks for independent draws).  When low_precision is set
    the q/k/v/hidden values are bf16-representable (stored as float32)."""
    def draw(i, shape):
        return np.random.default_rng(1000 * seed + i).standard_normal(shape, dtype=np.float32)
    lead = (B,) if batch_dims else ()
    h0 = draw(0, lead + (H, D, D))
    g = log_sigmoid(gate_shift + draw(1, lead + (T, H, D)).astype(np.float64)).astype(np.float32)
    v = draw(2, lead + (T, H, D))
    k = draw(3, lead + (T, H, D))
    q = draw(4, lead + (T, H, D))
    if low_precision:
        h0, v, k, q = (bf16_round(a) for a in (h0, v, k, q))
    return h0, g, v, k, q


# ----------------------------------------------------------------------------------------------
# the definition: recurrent_gla_naive (gla.py:26-47)
# ----------------------------------------------------------------------------------------------
def recurrent_gla_naive(hidden, log_fgate, value, key, query, reverse=False, dtype=np.float64):
    """S_t = exp(g_t)[:,None] * S_{t-1} + k_t v_t^T ; o_t = sum_k q_t[k] S_t[k,:]   (gla.py:35-37)

    The state is carried in `dtype` (the reference carries fp32, gla.py:44).  With reverse the scan
    runs from t=T-1 down to 0 and outputs stay at their own t (jax.lax.scan reverse, gla.py:45).
    Returns (hidden_final, out) both in `dtype` (the caller casts, gla.py:46)."""
    g = np.asarray(log_fgate, dtype=dtype)
    v = np.asarray(value, dtype=dtype)
    k = np.asarray(key, dtype=dtype)
    q = np.asarray(query, dtype=dtype)
    S = np.array(hidden, dtype=dtype, copy=True)
    T = g.shape[-3]
    out = np.empty(v.shape, dtype=dtype)
    f = np.exp(g)
    steps = range(T - 1, -1, -1) if reverse else range(T)
    for t in steps:
        S = f[..., t, :, :, None] * S + k[..., t, :, :, None] * v[..., t, :, None, :]
        out[..., t, :, :] = np.einsum("...hk,...hkv->...hv", q[..., t, :, :], S)
    return S, out


def recurrent_gla_naive_grad(hidden, log_fgate, value, key, query, dhidden_final, dout,
                             reverse=False, dtype=np.float64):
    """Gradients of recurrent_gla_naive by the two-sweep scheme of the reference's recurrent
    backward (gla.py:297-359): sweep 1 recomputes S_t and forms dq_t = S_t do_t; sweep 2 runs
    backwards with dS = dcarry + q_t do_t^T, dv_t = k_t^T dS, dk_t = dS v_t, dcarry = f_t * dS.
    d(log_fgate) uses the identity of gla.py:263:
        dg = revcumsum_t(dq*q - dk*k) + sum_v(dcarry_final * hidden_final).
    O(1) state memory, so it is usable at full benchmark shapes.
    Returns (dhidden, dlog_fgate, dvalue, dkey, dquery, hidden_final, out)."""
    g = np.asarray(log_fgate, dtype=dtype)
    v = np.asarray(value, dtype=dtype)
    k = np.asarray(key, dtype=dtype)
    q = np.asarray(query, dtype=dtype)
    do = np.asarray(dout, dtype=dtype)
    if reverse:  # gla.py:421-438: reverse == flip inputs, run forward in time, flip outputs
        fl = lambda a: a[..., ::-1, :, :]
        r = recurrent_gla_naive_grad(hidden, fl(g), fl(v), fl(k), fl(q), dhidden_final, fl(do),
                                     reverse=False, dtype=dtype)
        return (r[0], fl(r[1]), fl(r[2]), fl(r[3]), fl(r[4]), r[5], fl(r[6]))
    S = np.array(hidden, dtype=dtype, copy=True)
    T = g.shape[-3]
    f = np.exp(g)
    out = np.empty(v.shape, dtype=dtype)
    dq = np.empty(q.shape, dtype=dtype)
    for t in range(T):
        S = f[..., t, :, :, None] * S + k[..., t, :, :, None] * v[..., t, :, None, :]
        out[..., t, :, :] = np.einsum("...hk,...hkv->...hv", q[..., t, :, :], S)
        dq[..., t, :, :] = np.einsum("...hkv,...hv->...hk", S, do[..., t, :, :])
    hidden_final = S
    dcarry_final = np.asarray(dhidden_final, dtype=dtype)
    dcarry = dcarry_final.copy()
    dk = np.empty(k.shape, dtype=dtype)
    dv = np.empty(v.shape, dtype=dtype)
    for t in range(T - 1, -1, -1):
        dS = dcarry + q[..., t, :, :, None] * do[..., t, :, None, :]
        dv[..., t, :, :] = np.einsum("...hk,...hkv->...hv", k[..., t, :, :], dS)
        dk[..., t, :, :] = np.einsum("...hkv,...hv->...hk", dS, v[..., t, :, :])
        dcarry = f[..., t, :, :, None] * dS
    dlam = dq * q - dk * k
    dg = np.flip(np.cumsum(np.flip(dlam, axis=-3), axis=-3), axis=-3)
    dg = dg + (dcarry_final * hidden_final).sum(axis=-1)[..., None, :, :]
    return dcarry, dg, dv, dk, dq, hidden_final, out


# ----------------------------------------------------------------------------------------------
# the scans of ops.py
# ----------------------------------------------------------------------------------------------
def cumsum(src, axis, init=None, reverse=False, dtype=np.float64):
    """Inclusive cumulative sum along `axis` in `dtype`, plus `init` broadcast over that axis;
    with reverse the sum runs from the far end (ops.py:152-162: triton_scan(add) with init folded in
    afterwards, ops.py:91-103; blocking of ops.py:262-280 does not change the result)."""
    x = np.asarray(src, dtype=dtype)
    if reverse:
        x = np.flip(x, axis=axis)
    y = np.cumsum(x, axis=axis)
    if reverse:
        y = np.flip(y, axis=axis)
    if init is not None:
        y = y + np.expand_dims(np.asarray(init, dtype=dtype), axis)
    return y


def rnn_scan(log_fgate, kv, init_log_fgate=None, init_kv=None, reverse=False, dtype=np.float64):
    """Diagonal linear recurrence over the leading axis (ops.py:286-297, 299-334, 396-456):
        forward:  x_n = exp(a_n)[:,None] * x_{n-1} + b_n,   x_{-1} = init_kv
        reverse:  x_n = exp(a_n)[:,None] * x_{n+1} + b_n,   x_{N}  = init_kv
    Returns (cumulated a including init_log_fgate, x) like rnn_recursive."""
    a = np.asarray(log_fgate, dtype=dtype)
    b = np.asarray(kv, dtype=dtype)
    N = a.shape[0]
    ca = np.zeros_like(a[0]) if init_log_fgate is None else np.asarray(init_log_fgate, dtype=dtype)
    x = np.zeros_like(b[0]) if init_kv is None else np.asarray(init_kv, dtype=dtype)
    out_a = np.empty_like(a)
    out_x = np.empty_like(b)
    order = range(N - 1, -1, -1) if reverse else range(N)
    for n in order:
        ca = ca + a[n]
        x = np.exp(a[n])[:, None] * x + b[n]
        out_a[n] = ca
        out_x[n] = x
    return out_a, out_x


# ----------------------------------------------------------------------------------------------
# intra-chunk gated scores (gla.py:964-1029 forward, gla.py:1036-1189 backward)
# ----------------------------------------------------------------------------------------------
def _dyadic_blocks(start, end, out):
    """All (start, middle, end) triples of the dyadic recursion compute(start, end) of
    gla.py:985-996; the grouped levels 16/8/4/2 of gla.py:1000-1027 are the same triples with
    end-start < 32 (group g of size C: start+gC, anchor row start+gC+C/2-1)."""
    if end - start < 2:
        return
    middle = (start + end) // 2
    out.append((start, middle, end))
    _dyadic_blocks(start, middle, out)
    _dyadic_blocks(middle, end, out)


def compute_score(log_lambda, key, query, rnd=_ident, dtype=np.float64):
    """A[i,j] = sum_d q[i,d] k[j,d] exp(L[i,d]-L[j,d]) for j<i, A[i,i] = q_i.k_i, 0 above the
    diagonal, on one [L,D] block, evaluated the way the reference does: for every dyadic block the
    anchor is L[middle-1]; rows middle..end are scaled by exp(L-anchor) <= 1, rows start..middle by
    exp(anchor-L) <= 1, both rounded by `rnd` (the reference rounds to the input dtype,
    gla.py:991-992) before the dot."""
    lam = np.asarray(log_lambda, dtype=dtype)
    k = np.asarray(key, dtype=dtype)
    q = np.asarray(query, dtype=dtype)
    L = lam.shape[0]
    A = np.zeros((L, L), dtype=dtype)
    A[np.arange(L), np.arange(L)] = (q * k).sum(axis=-1)          # gla.py:983
    blocks = []
    _dyadic_blocks(0, L, blocks)
    for (s, m, e) in blocks:
        anchor = lam[m - 1]
        qw = rnd(q[m:e] * np.exp(lam[m:e] - anchor)).astype(dtype)
        kw = rnd(k[s:m] * np.exp(anchor - lam[s:m])).astype(dtype)
        A[m:e, s:m] = qw @ kw.T
    return A


def compute_score_backward(log_lambda, key, query, dscore, rnd=_ident, dtype=np.float64):
    """Cotangents of compute_score (gla.py:1061-1189): per dyadic block
    dqw = dA_blk kw, dq += dqw*wq, dL_q += dqw*qw ; dkw = dA_blk^T qw, dk += dkw*wk, dL_k -= dkw*kw;
    the anchor receives no gradient; the diagonal adds dA_ii*q_i to dk_i and dA_ii*k_i to dq_i
    (gla.py:1181-1184).  Returns (dlog_lambda, dkey, dquery)."""
    lam = np.asarray(log_lambda, dtype=dtype)
    k = np.asarray(key, dtype=dtype)
    q = np.asarray(query, dtype=dtype)
    dA = np.asarray(dscore, dtype=dtype)
    L = lam.shape[0]
    dlam = np.zeros_like(lam)
    dk = np.zeros_like(k)
    dq = np.zeros_like(q)
    blocks = []
    _dyadic_blocks(0, L, blocks)
    for (s, m, e) in blocks:
        anchor = lam[m - 1]
        wq = np.exp(lam[m:e] - anchor)
        wk = np.exp(anchor - lam[s:m])
        qw = rnd(q[m:e] * wq).astype(dtype)
        kw = rnd(k[s:m] * wk).astype(dtype)
        blk = dA[m:e, s:m]
        dqw = blk @ kw
        dkw = blk.T @ qw
        dq[m:e] += dqw * wq
        dk[s:m] += dkw * wk
        dlam[m:e] += dqw * qw
        dlam[s:m] -= dkw * kw
    d = dA[np.arange(L), np.arange(L)][:, None]
    dk += d * q
    dq += d * k
    return dlam, dk, dq


# ----------------------------------------------------------------------------------------------
# chunk_gla, per head on [N, C, D] (gla.py:483-550, 695-729, 792-855 / 552-625, 731-790, 857-960)
# ----------------------------------------------------------------------------------------------
def _intra_forward(lam, v, k, q, block_size_t, rnd, dtype):
    """compute_intra_contrib (gla.py:792-855): halve the chunk until it is <= block_size_t; the
    off-diagonal half x half block uses anchor = last row of the left half (gla.py:814-821), leaves
    use compute_score.  Returns (contrib[N,C,D], list of scores, deepest level first)."""
    scores = []

    def scan(lam, v, k, q):
        N, C, D = lam.shape
        if C <= block_size_t:
            sc = np.stack([compute_score(lam[n], k[n], q[n], rnd, dtype) for n in range(N)])
            sc = rnd(sc).astype(dtype)                            # scores stored in key dtype (gla.py:463,477)
            scores.append(sc)
            return rnd(sc @ v).astype(dtype)
        M = C // 2
        halves = [a.reshape(2 * N, M, D) for a in (lam, v, k, q)]
        inner = scan(*halves).reshape(N, C, D)
        anchor = lam[:, M - 1:M]
        qw = rnd(q[:, M:] * np.exp(lam[:, M:] - anchor)).astype(dtype)
        kw = rnd(k[:, :M] * np.exp(anchor - lam[:, :M])).astype(dtype)
        sc = rnd(qw @ np.swapaxes(kw, -1, -2)).astype(dtype)
        scores.append(sc)
        inner[:, M:] = rnd(inner[:, M:] + rnd(sc @ v[:, :M])).astype(dtype)
        return inner

    return scan(lam, v, k, q), scores


def _intra_backward(lam, v, k, q, dout, scores, block_size_t, rnd, dtype):
    """compute_intra_contrib_backward (gla.py:857-960).  Saved scores are reused (popped, outermost
    level first).  `rnd` marks what the reference stores in the input dtype: dvalue and dscore are plain
    matmuls of bf16 operands, whose result takes the operand dtype (gla.py:880-881, 926-927); dkey and
    dquery leave the score kernel and attention_backward in the key/query dtype (gla.py:1185-1186, 893, 900)
    and are summed in it (gla.py:953-955); d(log_lambda) and the products feeding it stay fp32
    (matmul_fp32, gla.py:892-901, 1073-1087).  Returns (dlam, dv, dk, dq)."""
    scores = list(scores)

    def rec(lam, v, k, q, do):
        N, C, D = lam.shape
        sc = scores.pop()
        if C <= block_size_t:
            dv = rnd(np.swapaxes(sc, -1, -2) @ do).astype(dtype)          # gla.py:926
            dsc = rnd(do @ np.swapaxes(v, -1, -2)).astype(dtype)          # gla.py:927
            outs = [compute_score_backward(lam[n], k[n], q[n], dsc[n], rnd, dtype) for n in range(N)]
            dlam = np.stack([o[0] for o in outs])
            dk = rnd(np.stack([o[1] for o in outs])).astype(dtype)        # gla.py:1185
            dq = rnd(np.stack([o[2] for o in outs])).astype(dtype)        # gla.py:1186
            return dlam, dv, dk, dq
        M = C // 2
        halves = [a.reshape(2 * N, M, D) for a in (lam, v, k, q, do)]
        dlam, dv, dk, dq = (a.reshape(N, C, D) for a in rec(*halves))
        # attention_backward, gla.py:878-906
        dv_i = rnd(np.swapaxes(sc, -1, -2) @ do[:, M:]).astype(dtype)
        dsc = rnd(do[:, M:] @ np.swapaxes(v[:, :M], -1, -2)).astype(dtype)
        anchor = lam[:, M - 1:M]
        wq = np.exp(lam[:, M:] - anchor)
        wk = np.exp(anchor - lam[:, :M])
        qw = rnd(q[:, M:] * wq).astype(dtype)
        kw = rnd(k[:, :M] * wk).astype(dtype)
        dqw = dsc @ kw
        dkw = np.swapaxes(dsc, -1, -2) @ qw
        dlam = dlam.copy(); dv = dv.copy(); dk = dk.copy(); dq = dq.copy()
        dq[:, M:] = rnd(dq[:, M:] + rnd(dqw * wq)).astype(dtype)         # gla.py:893, 954
        dk[:, :M] = rnd(dk[:, :M] + rnd(dkw * wk)).astype(dtype)         # gla.py:900, 955
        dlam[:, M:] += dqw * qw
        dlam[:, :M] -= dkw * kw
        dv[:, :M] = rnd(dv[:, :M] + dv_i).astype(dtype)                  # gla.py:953
        return dlam, dv, dk, dq

    return rec(lam, v, k, q, dout)


def _chunk_head_forward(h0, g, v, k, q, block_size_t, rnd, dtype):
    """chunk_gla_forward for one head, inputs [N,C,D] (gla.py:483-550)."""
    lam = cumsum(g, axis=-2, dtype=dtype)                         # gla.py:509
    lam_chunk = lam[:, -1, :]                                      # gla.py:512
    intra, scores = _intra_forward(lam, v, k, q, block_size_t, rnd, dtype)
    # compute_inter_contrib, gla.py:695-729
    kw = rnd(k * np.exp(lam_chunk[:, None, :] - lam)).astype(dtype)
    kv = rnd(np.swapaxes(kw, -1, -2) @ v).astype(dtype)
    _, state = rnn_scan(lam_chunk, kv, np.zeros_like(lam_chunk[0]), h0, dtype=dtype)
    state = rnd(state).astype(dtype)                               # gla.py:719
    allst = np.concatenate([np.asarray(h0, dtype=dtype)[None], state], axis=0)
    state, hidden_final = allst[:-1], allst[-1]
    qw = rnd(q * np.exp(lam)).astype(dtype)
    inter = rnd(qw @ state).astype(dtype)
    out = rnd(intra + inter).astype(dtype)
    return hidden_final, out, (scores, state)


def _chunk_head_backward(g, v, k, q, res, dhidden_final, dout, block_size_t, rnd, dtype):
    """chunk_gla_backward for one head (gla.py:552-625, 731-790).  `rnd` marks what the reference holds in
    the input dtype: dstate = Q~^T dO and dvalue = K~ dkv are plain matmuls of bf16 operands (gla.py:750,
    775), the reverse scan returns its states in the dtype of dstate (ops.py:326, 373-374), dquery is cast
    (gla.py:753); dkey of this path stays fp32 (gla.py:778), as does everything that feeds d(log_fgate)."""
    scores, state = res
    lam = cumsum(g, axis=-2, dtype=dtype)
    lam_chunk = lam[:, -1, :]
    dlam_i, dv_i, dk_i, dq_i = _intra_backward(lam, v, k, q, dout, scores, block_size_t, rnd, dtype)
    # compute_inter_contrib_backward, gla.py:731-790
    log_gamma = lam_chunk[:, None, :] - lam
    qw = rnd(q * np.exp(lam)).astype(dtype)
    dstate = rnd(np.swapaxes(qw, -1, -2) @ dout).astype(dtype)    # gla.py:750
    dqw = dout @ np.swapaxes(state, -1, -2)                       # gla.py:752
    dq_o = rnd(dqw * np.exp(lam)).astype(dtype)                   # gla.py:753
    dlam_q = dqw * qw
    _, dkv = rnn_scan(lam_chunk, dstate, np.zeros_like(lam_chunk[0]), dhidden_final,
                      reverse=True, dtype=dtype)                  # gla.py:759-765
    dkv = rnd(dkv).astype(dtype)                                   # ops.py:326, 373-374
    allst = np.concatenate([dkv, np.asarray(dhidden_final, dtype=dtype)[None]], axis=0)
    dh0, dkv = allst[0], allst[1:]                                 # gla.py:768-771
    kw = rnd(k * np.exp(log_gamma)).astype(dtype)
    dv_o = rnd(kw @ dkv).astype(dtype)                             # gla.py:775
    dkw = v @ np.swapaxes(dkv, -1, -2)
    dk_o = dkw * np.exp(log_gamma)
    dlam_k = -dkw * kw
    dlam_chunk = -dlam_k.sum(axis=1) + (state * np.exp(lam_chunk)[:, :, None] * dkv).sum(axis=-1)
    dlam = dlam_k + dlam_q + dlam_i                                # gla.py:786, 615
    dg = cumsum(dlam, axis=-2, init=dlam_chunk, reverse=True, dtype=dtype)   # gla.py:616-617
    return (dh0, dg, rnd(dv_o + dv_i).astype(dtype), dk_o + dk_i,
            rnd(dq_o + dq_i).astype(dtype))                        # gla.py:618-620


def _to_heads(x, chunk_size):
    """'(n c) h d -> h n c d' (gla.py:673-675)."""
    T, H, D = x.shape
    return np.ascontiguousarray(x.reshape(T // chunk_size, chunk_size, H, D).transpose(2, 0, 1, 3))


def _from_heads(x):
    """'h n c d -> (n c) h d' (gla.py:691)."""
    H, N, C, D = x.shape
    return np.ascontiguousarray(x.transpose(1, 2, 0, 3).reshape(N * C, H, D))


def chunk_gla_forward(hidden_init, log_fgate, value, key, query, chunk_size, block_size_t=64,
                      rnd=_ident, dtype=np.float64):
    """chunk_gla (gla.py:657-692) on unbatched [T,H,D] inputs.  Returns
    (hidden_final, out, residuals)."""
    assert chunk_size & (chunk_size - 1) == 0, "chunk length must be a power of 2 (gla.py:500)"
    g, v, k, q = (_to_heads(np.asarray(a, dtype=dtype), chunk_size)
                  for a in (log_fgate, value, key, query))
    H = g.shape[0]
    hf, out, res = [], [], []
    for h in range(H):
        a, b, c = _chunk_head_forward(np.asarray(hidden_init[h], dtype=dtype), g[h], v[h], k[h], q[h],
                                      block_size_t, rnd, dtype)
        hf.append(a); out.append(b); res.append(c)
    return np.stack(hf), _from_heads(np.stack(out)), res


def chunk_gla_backward(log_fgate, value, key, query, res, dhidden_final, dout, chunk_size,
                       block_size_t=64, rnd=_ident, dtype=np.float64):
    """custom_vjp backward of chunk_gla; returns (dhidden_init, dlog_fgate, dvalue, dkey, dquery)
    in argument order (gla.py:625)."""
    g, v, k, q, do = (_to_heads(np.asarray(a, dtype=dtype), chunk_size)
                      for a in (log_fgate, value, key, query, dout))
    H = g.shape[0]
    outs = [_chunk_head_backward(g[h], v[h], k[h], q[h], res[h],
                                 np.asarray(dhidden_final[h], dtype=dtype), do[h],
                                 block_size_t, rnd, dtype) for h in range(H)]
    dh0 = np.stack([o[0] for o in outs])
    dg, dv, dk, dq = (_from_heads(np.stack([o[i] for o in outs])) for i in (1, 2, 3, 4))
    return dh0, dg, dv, dk, dq


def chunk_gla(hidden_init, log_fgate, value, key, query, chunk_size, **kw):
    hf, out, _ = chunk_gla_forward(hidden_init, log_fgate, value, key, query, chunk_size, **kw)
    return hf, out
