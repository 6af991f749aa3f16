/* Body of the C restatement of recurrent_gla_naive, instantiated for REAL = float and double by
 * gla_naive.c.  TEST INFRASTRUCTURE ONLY: nothing in the product links or loads this.
 *
 * Layout: log_fgate/value/key/query/out/dout are [B,T,H,D] row-major, hidden is [B,H,DK,DV].
 * One OpenMP task per (b,h) pair; inside, the literal T-step recurrence of gla.py:35-37 with the
 * state in REAL (the reference carries it in fp32, gla.py:44). */

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

/* forward: S_t = exp(g_t) * S_{t-1} + k_t v_t^T ; o_t = S_t^T q_t   (gla.py:35-37).
 * reverse != 0 scans t = T-1 .. 0 with outputs left at their own t (gla.py:45). */
int FN(gla_naive_fwd_)(int B, int T, int H, int DK, int DV, const REAL *h0, const REAL *g,
                       const REAL *v, const REAL *k, const REAL *q, int reverse, REAL *hT, REAL *out,
                       int nthreads)
{
    if (B <= 0 || T <= 0 || H <= 0 || DK <= 0 || DV <= 0) return -1;
    if (nthreads < 1) nthreads = 1;
    int fail = 0;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 1)
    for (int bh = 0; bh < B * H; ++bh) {
        int b = bh / H, h = bh % H;
        REAL *S = (REAL *)malloc(sizeof(REAL) * (size_t)DK * DV);
        if (!S) { fail = 1; continue; }
        memcpy(S, h0 + (size_t)bh * DK * DV, sizeof(REAL) * (size_t)DK * DV);
        for (int s = 0; s < T; ++s) {
            int t = reverse ? T - 1 - s : s;
            size_t ok = (((size_t)b * T + t) * H + h) * DK;
            size_t ov = (((size_t)b * T + t) * H + h) * DV;
            const REAL *gt = g + ok, *kt = k + ok, *qt = q + ok, *vt = v + ov;
            REAL *ot = out + ov;
            for (int j = 0; j < DV; ++j) ot[j] = 0;
            for (int i = 0; i < DK; ++i) {
                REAL f = EXP(gt[i]), ki = kt[i], qi = qt[i];
                REAL *Si = S + (size_t)i * DV;
                for (int j = 0; j < DV; ++j) {
                    REAL sij = f * Si[j] + ki * vt[j];
                    Si[j] = sij;
                    ot[j] += qi * sij;
                }
            }
        }
        memcpy(hT + (size_t)bh * DK * DV, S, sizeof(REAL) * (size_t)DK * DV);
        free(S);
    }
    return fail ? -2 : 0;
}

/* backward by the two sweeps of gla.py:297-359 and the identity of gla.py:263:
 *   sweep 1 (t up):   S_t as above,            dq_t = S_t do_t
 *   sweep 2 (t down): dS = dcarry + q_t do_t^T, dv_t = dS^T k_t, dk_t = dS v_t, dcarry = exp(g_t)*dS
 *   dg_t = sum_{s>=t}(dq_s*q_s - dk_s*k_s) + sum_v(dhT * hT)
 * Forward direction only (the reference's reverse flips the inputs around this, gla.py:421-438). */
int FN(gla_naive_bwd_)(int B, int T, int H, int DK, int DV, const REAL *h0, const REAL *g,
                       const REAL *v, const REAL *k, const REAL *q, const REAL *dhT, const REAL *dout,
                       REAL *dh0, REAL *dg, REAL *dv, REAL *dk, REAL *dq, REAL *hT, REAL *out,
                       int nthreads)
{
    if (B <= 0 || T <= 0 || H <= 0 || DK <= 0 || DV <= 0) return -1;
    if (nthreads < 1) nthreads = 1;
    int fail = 0;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 1)
    for (int bh = 0; bh < B * H; ++bh) {
        int b = bh / H, h = bh % H;
        size_t nS = (size_t)DK * DV;
        REAL *S = (REAL *)malloc(sizeof(REAL) * (nS + (size_t)2 * DK));
        if (!S) { fail = 1; continue; }
        REAL *fin = S + nS;      /* sum_v dhT*hT, [DK] */
        REAL *run = fin + DK;    /* running reverse cumsum, [DK] */
        memcpy(S, h0 + (size_t)bh * nS, sizeof(REAL) * nS);
        for (int t = 0; t < T; ++t) {
            size_t ok = (((size_t)b * T + t) * H + h) * DK;
            size_t ov = (((size_t)b * T + t) * H + h) * DV;
            const REAL *gt = g + ok, *kt = k + ok, *qt = q + ok, *vt = v + ov, *dot = dout + ov;
            REAL *ot = out + ov, *dqt = dq + ok;
            for (int j = 0; j < DV; ++j) ot[j] = 0;
            for (int i = 0; i < DK; ++i) {
                REAL f = EXP(gt[i]), ki = kt[i], qi = qt[i], acc = 0;
                REAL *Si = S + (size_t)i * DV;
                for (int j = 0; j < DV; ++j) {
                    REAL sij = f * Si[j] + ki * vt[j];
                    Si[j] = sij;
                    ot[j] += qi * sij;
                    acc += sij * dot[j];
                }
                dqt[i] = acc;
            }
        }
        memcpy(hT + (size_t)bh * nS, S, sizeof(REAL) * nS);
        const REAL *dhTb = dhT + (size_t)bh * nS;
        for (int i = 0; i < DK; ++i) {
            REAL acc = 0;
            for (int j = 0; j < DV; ++j) acc += dhTb[(size_t)i * DV + j] * S[(size_t)i * DV + j];
            fin[i] = acc;
            run[i] = 0;
        }
        memcpy(S, dhTb, sizeof(REAL) * nS);   /* S now holds dcarry */
        for (int t = T - 1; t >= 0; --t) {
            size_t ok = (((size_t)b * T + t) * H + h) * DK;
            size_t ov = (((size_t)b * T + t) * H + h) * DV;
            const REAL *gt = g + ok, *kt = k + ok, *qt = q + ok, *vt = v + ov, *dot = dout + ov;
            REAL *dvt = dv + ov, *dkt = dk + ok, *dgt = dg + ok;
            const REAL *dqt = dq + ok;
            for (int j = 0; j < DV; ++j) dvt[j] = 0;
            for (int i = 0; i < DK; ++i) {
                REAL f = EXP(gt[i]), ki = kt[i], qi = qt[i], acc = 0;
                REAL *Ci = S + (size_t)i * DV;
                for (int j = 0; j < DV; ++j) {
                    REAL d = Ci[j] + qi * dot[j];
                    dvt[j] += ki * d;
                    acc += d * vt[j];
                    Ci[j] = f * d;
                }
                dkt[i] = acc;
                run[i] += dqt[i] * qi - acc * ki;
                dgt[i] = run[i] + fin[i];
            }
        }
        memcpy(dh0 + (size_t)bh * nS, S, sizeof(REAL) * nS);
        free(S);
    }
    return fail ? -2 : 0;
}

#undef FN
#undef CAT
#undef CAT_
