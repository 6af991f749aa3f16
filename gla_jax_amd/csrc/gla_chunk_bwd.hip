// chunk_gla backward, gradient kernel: one workgroup per chunk produces dq, dk, dv and dlog_fgate
// for its C tokens from the chunk-start state S_n and the gradient dS' of the chunk-end state
// (gla.py:552-625 with compute_intra_contrib_backward gla.py:857-960, compute_score backward
// gla.py:1036-1189 and compute_inter_contrib_backward gla.py:731-790).
//
// Same secondary chunking as the forward (16-token sub-blocks, one per wave; l_i = gate prefix in
// the sub-block, tau_m = sub-block total, r_m = e^{tau_m}):
//   row-owner role (query rows i of sub-block I):
//     dq_i = e^{l_i} * H_I + (sub-block part),   H_I = (((dO_i S^T) r_0 + G_0) r_1 + G_1) ... r_{I-1} + G_{I-1}
//     with G_J = dA_IJ (k e^{tau_J - l})_J  -- a Horner chain over J, one 16x16xD MFMA per link, the
//     accumulator scaled in registers between links; the state term rides the same chain.
//   column-owner role (key rows j of sub-block J):
//     dv_j = sum_{I>=J} A_IJ^T dO_I + K~_j dS',
//     dk_j = e^{tau_J - l_j} * ((((V_j dS'^T) r_{NB-1} + H_{NB-1}) r_{NB-2} + ...) r_{J+1} + H_{J+1}) + (sub-block part)
//     with H_I = dA_IJ^T (q e^{l})_I -- the mirrored chain, carrying the dS' term.
//   inside a sub-block: the dyadic levels 16/8/4/2 of the reference; per level the mixed tile X (q rows
//     scaled by e^{prefix}, k rows by e^{suffix}) gets dX = (M + M^T) X with M the masked dA block.
//   d(log-gate cumsum) per token is q*dq - k*dk (the anchors cancel, gla.py:1078-1087); dlog_fgate is
//     its reverse cumsum inside the chunk plus the chunk-level term of gla.py:782.
// All sums that feed dlog_fgate stay in fp32 registers (gla.py:1073-1087 asks for fp32 there).
//
// Register plan.  Everything indexed by (token, feature) is needed only 32 features at a time, while the
// 16x16 score blocks do not depend on the feature at all.  So each role first computes and caches
// its score blocks (packed MFMA operands, 2 registers each), then walks the head dimension in slices
// of 32 features: levels, chain, epilogue, store.  What has to survive from the first role to the
// second (the sub-block part of dk, the query-side gate gradient) is parked in the token's rows of
// outputs that are written last, and read back (L2 hits) by the same lane.
#include "gla_chunk_common.hpp"
#include "gla_chunk_kernels.hpp"

namespace gla {

__device__ __forceinline__ bf16x8 join4(bf16x4 lo, bf16x4 hi)
{
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ __forceinline__ f32x8 join4(f32x4 lo, f32x4 hi)
{
    f32x8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r.v[e] = lo[e]; r.v[4 + e] = hi[e]; }
    return r;
}

template <typename T, int C, int D>
__global__ __launch_bounds__(C * 4) void chunk_grad_kernel(
    const float *__restrict__ g, const T *__restrict__ v, const T *__restrict__ k,
    const T *__restrict__ q, const T *__restrict__ dout, const T *__restrict__ states,
    const T *__restrict__ dstates, const float *__restrict__ decay, float *__restrict__ dg,
    T *__restrict__ dv, T *__restrict__ dk, T *__restrict__ dq, int T_len, int H)
{
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);   // row stride of the per-wave slice scratch
    constexpr int TR = C > D ? C : D;              // rows of one LDS tile
    constexpr int SR = (D * D / 8) / (C * 4);      // 16-byte pieces of a D x D state per thread
    static_assert(SR * C * 4 * 8 == D * D, "state staging assumes whole pieces per thread");
    typedef typename FragTypes<T>::d8 D8;
    typedef typename FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *tile0 = reinterpret_cast<T *>(smem);        // value, later dout                  [token][dv]
    T *tile1 = tile0 + TR * LS;                    // k e^{tau_J - l_j}                  [token][dk]
    T *tile2 = tile1 + TR * LS;                    // S_n, later dS'                     [dv][dk]
    T *tile3 = tile2 + TR * LS;                    // q e^{l_i}                          [token][dk]
    T *xs = tile3 + TR * LS;                       // [NB][16][XS] per-wave scratch
    float *rtab = reinterpret_cast<float *>(xs + NB * 16 * XS);   // [NB][D] e^{tau_m}
    float *dltab = rtab + NB * D;                  // [NB][D] sub-block sums of the gate-cumsum gradient
    float *lbar = dltab + NB * D;                  // [D] chunk-level gate gradient
    float *ttab = lbar + D;                        // [NB][D] tau_m (log2 units)

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: scalar branches on it
    const int r = lane & 15, c = lane >> 4;
    // heads vary fastest over the grid: workgroups that run together touch the same DRAM pages of the
    // [B, T, H, D] arrays (a token's H rows are contiguous)
    const int h = blockIdx.x % H, n = blockIdx.x / H, b = blockIdx.y;
    const int N = T_len / C;
    const int64_t tok = (int64_t)b * T_len + (int64_t)n * C + 16 * w + r;
    const int64_t rowoff = (tok * H + h) * D;
    const int64_t bhn = ((int64_t)b * H + h) * N + n;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const TrLane<T> Lx = make_tr_lane<T>(XS);
    const int wrow = 16 * w * LS + L.nat;          // this lane's row of a [token][feature] tile
    T *xw = xs + w * 16 * XS;                      // [16][XS]: one 32-feature slice of the wave's rows

    // Piece i of a D x D state that this thread moves between global memory and its LDS tile.
    const int st_row = threadIdx.x / (D / 8), st_c8 = (threadIdx.x % (D / 8)) * 8;
    constexpr int kStRows = C * 4 / (D / 8);       // rows covered by one round of the workgroup

    D8 dof[KS];
    f32x4 Aown = {0.f, 0.f, 0.f, 0.f};   // scores A[i = 4c+e][j = r] of the own sub-block
    T4 symb[4];                          // per level: masked (dA + dA^T) of the own sub-block, MFMA operand
                                         // (one anchor: [0] = dA^T below the diagonal, [1] = dA below it)
    bool one_anchor;                     // wave-uniform: the sub-block's gates are mild enough for ONE anchor
    float dd = 0.f;                      // dA_ii of this lane's row
    {
        float p[NV], s[NV];
        D8 vf[KS], qf[KS], kf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = 32 * ks + 8 * c;
            f32x8 gg = ld8(g + rowoff + d0);
#pragma unroll
            for (int e = 0; e < 8; ++e) p[8 * ks + e] = gg.v[e] * kLog2e;
            qf[ks] = ld8(q + rowoff + d0);
            kf[ks] = ld8(k + rowoff + d0);
            vf[ks] = ld8(v + rowoff + d0);
            dof[ks] = ld8(dout + rowoff + d0);
            st8(tile0 + wrow + 32 * ks, vf[ks]);
        }
        // the chunk-start state is requested now and lands in its tile just before the first barrier
        D8 sreg[SR];
        {
            const T *sp = states + bhn * D * D;
#pragma unroll
            for (int i = 0; i < SR; ++i) sreg[i] = ld8(sp + (st_row + i * kStRows) * D + st_c8);
        }
        if (threadIdx.x < D) lbar[threadIdx.x] = 0.f;

        // dAn[e] = dA[i = 4c+e][j = r],  dAt[e] = dA[i = r][j = 4c+e]   (dA = dO V^T), own sub-block
        f32x4 dAn = {0.f, 0.f, 0.f, 0.f}, dAt = {0.f, 0.f, 0.f, 0.f};
        float dot = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            dAn = mma_d(dof[ks], vf[ks], dAn);
            dAt = mma_d(vf[ks], dof[ks], dAt);
            float a[8], bq[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) dot += a[e] * bq[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
        dd = reduce_over_cgroups(dd);
        dot = reduce_over_cgroups(dot);
#pragma unroll
        for (int e = 0; e < 4; ++e) Aown[e] = (4 * c + e == r) ? dot : 0.f;   // A_ii = q_i.k_i (gla.py:983)

        // p = l_i (inclusive prefix over the 16 rows, log2 units), s = tau - l_i; the totals go through
        // the wave's row of ttab (same-wave LDS accesses execute in order) and stay there.
#pragma unroll
        for (int i = 0; i < NV; ++i) p[i] = prefix_sum_rows(p[i]);
        if (r == 15) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) st8(ttab + w * D + 32 * ks + 8 * c, pack8<float>(p + 8 * ks));
        }
        asm volatile("" ::: "memory");
        {
            float span = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 tau = ld8(ttab + w * D + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    s[8 * ks + e] = tau.v[e] - p[8 * ks + e];
                    span = fmaxf(span, fmaxf(fabsf(p[8 * ks + e]), fabsf(s[8 * ks + e])));
                }
            }
            one_anchor = wave_all_below(span, kOneAnchorSpan);
        }

        // Harder gates: pass 1 over the dyadic levels, full head dimension: the mixed tile X of every level
        // -> the level's score blocks (they contract over all features), and the gate prefix/suffix sums.
        auto level_scores = [&](auto hc, auto lc) {
            constexpr int h_ = decltype(hc)::value, L_ = decltype(lc)::value;
            const bool upper = (r & h_) != 0;
            f32x4 G = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                float a[8], bq[8], x[8];
                unpack8(qf[ks], a);
                unpack8(kf[ks], bq);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    x[e] = (upper ? a[e] : bq[e]) * fast_exp2(upper ? p[8 * ks + e] : s[8 * ks + e]);
                D8 X = pack8<T>(x);
                G = mma_d(X, X, G);
            }
            f32x4 sym;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int o = 4 * c + e;                       // the other row
                const bool same = (o ^ r) < 2 * h_;
                const bool o_up = (o & h_) != 0;
                Aown[e] += (same && o_up && !upper) ? G[e] : 0.f;
                sym[e] = (same && upper && !o_up) ? dAt[e] : ((same && o_up && !upper) ? dAn[e] : 0.f);
            }
            symb[L_] = pack4<T>(sym);
            hier_step<h_>(p, s, upper);
            __builtin_amdgcn_sched_barrier(0);
        };
        if (!one_anchor) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 gg = ld8(refetch(g + rowoff) + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) { p[8 * ks + e] = gg.v[e] * kLog2e; s[8 * ks + e] = 0.f; }
            }
            level_scores(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
            level_scores(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
            level_scores(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
            level_scores(std::integral_constant<int, 8>{}, std::integral_constant<int, 3>{});
        }

        // p = l_i, s = tau - l_i (log2 units): table of e^{tau}, rescaled key and query tiles
        if (r == 0) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 t;
#pragma unroll
                for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(p[8 * ks + e] + s[8 * ks + e]);
                st8(rtab + w * D + 32 * ks + 8 * c, t);
            }
        }
        // One anchor (the end of the sub-block): A_ij = [q_i e^{l_i - tau}] . [k_j e^{tau - l_j}]; the key
        // factor is the operand of the other sub-blocks as well.
        f32x4 G = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], bq[8], qo[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                qo[e] = a[e] * fast_exp2(-s[8 * ks + e]);
                a[e] *= fast_exp2(p[8 * ks + e]);
                bq[e] *= fast_exp2(s[8 * ks + e]);
            }
            const D8 kh = pack8<T>(bq);
            st8(tile3 + wrow + 32 * ks, pack8<T>(a));
            st8(tile1 + wrow + 32 * ks, kh);
            if (one_anchor) G = mma_d(pack8<T>(qo), kh, G);
        }
        if (one_anchor) {
            f32x4 lowT, low;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                Aown[e] += (4 * c + e > r) ? G[e] : 0.f;
                lowT[e] = (4 * c + e < r) ? dAt[e] : 0.f;
                low[e] = (4 * c + e > r) ? dAn[e] : 0.f;
            }
            symb[0] = pack4<T>(lowT);
            symb[1] = pack4<T>(low);
        }
#pragma unroll
        for (int i = 0; i < SR; ++i) st8(tile2 + (st_row + i * kStRows) * LS + st_c8, sreg[i]);
    }
    __syncthreads();

    // ---- row-owner role ----------------------------------------------------------------------------
    // Per-row inputs of a slice are fetched one slice ahead (L2 hits, but still a microsecond away).
    f32x8 gN = ld8(refetch(g + rowoff) + 8 * c);
    D8 qN = ld8(refetch(q + rowoff) + 8 * c), kN = ld8(refetch(k + rowoff) + 8 * c);
    // score blocks dA^T of the earlier sub-blocks: dAT_J[j][i] = v_j . dO_i  (J < w)
    T4 dATc[NB];
#pragma unroll
    for (int J = 0; J < NB - 1; ++J) {
        dATc[J] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
        if (J < w) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) a = mma_d(ld8(tile0 + L.nat + 16 * J * LS + 32 * ks), dof[ks], a);
            dATc[J] = pack4<T>(a);
        }
    }
    dATc[NB - 1] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
    __builtin_amdgcn_sched_barrier(0);

    // Gradient w.r.t. the gate cumsum L of a row, "dL".  Every term dA_ij * q~_i * k~_j enters row i with +
    // and row j with -; both copies are formed from the SAME rounded operands (the values the MFMAs
    // consume), so they cancel exactly in the reverse cumsum (gla.py:1077-1087 asks for this).
    //
    // The head dimension is walked in slices of 32 features by a real (not unrolled) loop, so that only
    // one slice's temporaries are live.  What has to survive from this loop to the column-owner loop
    // is parked in the token's rows of the outputs that are written last: the sub-block part of dk in the
    // dlog_fgate row (fp32), the query-side dL in the dk and dv rows (together D fp32 values).
#pragma unroll 1
    for (int ks = 0; ks < KS; ++ks) {
        const int fo = 32 * ks;
        float p8[8], s8[8], a[8], bq[8], dq8[8], dk8[8], dl8[8];
        {
#pragma unroll
            for (int e = 0; e < 8; ++e) { p8[e] = gN.v[e] * kLog2e; s8[e] = 0.f; }
            unpack8(qN, a);
            unpack8(kN, bq);
            if (ks + 1 < KS) {
                gN = ld8(refetch(g + rowoff) + fo + 32 + 8 * c);
                qN = ld8(refetch(q + rowoff) + fo + 32 + 8 * c);
                kN = ld8(refetch(k + rowoff) + fo + 32 + 8 * c);
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            dq8[e] = dd * bq[e];         // diagonal term dA_ii q_i k_i: no gate gradient (gla.py:1181-1185)
            dk8[e] = dd * a[e];
            dl8[e] = 0.f;
        }
        // A level of the dyadic recursion restricted to the slice: rebuilds the slice of X, dX = (M + M^T) X
        // by one MFMA per 16 features, and adds its share to the sub-block parts of dq / dk / dL.  The
        // per-wave scratch is written and read by the same wave only; LDS executes one wave's accesses
        // in order, so a compiler-level fence is all the ordering that is needed.
        auto slice_level = [&](auto hc, auto lc) {
            constexpr int h_ = decltype(hc)::value, L_ = decltype(lc)::value;
            const bool upper = (r & h_) != 0;
            float fac[8], x[8], xr[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                fac[e] = fast_exp2(upper ? p8[e] : s8[e]);
                x[e] = (upper ? a[e] : bq[e]) * fac[e];
            }
            D8 X = pack8<T>(x);
            unpack8(X, xr);
            st8(xw + Lx.nat, X);
            asm volatile("" ::: "memory");
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                f32x4 dx = {0.f, 0.f, 0.f, 0.f};
                dx = mma_t(lds_tr4(xw + Lx.k4 + 4 * tt, XS), symb[L_], dx);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float z = dx[e] * fac[4 * tt + e];
                    const float y = dx[e] * xr[4 * tt + e];
                    dq8[4 * tt + e] += upper ? z : 0.f;
                    dk8[4 * tt + e] += upper ? 0.f : z;
                    dl8[4 * tt + e] += upper ? y : -y;
                }
            }
            asm volatile("" ::: "memory");
            hier_step<h_>(p8, s8, upper);
        };
        if (one_anchor) {
            // the own sub-block is one more link on either side: dq~ = dA k~, dk~ = dA^T q~ (below the diagonal)
            f32x8 tau = ld8(ttab + w * D + fo + 8 * c);
            float fq[8], fk[8], x[8], xr[8], kr[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                p8[e] = prefix_sum_rows(p8[e]);
                s8[e] = tau.v[e] - p8[e];
                fq[e] = fast_exp2(-s8[e]);
                fk[e] = fast_exp2(s8[e]);
                x[e] = a[e] * fq[e];
                kr[e] = bq[e] * fk[e];
            }
            D8 X = pack8<T>(x);
            unpack8(X, xr);
            unpack8(pack8<T>(kr), kr);
            st8(xw + Lx.nat, X);
            asm volatile("" ::: "memory");
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
                f32x4 gq = mma_t(lds_tr4(tile1 + L.k4 + fo + 4 * tt + 16 * w * LS, LS), symb[0], z4);
                f32x4 hk = mma_t(lds_tr4(xw + Lx.k4 + 4 * tt, XS), symb[1], z4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dq8[4 * tt + e] += gq[e] * fq[4 * tt + e];
                    dk8[4 * tt + e] += hk[e] * fk[4 * tt + e];
                    dl8[4 * tt + e] += gq[e] * xr[4 * tt + e] - hk[e] * kr[4 * tt + e];
                }
            }
            asm volatile("" ::: "memory");
        } else {
            slice_level(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
            slice_level(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
            slice_level(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
            slice_level(std::integral_constant<int, 8>{}, std::integral_constant<int, 3>{});
        }
        {
            f32x8 pk;
#pragma unroll
            for (int e = 0; e < 8; ++e) pk.v[e] = dk8[e];
            st8(dg + rowoff + fo + 8 * c, pk);               // parked until the dk epilogue
        }

        // dq chain of the slice: state term first, then the earlier sub-blocks in ascending order
        f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const T *bp = tile2 + L.k8 + fo + 4 * tt + 32 * k2 * LS;
                acc[tt] = mma_d(join4(lds_tr4(bp, LS), lds_tr4(bp + 4 * LS, LS)), dof[k2], acc[tt]);
            }
        }
#pragma unroll
        for (int J = 0; J < NB - 1; ++J) {
            if (J < w) {
                f32x8 rr = ld8(rtab + J * D + fo + 8 * c);
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[tt][e] *= rr.v[4 * tt + e];
                    acc[tt] = mma_t(lds_tr4(tile1 + L.k4 + fo + 4 * tt + 16 * J * LS, LS), dATc[J], acc[tt]);
                }
            }
        }
        {
            float o[8], qe[8], qr[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) qe[e] = a[e] * fast_exp2(p8[e]);
            unpack8(pack8<T>(qe), qr);                   // q e^{l} as the MFMAs of the key side see it
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float hacc = acc[e >> 2][e & 3];
                o[e] = fast_exp2(p8[e]) * hacc + dq8[e];
                const float dl = dl8[e] + qr[e] * hacc;
                if (e < 4) lo[e] = dl; else hi[e - 4] = dl;
            }
            st8(dq + rowoff + fo + 8 * c, pack8<T>(o));
            // query-side dL, parked: 8 fp32 = the slice's 8 elements of the dk row + of the dv row
            if constexpr (sizeof(T) == 2) {
                *reinterpret_cast<f32x4 *>(dk + rowoff + fo + 8 * c) = lo;
                *reinterpret_cast<f32x4 *>(dv + rowoff + fo + 8 * c) = hi;
            } else {
                f32x8 both = join4(lo, hi);
                st8(reinterpret_cast<float *>(dk + rowoff + fo + 8 * c), both);
            }
        }
    }
    // What the column-owner loop needs per slice (the parked values and the gates), again one slice ahead.
    f32x8 gN2, dlN, pkN;
    auto fetch_parked = [&](int fo) {
        gN2 = ld8(refetch(g + rowoff) + fo + 8 * c);
        pkN = ld8(refetch(dg + rowoff) + fo + 8 * c);
        if constexpr (sizeof(T) == 2) {
            dlN = join4(*reinterpret_cast<const f32x4 *>(refetch(dk + rowoff) + fo + 8 * c),
                        *reinterpret_cast<const f32x4 *>(refetch(dv + rowoff) + fo + 8 * c));
        } else {
            dlN = ld8(reinterpret_cast<const float *>(refetch(dk + rowoff) + fo + 8 * c));
        }
    };
    fetch_parked(0);
    D8 dsreg[SR];                                  // dS' of the chunk, requested before the barrier
    {
        const T *dsp = dstates + bhn * D * D;
#pragma unroll
        for (int i = 0; i < SR; ++i) dsreg[i] = ld8(dsp + (st_row + i * kStRows) * D + st_c8);
    }
    const f32x8 dec = ld8(decay + bhn * D + st_c8);
    __syncthreads();

    // ---- second set of tiles: dO, dS'^T; chunk-level term sum_v S*dS' ------------------------------
    {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) st8(tile0 + wrow + 32 * ks, dof[ks]);
        float part[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) part[e] = 0.f;
#pragma unroll
        for (int i = 0; i < SR; ++i) {
            T *cell = tile2 + (st_row + i * kStRows) * LS + st_c8;
            float a[8], bq[8];
            unpack8(ld8(cell), a);
            unpack8(dsreg[i], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) part[e] += a[e] * bq[e];
            st8(cell, dsreg[i]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) atomicAdd(lbar + st_c8 + e, part[e] * dec.v[e]);
    }
    __syncthreads();

    // ---- column-owner role -------------------------------------------------------------------------
    // score blocks of the later sub-blocks: A_IJ (needs the key side walked up by r_I) and dA_IJ
    T4 Ac[NB], dAc[NB];
    D8 Kt[KS], vf[KS];                   // k e^{L_end - L_j} as MFMA operand; value rows
    {
        float kch[NV];
        const T *vp = refetch(v + rowoff);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vf[ks] = ld8(vp + 32 * ks + 8 * c);
            unpack8(ld8(tile1 + wrow + 32 * ks), kch + 8 * ks);
        }
#pragma unroll
        for (int I = 1; I < NB; ++I) {
            Ac[I] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
            dAc[I] = Ac[I];
            if (I > w) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    a = mma_d(ld8(tile3 + L.nat + 16 * I * LS + 32 * ks), pack8<T>(kch + 8 * ks), a);
                    da = mma_d(ld8(tile0 + L.nat + 16 * I * LS + 32 * ks), vf[ks], da);
                    f32x8 rr = ld8(rtab + I * D + 32 * ks + 8 * c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) kch[8 * ks + e] *= rr.v[e];
                }
                Ac[I] = pack4<T>(a);
                dAc[I] = pack4<T>(da);
            }
        }
        Ac[0] = pack4<T>(Aown);
        dAc[0] = Ac[0];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) Kt[ks] = pack8<T>(kch + 8 * ks);
    }

#pragma unroll 1
    for (int ks = 0; ks < KS; ++ks) {
        const int fo = 32 * ks;
        // what the row-owner loop parked for this slice (read before the rows are overwritten below)
        const f32x8 dlq = dlN, parked = pkN, gg = gN2;
        if (ks + 1 < KS) fetch_parked(fo + 32);
        // dv slice
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    acc[tt] = mma_d(ld8(tile2 + L.own + (fo + 4 * tt) * LS + 32 * k2), Kt[k2], acc[tt]);
            }
#pragma unroll
            for (int I = 0; I < NB; ++I) {
                if (I >= w) {
                    const T4 b4 = I == w ? Ac[0] : Ac[I];
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt)
                        acc[tt] = mma_t(lds_tr4(tile0 + L.k4 + fo + 4 * tt + 16 * I * LS, LS), b4, acc[tt]);
                }
            }
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = acc[e >> 2][e & 3];
            st8(dv + rowoff + fo + 8 * c, pack8<T>(o));
        }
        // dk slice
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    const T *bp = tile2 + L.k8 + fo + 4 * tt + 32 * k2 * LS;
                    acc[tt] = mma_d(join4(lds_tr4(bp, LS), lds_tr4(bp + 4 * LS, LS)), vf[k2], acc[tt]);
                }
            }
            float kr[8];
            unpack8(ld8(tile1 + wrow + fo), kr);           // k e^{tau-l} as the MFMAs saw it
            // chunk-level gate gradient, key part: sum_j (k e^{L_end - L_j}) * (V dS'^T)_j, with
            // k e^{L_end - L_j} = (k e^{tau - l_j}) * prod_{m > w} r_m
            {
                float sig[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) sig[e] = 1.f;
                for (int m = w + 1; m < NB; ++m) {
                    f32x8 rr = ld8(rtab + m * D + fo + 8 * c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) sig[e] *= rr.v[e];
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float z = reduce_over_rows(kr[e] * acc[e >> 2][e & 3]) * sig[e];
                    if (r == 0) atomicAdd(lbar + fo + 8 * c + e, z);
                }
            }
#pragma unroll
            for (int I = NB - 1; I >= 1; --I) {
                if (I > w) {
                    f32x8 rr = ld8(rtab + I * D + fo + 8 * c);
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[tt][e] *= rr.v[4 * tt + e];
                        acc[tt] = mma_t(lds_tr4(tile3 + L.k4 + fo + 4 * tt + 16 * I * LS, LS), dAc[I], acc[tt]);
                    }
                }
            }
            // epilogue: e^{tau - l} of the slice is rebuilt from the gates
            float s8[8], o[8];
            {
                f32x8 tau = ld8(ttab + w * D + fo + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) s8[e] = tau.v[e] - prefix_sum_rows(gg.v[e] * kLog2e);
            }
            f32x8 sfx;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float hacc = acc[e >> 2][e & 3];
                o[e] = fast_exp2(s8[e]) * hacc + parked.v[e];
                // dL of the row, then its reverse cumsum inside the sub-block (gla.py:616-617)
                sfx.v[e] = suffix_sum_rows(dlq.v[e] - kr[e] * hacc);
            }
            st8(dk + rowoff + fo + 8 * c, pack8<T>(o));
            st8(dg + rowoff + fo + 8 * c, sfx);               // parked until the other sub-blocks' totals are known
            if (r == 0) st8(dltab + w * D + fo + 8 * c, sfx);
        }
    }
    f32x8 own[KS];                                 // the row's suffix sums, parked by the loop above
    {
        const float *dgp = refetch(dg + rowoff);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) own[ks] = ld8(dgp + 32 * ks + 8 * c);
    }
    __syncthreads();

    // ---- dlog_fgate = reverse cumsum over the whole chunk + the chunk-level term (gla.py:782) ------------
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * c;
        f32x8 o = ld8(lbar + d0);
#pragma unroll
        for (int e = 0; e < 8; ++e) o.v[e] += own[ks].v[e];
        for (int m = w + 1; m < NB; ++m) {
            f32x8 t = ld8(dltab + m * D + d0);
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] += t.v[e];
        }
        st8(dg + rowoff + d0, o);
    }
}

template <typename T, int C, int D>
int launch_chunk_grad(hipStream_t st, int B, int T_len, int H, const float *g, const void *v, const void *k,
                      const void *q, const void *dout, const void *states, const void *dstates,
                      const float *decay, float *dg, void *dv, void *dk, void *dq)
{
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    constexpr int TR = C > D ? C : D, NB = C / 16;
    const size_t lds = ((size_t)4 * TR * LS + (size_t)NB * 16 * XS) * sizeof(T) +
                       (size_t)(3 * NB + 1) * D * sizeof(float);
    auto kern = chunk_grad_kernel<T, C, D>;
    if (int e = allow_lds((const void *)kern, lds)) return e;
    dim3 grid(T_len / C * H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)v, (const T *)k, (const T *)q,
                       (const T *)dout, (const T *)states, (const T *)dstates, decay, dg, (T *)dv, (T *)dk,
                       (T *)dq, T_len, H);
    return launch_status();
}

#define GLA_INST_GRAD(T, C, D)                                                                           \
    template int launch_chunk_grad<T, C, D>(hipStream_t, int, int, int, const float *, const void *,     \
                                            const void *, const void *, const void *, const void *,     \
                                            const void *, const float *, float *, void *, void *, void *);
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_GRAD)

}  // namespace gla
