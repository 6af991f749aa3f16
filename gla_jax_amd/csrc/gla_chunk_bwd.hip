// chunk_gla backward, gradient kernel: one workgroup per chunk produces dq, dk, dv and dlog_fgate
// for its C tokens from the chunk-start state S_n and the gradient dS' of the chunk-end state
// (gla.py:552-625 with compute_intra_contrib_backward gla.py:857-960, compute_score backward
// gla.py:1036-1189 and compute_inter_contrib_backward gla.py:731-790).
//
// Same secondary chunking as the forward (16-token sub-blocks, one per wave; l_i = gate prefix in
// the sub-block, tau_m = sub-block total, r_m = e^{tau_m}).  A wave plays two roles for ITS 16 tokens:
//   row owner (query rows i of sub-block I):
//     dq_i = e^{l_i} * H_I + (sub-block part),   H_I = (((dO_i S^T) r_0 + G_0) r_1 + G_1) ... r_{I-1} + G_{I-1}
//     with G_J = dA_IJ (k e^{tau_J - l})_J  -- a Horner chain over J, one 16x16xD MFMA per link, the
//     accumulator scaled in registers between links; the state term rides the same chain.
//   column owner (key rows j of sub-block J):
//     dv_j = sum_{I>=J} A_IJ^T dO_I + K~_j dS',
//     dk_j = e^{tau_J - l_j} * ((((V_j dS'^T) r_{NB-1} + H_{NB-1}) r_{NB-2} + ...) r_{J+1} + H_{J+1}) + (sub-block part)
//     with H_I = dA_IJ^T (q e^{l})_I -- the mirrored chain, carrying the dS' term.
//   inside a sub-block: ONE anchor when the gates are mild (the own sub-block is then one more link of
//     either chain), else the dyadic levels 16/8/4/2 of the reference: per level the mixed tile X (q rows
//     scaled by e^{prefix}, k rows by e^{suffix}) gets dX = (M + M^T) X with M the masked dA block.
//   d(log-gate cumsum) per token is q*dq - k*dk (the anchors cancel, gla.py:1078-1087); dlog_fgate is
//     its reverse cumsum inside the chunk plus the chunk-level term of gla.py:782.
// All sums that feed dlog_fgate stay in fp32 registers (gla.py:1073-1087 asks for fp32 there).
//
// Memory plan.  The kernel is bound by HBM traffic, so every input is read once (the gates and q, k a
// second time, see below) and every output written once.  The 16x16 score blocks do not depend on the
// feature: both roles compute and cache them first (packed MFMA operands, 2 registers each).  Then the
// head dimension is walked in slices of 32 features by a rolled loop in which a wave finishes dq, dk, dv
// and the gate gradient of its rows for that slice, so nothing has to be parked between the roles.  The
// state operands of a slice (32 rows of S_n [dk][dv], dS' [dk][dv] and dS' [dv][dk]) are staged in
// the LDS tile that held the values, fetched one slice ahead; the per-row inputs of a slice (gates, q, k)
// are fetched one slice ahead as well.
#include "gla_subblock.hpp"
#include "gla_chunk_kernels.hpp"

namespace gla {

// WIDE: dv, dk and dq are float arrays (the sums of two such runs are rounded once: head dimension 256,
// gla_split.hip).
template <typename T, int C, int D, int DM, bool WIDE>
__global__ __launch_bounds__(C * 4) void chunk_grad_kernel(
    const float *__restrict__ g, const T *__restrict__ v, const T *__restrict__ k,
    const T *__restrict__ q, const T *__restrict__ dout, const T *__restrict__ statesN,
    const T *__restrict__ dstatesT, const T *__restrict__ dstatesN, float *__restrict__ dg,
    std::conditional_t<WIDE, float, T> *__restrict__ dv, std::conditional_t<WIDE, float, T> *__restrict__ dk,
    std::conditional_t<WIDE, float, T> *__restrict__ dq, int T_len, int H)
{
    typedef std::conditional_t<WIDE, float, T> TG;      // element type of dv, dk, dq
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);   // row stride of the per-wave slice scratch
    constexpr int VR = C > 96 ? C : 96;            // the value tile is recycled for 3 x 32 staged state rows
    typedef typename FragTypes<T>::d8 D8;
    typedef typename FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *tV = reinterpret_cast<T *>(smem);           // value, later the staged state rows [token][dv]
    T *tO = tV + VR * LS;                          // dout                               [token][dv]
    T *tK = tO + C * LS;                           // k e^{tau_J - l_j}                  [token][dk]
    T *tQ = tK + C * LS;                           // q e^{l_i}                          [token][dk]
    T *xs = tQ + C * LS;                           // [NB][16][XS] per-wave scratch
    float *rtab = reinterpret_cast<float *>(xs + NB * 16 * XS);   // [NB][D] e^{tau_m}
    float *dltab = rtab + NB * D;                  // [NB][D] sub-block sums of the gate-cumsum gradient
    float *ttab = dltab + NB * D;                  // [NB][D] tau_m (log2 units)
    float *lbar = ttab + NB * D;                   // [D] chunk-level gate gradient, the part that comes from S_n
    float *lbtab = lbar + D;                       // [NB][32] ... and per sub-block the part of its rows, one slice

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: scalar branches on it
    const int r = lane & 15, c = lane >> 4;
    // heads vary fastest over the grid: workgroups that run together touch the same DRAM pages of the
    // [B, T, H, D] arrays (a token's H rows are contiguous)
    const int h = blockIdx.x % H, n = blockIdx.x / H, b = blockIdx.y;
    const int N = T_len / C;
    const int64_t tok = (int64_t)b * T_len + (int64_t)n * C + 16 * w + r;
    const int64_t rowoff = (tok * H + h) * DM;     // DM features per row in memory (DM < D: see RowMap)
    const int64_t bhn = ((int64_t)b * H + h) * N + n;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const TrLane<T> Lx = make_tr_lane<T>(XS);
    const int wrow = 16 * w * LS + L.nat;          // this lane's row of a [token][feature] tile
    T *xw = xs + w * 16 * XS;                      // [16][XS]: one 32-feature slice of the wave's rows
    // a second slice scratch per wave, [16][XS2] (remainders of the own sub-block's operands, bf16 only): in the
    // rows of the value tile that the staged state rows leave free when the chunk has more than 96 tokens,
    // behind the tables otherwise
    constexpr int XS2 = 32;
    constexpr bool kSpareRows = (C - 96) * LS >= NB * 16 * XS2;
    T *xw2 = (kSpareRows ? tV + 96 * LS : reinterpret_cast<T *>(lbtab + NB * 32)) + w * 16 * XS2;
    const TrLane<T> Lx2 = make_tr_lane<T>(XS2);

    // ---- staging of the state operands -----------------------------------------------------------------
    // A slice needs rows 32*slice .. +31 of S_n [dk][dv], dS' [dk][dv] and dS' [dv][dk]: 3 x 32 rows of
    // D elements.  They go through registers: requested a slice ahead, written to LDS between two barriers.
    // 16-bit data: S_n and dS' are single arrays of 32 x 32 tiles (state_offset).  Their 32 rows [dk][all dv] are
    // staged as rows; the third operand, 32 rows of dS'^T [dv][all dk], is the slab [all dk][32 dv] of the same array,
    // read as it lies (whole tiles) and transposed on its way into LDS.  fp32 data: dS' comes in both orientations,
    // row-major.
    T *sS = tV, *sDn = tV + 32 * LS, *sDt = tV + 64 * LS;
    constexpr bool kTiled = sizeof(T) == 2;
    constexpr int kPieces = 32 * D / 8;                       // 8-element pieces of one staged operand
    constexpr int kPer = (kPieces + C * 4 - 1) / (C * 4);     // pieces per thread
    D8 pfS[kPer], pfDn[kPer], pfDt[kPer];
    f32x8 gN;                                                 // per-row inputs of the next slice
    D8 qN, kN;
    auto stage_fetch = [&](int slice) {
        // the residual holds N + 1 states per (b,h): slot n is the state before chunk n, slot N the final one
        const T *Sn = statesN + (bhn + ((int64_t)b * H + h)) * D * D;
        const T *dSn = dstatesN + bhn * D * D, *dSt = dstatesT + bhn * D * D;
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int idx = threadIdx.x + u * C * 4;
            if (kPieces % (C * 4) == 0 || idx < kPieces) {
                const int off = (32 * slice + idx / (D / 8)) * D + (idx % (D / 8)) * 8;
                const int toff = state_offset<T, D>(32 * slice + idx / (D / 8), (idx % (D / 8)) * 8);
                pfS[u] = ld8_once(Sn + toff);
                if constexpr (kTiled) {
                    pfDn[u] = ld8(dSn + toff);    // read again by the workgroup as part of the slabs of other slices
                    pfDt[u] = ld8(dSn + (((idx >> 7) * (D / 32) + slice) << 10) + (idx & 127) * 8);   // tiles (i, slice)
                } else {
                    pfDn[u] = ld8_once(dSn + off);
                    pfDt[u] = ld8_once(dSt + off);
                }
            }
        }
    };
    auto row_fetch = [&](int slice) {
        gN = ld8_row<D, DM>(refetch(g + rowoff) + 32 * slice, c);
        qN = ld8_row<D, DM>(refetch(q + rowoff) + 32 * slice, c);
        kN = ld8_row<D, DM>(refetch(k + rowoff) + 32 * slice, c);
    };
    auto stage_store = [&](int slice) {
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int idx = threadIdx.x + u * C * 4;
            if (kPieces % (C * 4) == 0 || idx < kPieces) {
                const int row = idx / (D / 8), c8 = (idx % (D / 8)) * 8;
                st8(sS + row * LS + c8, pfS[u]);
                st8(sDn + row * LS + c8, pfDn[u]);
                if constexpr (kTiled) {
                    // the piece holds 8 value features of ONE key feature: it goes to 8 rows of the staged [dv][dk]
                    // operand, two bytes each (8 KB per slice and workgroup: the transposition costs next to nothing
                    // here, and the products keep the form and the registers they had)
                    const int dkk = 32 * (idx >> 7) + ((idx & 127) >> 2), dvv = 8 * (idx & 3);
#pragma unroll
                    for (int e = 0; e < 8; ++e) sDt[(dvv + e) * LS + dkk] = pfDt[u][e];
                } else {
                    st8(sDt + row * LS + c8, pfDt[u]);
                }
                // chunk-level gate gradient (gla.py:782), first term: e^{L_end} sum_v S_n * dS' per key feature.
                // (The sum of both terms is sum_v dS' * S_{n+1}; formed that way from the stored S_{n+1} it carries
                // the rounding of a whole state instead of a decayed one, which cost two sweep cases their bound.)
                // The D/8 threads that hold one row are neighbours in a wave.
                float x[8], y[8], part = 0.f;
                unpack8(pfS[u], x);
                unpack8(pfDn[u], y);
#pragma unroll
                for (int e = 0; e < 8; ++e) part += x[e] * y[e];
                static_assert(D / 8 >= 4, "at least a quad of threads holds one staged row");
                part += dpp_f32<kDppQuadXor1>(part);
                part += dpp_f32<kDppQuadXor2>(part);
                if constexpr (D / 8 >= 8) part += dpp_f32<kDppRowHalfMirror>(part);
                if constexpr (D / 8 >= 16) part += dpp_f32<kDppRowMirror>(part);
                if constexpr (D / 8 == 32) part += shfl_xor_f32(part, 16);   // a row spans two 16-lane groups
                if (c8 == 0) {
                    float lend = 0.f;                            // L_end of the feature, log2 units
#pragma unroll
                    for (int m = 0; m < NB; ++m) lend += ttab[m * D + 32 * slice + row];
                    lbar[32 * slice + row] = part * fast_exp2(lend);
                }
            }
        }
    };

    f32x4 Aown = {0.f, 0.f, 0.f, 0.f};   // scores A[i = 4c+e][j = r] of the own sub-block
    T4 symb[4];                          // per level: masked (dA + dA^T) of the own sub-block, MFMA operand
                                         // (one anchor: [0] = dA^T below the diagonal, [1] = dA below it)
    bool one_anchor;                     // wave-uniform: the sub-block's gates are mild enough for ONE anchor
    float dd = 0.f;                      // dA_ii of this lane's row
    D8 vf[KS];                           // this lane's value row (B operand of the dS' product)
    {
        // Requests go out in the order the results are needed: gates (prefix sums), q and k (rescaled
        // tiles, scores), then values and dout (their tiles, dA); memory returns them in that order, so the
        // first steps run while the rest is still on its way.
        float p[NV], s[NV];
        D8 qf[KS], kf[KS], dof[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 gg = ld8_row<D, DM>(g + rowoff + 32 * ks, c);
#pragma unroll
            for (int e = 0; e < 8; ++e) p[8 * ks + e] = gg.v[e] * kLog2e;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qf[ks] = ld8_row<D, DM>(q + rowoff + 32 * ks, c);
            kf[ks] = ld8_row<D, DM>(k + rowoff + 32 * ks, c);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vf[ks] = ld8_row_once<D, DM>(v + rowoff + 32 * ks, c);
            dof[ks] = ld8_row_once<D, DM>(dout + rowoff + 32 * ks, c);
        }
        stage_fetch(0);

        // dAn[e] = dA[i = 4c+e][j = r],  dAt[e] = dA[i = r][j = 4c+e]   (dA = dO V^T), own sub-block
        f32x4 dAn = {0.f, 0.f, 0.f, 0.f}, dAt = {0.f, 0.f, 0.f, 0.f};
        auto own_dA = [&]() {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                st8(tV + wrow + 32 * ks, vf[ks]);
                st8(tO + wrow + 32 * ks, dof[ks]);
                dAn = mma_d(dof[ks], vf[ks], dAn);
                dAt = mma_d(vf[ks], dof[ks], dAt);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
            dd = reduce_over_cgroups(dd);
        };

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
            own_dA();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 gg = ld8_row<D, DM>(refetch(g + rowoff) + 32 * ks, c);
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
        float dot = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], bq[8], qo[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                dot += a[e] * bq[e];
                qo[e] = a[e] * fast_exp2(-s[8 * ks + e]);
                a[e] *= fast_exp2(p[8 * ks + e]);
                bq[e] *= fast_exp2(s[8 * ks + e]);
            }
            const D8 kh = pack8<T>(bq);
            st8(tQ + wrow + 32 * ks, pack8<T>(a));
            st8(tK + wrow + 32 * ks, kh);
            if (one_anchor) G = mma_d(pack8<T>(qo), kh, G);
        }
        dot = reduce_over_cgroups(dot);
#pragma unroll
        for (int e = 0; e < 4; ++e) Aown[e] += (4 * c + e == r) ? dot : 0.f;   // A_ii = q_i.k_i (gla.py:983)
        if (one_anchor) {
            own_dA();
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
    }
    row_fetch(0);
    __syncthreads();

    // ---- score blocks of both roles, cached as MFMA operands (2 registers each) -----------------------
    //   row owner:    dA^T of the earlier sub-blocks, dAx[J][j][i] = v_j . dO_i               (J < w)
    //   column owner: A_IJ (key side walked up by r_I) and dA_IJ = dAx[I] of the later ones   (I > w)
    T4 dAx[NB], Ac[NB], Acl;
    D8 Kt[KS];                           // k e^{L_end - L_j}: B operand of the dS' product of dv
    {
#pragma unroll
        for (int J = 0; J < NB; ++J) {
            dAx[J] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
            if (J < w) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    a = mma_d(ld8(tV + L.nat + 16 * J * LS + 32 * ks), ld8(tO + wrow + 32 * ks), a);
                dAx[J] = pack4<T>(a);
            }
        }
        float kch[NV];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) unpack8(ld8(tK + wrow + 32 * ks), kch + 8 * ks);
#pragma unroll
        for (int I = 1; I < NB; ++I) {
            Ac[I] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
            if (I > w) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    a = mma_d(ld8(tQ + L.nat + 16 * I * LS + 32 * ks), pack8<T>(kch + 8 * ks), a);
                    da = mma_d(ld8(tO + L.nat + 16 * I * LS + 32 * ks), vf[ks], da);
                    f32x8 rr = ld8(rtab + I * D + 32 * ks + 8 * c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) kch[8 * ks + e] *= rr.v[e];
                }
                Ac[I] = pack4<T>(a);
                dAx[I] = pack4<T>(da);
            }
        }
        // the own sub-block's scores enter dv = A^T dO as head + remainder: they are the largest of a column, and
        // under strong decay they carry most of dv
        split4<T>(Aown, Ac[0], Acl);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) Kt[ks] = pack8<T>(kch + 8 * ks);
    }
    __syncthreads();                 // every wave has cached its score blocks: the value tile is free
    stage_store(0);
    __syncthreads();

    // ---- the head dimension in slices of 32 features (a real loop: one slice's temporaries live) -------
    // Gradient w.r.t. the gate cumsum L of a row, "dL": every term dA_ij * q~_i * k~_j enters row i with +
    // and row j with -; both copies are formed from the SAME rounded operands (the values the MFMAs
    // consume), so they cancel exactly in the reverse cumsum (gla.py:1077-1087 asks for this).
#pragma unroll 1
    for (int ks = 0; ks < KS; ++ks) {
        const int fo = 32 * ks;
        float p8[8], s8[8], a[8], bq[8], dq8[8], dk8[8], dl8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) { p8[e] = gN.v[e] * kLog2e; s8[e] = 0.f; }
        unpack8(qN, a);
        unpack8(kN, bq);
        if (ks + 1 < KS) {
            row_fetch(ks + 1);
            stage_fetch(ks + 1);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            dq8[e] = dd * bq[e];         // diagonal term dA_ii q_i k_i: no gate gradient (gla.py:1181-1185)
            dk8[e] = dd * a[e];
            dl8[e] = 0.f;
        }
        if (one_anchor) {
            // the own sub-block is one more link on either side: dq~ = dA k~, dk~ = dA^T q~ (below the diagonal).
            // Both operands, q e^{l - tau} and k e^{tau - l}, enter as bf16 head + remainder.  With ONE anchor
            // per sub-block each row has a single rounding of either operand, shared by all of its 15 partners,
            // and under strong decay the pairs next to the diagonal carry most of the gate gradient: with plain
            // bf16 operands d(log_fgate) came out 1.2x (up to 2.7x) less accurate than the reference's dyadic
            // anchors give it (whose operand next to the anchor is exact); with the remainders it is 0.7x.
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
            f32x4 gq[2], hk[2];
            const f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
            if constexpr (sizeof(T) == 2) {
                // head + remainder carry 16 bits of mantissa: the multipliers of the gate gradient below are the
                // unrounded x and k e^{tau-l} themselves (they differ from what the MFMAs see by 2^-17, far below
                // the rounding of dA; the + and - copy of a pair term need not agree to the last bit)
                float t8[8];
                const D8 Xh = pack8<T>(x);
                unpack8(Xh, t8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    xr[e] = x[e];
                    t8[e] = x[e] - t8[e];
                }
                const D8 Xl = pack8<T>(t8);
                unpack8(ld8(tK + wrow + fo), t8);             // k e^{tau-l} as the key tile holds it
#pragma unroll
                for (int e = 0; e < 8; ++e) t8[e] = kr[e] - t8[e];    // what the tile's rounding left of it
                const D8 Kl = pack8<T>(t8);
                st8(xw + Lx.nat, Xh);
                st8(xw2 + Lx2.nat, Kl);
                asm volatile("" ::: "memory");
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    gq[tt] = mma_t(lds_tr4(xw2 + Lx2.k4 + 4 * tt, XS2), symb[0], z4);
                    gq[tt] = mma_t(lds_tr4(tK + L.k4 + fo + 4 * tt + 16 * w * LS, LS), symb[0], gq[tt]);
                }
                asm volatile("" ::: "memory");   // the same scratch rows now take the remainder of the query side
                st8(xw2 + Lx2.nat, Xl);
                asm volatile("" ::: "memory");
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    hk[tt] = mma_t(lds_tr4(xw2 + Lx2.k4 + 4 * tt, XS2), symb[1], z4);
                    hk[tt] = mma_t(lds_tr4(xw + Lx.k4 + 4 * tt, XS), symb[1], hk[tt]);
                }
            } else {
                const D8 X = pack8<T>(x);
                unpack8(X, xr);
                unpack8(ld8(tK + wrow + fo), kr);
                st8(xw + Lx.nat, X);
                asm volatile("" ::: "memory");
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    gq[tt] = mma_t(lds_tr4(tK + L.k4 + fo + 4 * tt + 16 * w * LS, LS), symb[0], z4);
                    hk[tt] = mma_t(lds_tr4(xw + Lx.k4 + 4 * tt, XS), symb[1], z4);
                }
            }
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dq8[4 * tt + e] += gq[tt][e] * fq[4 * tt + e];
                    dk8[4 * tt + e] += hk[tt][e] * fk[4 * tt + e];
                    dl8[4 * tt + e] += gq[tt][e] * xr[4 * tt + e] - hk[tt][e] * kr[4 * tt + e];
                }
            }
            asm volatile("" ::: "memory");
        } else {
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
            slice_level(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
            slice_level(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
            slice_level(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
            slice_level(std::integral_constant<int, 8>{}, std::integral_constant<int, 3>{});
        }
        // p8 = l_i, s8 = tau - l_i of the slice

        // -- dq: state term dO S^T first, then the earlier sub-blocks in ascending order
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                D8 dob = ld8(tO + wrow + 32 * k2);           // this lane's dout row
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    acc[tt] = mma_d(ld8(sS + L.own + 4 * tt * LS + 32 * k2), dob, acc[tt]);
            }
#pragma unroll
            for (int J = 0; J < NB - 1; ++J) {
                if (J < w) {
                    f32x8 rr = ld8(rtab + J * D + fo + 8 * c);
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[tt][e] *= rr.v[4 * tt + e];
                        acc[tt] = mma_t(lds_tr4(tK + L.k4 + fo + 4 * tt + 16 * J * LS, LS), dAx[J], acc[tt]);
                    }
                }
            }
            float o[8], qe[8], qr[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) qe[e] = a[e] * fast_exp2(p8[e]);
            unpack8(pack8<T>(qe), qr);                   // q e^{l} as the MFMAs of the key side see it
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float hacc = acc[e >> 2][e & 3];
                o[e] = fast_exp2(p8[e]) * hacc + dq8[e];
                dl8[e] += qr[e] * hacc;
            }
            st8_row_once<D, DM>(dq + rowoff + fo, c, pack8<TG>(o));
        }
        // -- dk: state term V dS'^T first, then the later sub-blocks in descending order
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    acc[tt] = mma_d(ld8(sDn + L.own + 4 * tt * LS + 32 * k2), vf[k2], acc[tt]);
            }
            {
                // second term of the chunk-level gate gradient: sum over the chunk's rows of k e^{L_end - L_j} times
                // the state term (v_j dS'^T) just formed (the reference's -sum_c dLambda_k, gla.py:776-782); summed
                // over the wave's 16 rows here, over the sub-blocks after the barrier
                D8 kts = Kt[0];
#pragma unroll
                for (int i = 1; i < KS; ++i) kts = ks == i ? Kt[i] : kts;
                float kte[8];
                unpack8(kts, kte);
                f32x8 tb;
#pragma unroll
                for (int e = 0; e < 8; ++e) tb.v[e] = suffix_sum_rows(kte[e] * acc[e >> 2][e & 3]);
                if (r == 0) st8(lbtab + w * 32 + 8 * c, tb);
            }
#pragma unroll
            for (int I = NB - 1; I >= 1; --I) {
                if (I > w) {
                    f32x8 rr = ld8(rtab + I * D + fo + 8 * c);
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[tt][e] *= rr.v[4 * tt + e];
                        acc[tt] = mma_t(lds_tr4(tQ + L.k4 + fo + 4 * tt + 16 * I * LS, LS), dAx[I], acc[tt]);
                    }
                }
            }
            float o[8], krt[8];
            unpack8(ld8(tK + wrow + fo), krt);             // k e^{tau-l} as the MFMAs of the chains saw it
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float hacc = acc[e >> 2][e & 3];
                o[e] = fast_exp2(s8[e]) * hacc + dk8[e];
                dl8[e] -= krt[e] * hacc;
            }
            st8_row_once<D, DM>(dk + rowoff + fo, c, pack8<TG>(o));
        }
        // -- dv: state term K~ dS' first, then the own and the later sub-blocks
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    acc[tt] = mma_d(ld8(sDt + L.own + 4 * tt * LS + 32 * k2), Kt[k2], acc[tt]);
            }
#pragma unroll
            for (int I = 0; I < NB; ++I) {
                if (I >= w) {
                    const T4 b4 = I == w ? Ac[0] : Ac[I];
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
                        const T4 oa = lds_tr4(tO + L.k4 + fo + 4 * tt + 16 * I * LS, LS);
                        if constexpr (sizeof(T) == 2) {
                            if (I == w) acc[tt] = mma_t(oa, Acl, acc[tt]);
                        }
                        acc[tt] = mma_t(oa, b4, acc[tt]);
                    }
                }
            }
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = acc[e >> 2][e & 3];
            st8_row_once<D, DM>(dv + rowoff + fo, c, pack8<TG>(o));
        }
        // -- dL of the slice is complete: reverse cumsum inside the sub-block (gla.py:616-617), then, once
        // every wave has published its sub-block total, over the whole chunk + the chunk-level term (gla.py:782)
        f32x8 sfx;
#pragma unroll
        for (int e = 0; e < 8; ++e) sfx.v[e] = suffix_sum_rows(dl8[e]);
        if (r == 0) st8(dltab + w * D + fo + 8 * c, sfx);
        __syncthreads();             // totals and lbar of the slice complete; its staged rows are free
        {
            f32x8 o = ld8(lbar + fo + 8 * c);
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] += sfx.v[e];
            {
                // sum of the sub-blocks' shares: the 16 rows of a lane group read one share each (two of them the
                // same one) and add up inside each half of the group
                static_assert(NB == 8 || NB == 4 || NB == 2, "one share per lane of a quad, a half row or a pair");
                f32x8 t = ld8(lbtab + (r & (NB - 1)) * 32 + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float x = t.v[e];
                    x += dpp_f32<kDppQuadXor1>(x);
                    if (NB >= 4) x += dpp_f32<kDppQuadXor2>(x);
                    if (NB >= 8) x += dpp_f32<kDppRowHalfMirror>(x);
                    o.v[e] += x;
                }
            }
            for (int m = w + 1; m < NB; ++m) {
                f32x8 t = ld8(dltab + m * D + fo + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) o.v[e] += t.v[e];
            }
            st8_row_once<D, DM>(dg + rowoff + fo, c, o);
        }
        if (ks + 1 < KS) {
            stage_store(ks + 1);
            __syncthreads();
        }
    }
}

template <typename T, int C, int D, int DM, bool WIDE>
int launch_chunk_grad(hipStream_t st, int B, int T_len, int H, const float *g, const void *v, const void *k,
                      const void *q, const void *dout, const void *statesN, const void *dstatesT,
                      const void *dstatesN, float *dg, void *dv, void *dk, void *dq)
{
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    constexpr int NB = C / 16;
    constexpr int VR = C > 96 ? C : 96;
    const size_t lds = ((size_t)(3 * C + VR) * LS + (size_t)NB * 16 * XS) * sizeof(T) +
                       ((size_t)(3 * NB + 1) * D + NB * 32) * sizeof(float) +
                       ((C - 96) * LS >= NB * 16 * 32 || sizeof(T) != 2 ? 0 : (size_t)NB * 16 * 32 * sizeof(T));
    auto kern = chunk_grad_kernel<T, C, D, DM, WIDE>;
    typedef std::conditional_t<WIDE, float, T> TG;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(T_len / C * H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)v, (const T *)k, (const T *)q,
                       (const T *)dout, (const T *)statesN, (const T *)dstatesT, (const T *)dstatesN, dg,
                       (TG *)dv, (TG *)dk, (TG *)dq, T_len, H);
    return launch_status();
}

#define GLA_INST_GRAD_AS(T, C, D, DM, WIDE)                                                                    \
    template int launch_chunk_grad<T, C, D, DM, WIDE>(hipStream_t, int, int, int, const float *, const void *, \
                                                      const void *, const void *, const void *, const void *, \
                                                      const void *, const void *, float *, void *, void *, void *);
#define GLA_INST_GRAD(T, C, D, DM) GLA_INST_GRAD_AS(T, C, D, DM, false)
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_GRAD)
GLA_INST_GRAD_AS(__bf16, 128, 128, 128, true)
GLA_INST_GRAD_AS(__bf16, 64, 128, 128, true)
GLA_INST_GRAD_AS(__bf16, 32, 128, 128, true)

}  // namespace gla
