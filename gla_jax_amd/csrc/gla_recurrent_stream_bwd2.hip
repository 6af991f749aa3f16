// recurrent_gla backward for bf16 inputs at head dimension 64, two waves per 16-step sub-block: the two sweeps
// of gla_recurrent_stream_bwd.hip (see there for the block form and the formulas; gla.py:271-360, 263) with
// each sub-block's work cut in two along the features.  A (batch, head) pair offers one workgroup of
// sequential work; with one wave per sub-block that is one wave per SIMD, and every latency of the wave (LDS
// round trips, dependent MFMAs, the row scans) is idle time of the SIMD.  Here a workgroup has 2 * C / 16
// waves: wave W < NB takes sub-block W and the features 0..31, wave W >= NB takes sub-block 2 NB - 1 - W and the
// features 32..63.  Waves W and W + NB share a SIMD, and their sub-blocks are I and NB - 1 - I: the Horner
// chains of a sub-block have as many links as it has earlier (sweep 1) or later (sweep 2) sub-blocks, so every
// SIMD carries the same number of links.
//
// What a feature slice means per quantity: gates, q, k and everything elementwise in the key features (the
// rescaled tiles, dq, dk, q*dq, d(log_fgate)) are handled on the wave's 32 key features; dv on its 32 value
// features; the states are split by tiles (two 16x16 tiles per wave).  Products that contract over ALL features
// take their operands from LDS tiles that both waves of a sub-block fill (dA = dO V^T, the state terms), or are
// formed per slice and added up through LDS (the scores A = Q~ K~^T of sweep 2).
#include "gla_recurrent_stream_bwd.hpp"
#include "gla_recurrent_stream.hpp"

namespace gla {

// ---------------------------------------------------------------------------------------------------
// sweep 1: dq and q*dq, the state S in accumulator registers
// ---------------------------------------------------------------------------------------------------
template <typename TO, int C, int D>
__global__ __launch_bounds__(C * 8) void recurrent_stream_dq2_kernel(
    const void *__restrict__ h0, const float *__restrict__ g, const BT *__restrict__ v, const BT *__restrict__ k,
    const BT *__restrict__ q, const void *__restrict__ dhT, const TO *__restrict__ dout, BT *__restrict__ dq,
    float *__restrict__ qdq, int T_len, int H, int reverse, int hdt)
{
    typedef BT T;
    constexpr int NB = C / 16, NW = 2 * NB, KS = D / 32, NT = D / 16;
    static_assert(D == 64 && KS == 2, "a wave takes one 32-feature slice of two");
    static_assert(NT * NT == 2 * NW, "two state tiles per wave");
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    typedef FragTypes<T>::d8 D8;
    typedef FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *Vn = reinterpret_cast<T *>(smem);           // [C][LS]  value
    T *tO = Vn + C * LS;                           // [C][LS]  dout
    T *Kh = tO + C * LS;                           // [C][LS]  k * exp(tau_J - l_j), bf16 head
    T *Kl = Kh + C * LS;                           // [C][LS]  ... and remainder
    T *Sh = Kl + C * LS;                           // [D][LS]  state at the start of the block, [dk][dv], head
    T *Sl = Sh + D * LS;                           // [D][LS]  ... and remainder
    T *xs = Sl + D * LS;                           // [NW][2][16][XS] per-wave scratch (hard gates only)
    float *rtab = reinterpret_cast<float *>(xs + NW * 2 * 16 * XS);   // [NB][D] exp(tau_m)
    constexpr bool kSplitDout = sizeof(TO) == 4;   // an fp32 dout enters the products as bf16 head + remainder
    T *tOl = reinterpret_cast<T *>(rtab + NB * D); // [C][LS]  the remainder of dout (fp32 dout only)

    const int lane = threadIdx.x & 63;
    const int W = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int I = W < NB ? W : NW - 1 - W;         // the wave's sub-block
    const int fo = W < NB ? 0 : 32;                // ... and its first feature
    const int r = lane & 15, c = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y;
    const int64_t seq = ((int64_t)b * T_len * H + h) * D;
    const int64_t rowstride = (int64_t)H * D;
    const int64_t bh = (int64_t)b * H + h;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const TrLane<T> Lx = make_tr_lane<T>(XS);
    const int ptl = plain_tr_lane<T>(LS);
    const int wrow = 16 * I * LS + L.nat;          // this lane's row of a tile, features 8c..8c+7
    T *xh = xs + (2 * W) * 16 * XS, *xl = xh + 16 * XS;
    const int N = (T_len + C - 1) / C;
    const int tv = W % NB, nt0 = 2 * (W / NB);     // the wave's state tiles: value tile tv, key tiles nt0, nt0 + 1
    // the wave with the longer chain of the two on a SIMD goes first when both are ready
    if (I >= NB / 2) __builtin_amdgcn_s_setprio(1);

    // state: S[j][e] = state[dk = 16(nt0 + j) + r][dv = 16 tv + 4c + e]
    f32x4 S[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        float t4[4];
        load_hidden<4>(h0, hdt, bh * D * D + (int64_t)(16 * (nt0 + j) + r) * D + 16 * tv + 4 * c, t4);
        S[j] = f32x4{t4[0], t4[1], t4[2], t4[3]};
    }
    auto publish_state = [&]() {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            T4 hi, lo;
            split4<T>(S[j], hi, lo);
            const int off = (16 * (nt0 + j) + r) * LS + 16 * tv + 4 * c;
            *reinterpret_cast<T4 *>(Sh + off) = hi;
            *reinterpret_cast<T4 *>(Sl + off) = lo;
        }
    };
    publish_state();

    f32x8 gN;
    D8 qN, kN, vN;
    DoutRow<TO> dN;
    bool validN;
    int64_t rowN;
    // The rows of a block are requested in three pieces (gates; q, k; v, dout), see the loop.
    auto fetch_g = [&](int n) {
        const int s = n * C + 16 * I + r;
        validN = s < T_len;
        const int sc = validN ? s : T_len - 1;
        rowN = seq + (int64_t)(reverse ? T_len - 1 - sc : sc) * rowstride + fo + 8 * c;
        gN = ld8(g + rowN);
    };
    auto fetch_qk = [&]() {
        qN = ld8(q + rowN);
        kN = ld8(k + rowN);
    };
    auto fetch_vo = [&]() {
        vN = ld8(v + rowN);
        dN.load(dout + rowN);
    };
    fetch_g(0);
    fetch_qk();
    fetch_vo();

    // Memory traffic is spread over the block.  All workgroups of the launch run in step; when each of them
    // issues a block's requests and stores in one burst (74 KB per CU, 19 MB over the chip), the queues of the
    // memory path fill and the waves stand at their load and store instructions for microseconds while that
    // burst drains: a clock trace showed 3 000 to 6 500 cycles of a 13 000-cycle block spent issuing nine memory
    // instructions per wave.  So the next block's rows are requested in three pieces and the results of a block
    // are stored one block late, in two pieces, each between two stretches of arithmetic; a wave waits for its
    // memory operations in the order it issued them, and a store that is a block old has long been acknowledged
    // when the wait for the rows behind it comes.
    D8 o_late;
    f32x8 prod_late;
    int64_t row_late = 0;
    bool valid_late = false;
    auto store_late_dq = [&]() {
        if (valid_late) st8(dq + row_late, o_late);
    };
    auto store_late_qdq = [&]() {
        if (valid_late) st8(qdq + row_late, prod_late);
    };

#pragma unroll 1
    for (int n = 0; n < N; ++n) {
        const bool valid = validN;
        const int64_t row = rowN;            // element offset of the lane's 8 features of its row
        float p[8], bq[8];                   // l_i; k
        D8 qf;
        float rw[8];                         // e^{tau} of the slice
        bool one_anchor;
        {
            if ((n + 1) * C > T_len && !valid) {   // only the last block can hold padded steps
                float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                gN = pack8<float>(z);
                qN = kN = vN = pack8<T>(z);
                dN.zero();
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e] = gN.v[e] * kLog2e;
            qf = qN;
            unpack8(kN, bq);
            st8(Vn + wrow + fo, vN);
            st8(tO + wrow + fo, dN.operand());
            if constexpr (kSplitDout) st8(tOl + wrow + fo, dN.remainder());

            // gate prefix, totals through the wave's half of the table row, one anchor or not
            float *rt = rtab + I * D + fo + 8 * c;
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e] = prefix_sum_rows(p[e]);
            if (r == 15) st8(rt, pack8<float>(p));
            asm volatile("" ::: "memory");
            const f32x8 tau = ld8(rt);
            float span = 0.f, sv[8], ke[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sv[e] = tau.v[e] - p[e];
                span = fmaxf(span, fmaxf(fabsf(p[e]), fabsf(sv[e])));
            }
            one_anchor = wave_all_below(span, kOneAnchorSpan);
            if (__builtin_expect(!one_anchor, false)) {
                // hard gates: l_i and tau - l_i from the sibling hierarchy instead (a suffix sum of its own, not the
                // difference of two long prefix sums)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    p[e] = gN.v[e] * kLog2e;
                    sv[e] = 0.f;
                }
                hier_step<1>(p, sv, (r & 1) != 0);
                hier_step<2>(p, sv, (r & 2) != 0);
                hier_step<4>(p, sv, (r & 4) != 0);
                hier_step<8>(p, sv, (r & 8) != 0);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ke[e] = bq[e] * fast_exp2(sv[e]);        // tau - l_i <= 0 whatever the gates
                rw[e] = fast_exp2(p[e] + sv[e]);
            }
            D8 kh, kl;
            split8<T>(ke, kh, kl);
            st8(Kh + wrow + fo, kh);
            st8(Kl + wrow + fo, kl);
            asm volatile("" ::: "memory");
            if (r == 0) st8(rt, pack8<float>(rw));
        }
        lds_barrier();                       // tiles of this block and the published state are in place
        const bool more = n + 1 < N;
        store_late_dq();
        if (more) fetch_g(n + 1);
        __builtin_amdgcn_sched_barrier(0);

        // Everything from here to the stores reads LDS at addresses known now, so ALL of those reads are issued
        // first, in the order their results are needed, and the arithmetic follows behind a scheduling barrier:
        // the compiler on its own puts each read right in front of its use and the wave then waits out one LDS
        // round trip per operand (the chain of sub-block 3 took 4 400 cycles that way).  The sub-block index is a
        // compile-time constant inside (a scalar branch picks the copy), so the links are straight-line code.
        auto chain = [&](auto Ic) {
            constexpr int I_ = decltype(Ic)::value;
            constexpr int NJ = I_ > 0 ? I_ : 1;
            D8 dof[KS], dofl[KS], vf[KS], vJ[NJ][KS], sLo[KS][2], sHi[KS][2];
            f32x8 rr[NJ];
            T4 kh[NJ][2], kl[NJ][2], kho[2], klo[2];
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                dof[k2] = ld8(tO + wrow + 32 * k2);
                if constexpr (kSplitDout) dofl[k2] = ld8(tOl + wrow + 32 * k2);
                vf[k2] = ld8(Vn + wrow + 32 * k2);
            }
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    sLo[k2][tt] = ld8(Sl + L.own + (fo + 4 * tt) * LS + 32 * k2);
                    sHi[k2][tt] = ld8(Sh + L.own + (fo + 4 * tt) * LS + 32 * k2);
                }
#pragma unroll
            for (int J = 0; J < I_; ++J)
#pragma unroll
                for (int k2 = 0; k2 < KS; ++k2) vJ[J][k2] = ld8(Vn + L.nat + 16 * J * LS + 32 * k2);
#pragma unroll
            for (int J = 0; J < I_; ++J) {
                rr[J] = ld8(rtab + J * D + fo + 8 * c);
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    kh[J][tt] = lds_tr4(Kh + L.k4 + fo + 4 * tt + 16 * J * LS, LS);
                    kl[J][tt] = lds_tr4(Kl + L.k4 + fo + 4 * tt + 16 * J * LS, LS);
                }
            }
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                kho[tt] = lds_tr4(Kh + L.k4 + fo + 4 * tt + 16 * I_ * LS, LS);
                klo[tt] = lds_tr4(Kl + L.k4 + fo + 4 * tt + 16 * I_ * LS, LS);
            }
            __builtin_amdgcn_sched_barrier(0);

            // dA = dO V^T contracts over all value features.  dAt[e] = dA[i = r][j = 4c+e] of the own sub-block;
            // dA^T of the pairs with the earlier sub-blocks, [j][i] = v_j . do_i.
            f32x4 dAt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                if constexpr (kSplitDout) dAt = mma_d(vf[k2], dofl[k2], dAt);
                dAt = mma_d(vf[k2], dof[k2], dAt);
            }
            // the state term of the slice
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    acc[tt] = mma_d(sLo[k2][tt], dof[k2], acc[tt]);
                    if constexpr (kSplitDout) acc[tt] = mma_d(sHi[k2][tt], dofl[k2], acc[tt]);
                    acc[tt] = mma_d(sHi[k2][tt], dof[k2], acc[tt]);
                }
            __builtin_amdgcn_sched_barrier(0);
            store_late_qdq();
            if (more) fetch_qk();
            __builtin_amdgcn_sched_barrier(0);
            T4 dah[NJ], dal[NJ];
#pragma unroll
            for (int J = 0; J < I_; ++J) {
                f32x4 da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int k2 = 0; k2 < KS; ++k2) {
                    if constexpr (kSplitDout) da = mma_d(vJ[J][k2], dofl[k2], da);
                    da = mma_d(vJ[J][k2], dof[k2], da);
                }
                split4<T>(da, dah[J], dal[J]);
            }
            // the earlier sub-blocks in ascending order
#pragma unroll
            for (int J = 0; J < I_; ++J) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[tt][e] *= rr[J].v[4 * tt + e];
                    acc[tt] = mma_t_split(kh[J][tt], kl[J][tt], dah[J], dal[J], acc[tt]);
                }
            }
            // the own sub-block
            float dd = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
            dd = reduce_over_cgroups(dd);
            float dqo[8];                        // the own sub-block's part of dq (already scaled)
            f32x4 gq[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            if (__builtin_expect(one_anchor, true)) {
                f32x4 lowT;                      // dA^T below the diagonal
                T4 lowTh, lowTl;
#pragma unroll
                for (int e = 0; e < 4; ++e) lowT[e] = (4 * c + e < r) ? dAt[e] : 0.f;
                split4<T>(lowT, lowTh, lowTl);
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) gq[tt] = mma_t_split(kho[tt], klo[tt], lowTh, lowTl, gq[tt]);
#pragma unroll
                for (int e = 0; e < 8; ++e) dqo[e] = dd * bq[e];             // diagonal term (gla.py:1181-1185)
            } else {
                // hard gates: the dyadic levels on the slice, inputs fetched again
                f32x4 dAn = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int k2 = 0; k2 < KS; ++k2) {
                    if constexpr (kSplitDout) dAn = mma_d(dofl[k2], vf[k2], dAn);
                    dAn = mma_d(dof[k2], vf[k2], dAn);
                }
                const HardSliceDq hs = hard_slice_dq<XS, false>(
                    g + row, q + row, k + row, valid ? 1.f : 0.f, dd, dAt, dAn, (LdsBT)xh, (LdsBT)xl, Lx.nat, Lx.k4,
                    (LdsF32) nullptr, (LdsBT) nullptr, (LdsBT) nullptr);
#pragma unroll
                for (int e = 0; e < 8; ++e) dqo[e] = hs.dq8[e];
            }
            float o[8], a[8];
            unpack8(qf, a);
            f32x8 prod;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float el = fast_exp2(p[e]);
                const float es = one_anchor ? el * __builtin_amdgcn_rcpf(rw[e]) : 0.f;   // e^{-s} = e^{l} / e^{tau}
                o[e] = el * acc[e >> 2][e & 3] + es * gq[e >> 2][e & 3] + dqo[e];
                prod.v[e] = a[e] * o[e];
            }
            o_late = pack8<T>(o);
            prod_late = prod;
            row_late = row;
            valid_late = valid;
        };
        switch (I) {
        case 0: chain(std::integral_constant<int, 0>{}); break;
        case 1: chain(std::integral_constant<int, 1>{}); break;
        case 2: chain(std::integral_constant<int, 2>{}); break;
        default: chain(std::integral_constant<int, 3>{}); break;
        }
        __builtin_amdgcn_sched_barrier(0);
        if (more) fetch_vo();
        __builtin_amdgcn_sched_barrier(0);

        // ---- state update: S <- S e^{tau_J} + V_J^T (k e^{tau_J - l})_J over the sub-blocks in order ------
        {
            float rr[NB][2];
            T4 va[NB], ukl[NB][2], ukh[NB][2];
#pragma unroll
            for (int J = 0; J < NB; ++J) {
#pragma unroll
                for (int j = 0; j < 2; ++j) rr[J][j] = rtab[J * D + 16 * (nt0 + j) + r];
                va[J] = lds_tr4(Vn + ptl + 16 * J * LS + 16 * tv, LS);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    ukl[J][j] = lds_tr4(Kl + ptl + 16 * J * LS + 16 * (nt0 + j), LS);
                    ukh[J][j] = lds_tr4(Kh + ptl + 16 * J * LS + 16 * (nt0 + j), LS);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int J = 0; J < NB; ++J) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) S[j][e] *= rr[J][j];
                    S[j] = mma_t(va[J], ukl[J][j], S[j]);
                    S[j] = mma_t(va[J], ukh[J][j], S[j]);
                }
            }
        }
        lds_barrier();                       // every wave is done with the tiles and the old state
        publish_state();
    }

    store_late_dq();
    store_late_qdq();
    // The last term of gla.py:263, sum_v dhT * hT per key feature, from the state this sweep ends with (just
    // published as bf16 head + remainder).  Every d(log_fgate)_t is a sum over the steps s >= t, so the term is
    // added to q*dq of the LAST step and reaches all of them through sweep 2's running sum.
    __syncthreads();           // the published state and every q*dq row are in place
    {
        constexpr int LPF = C * 8 / D;                                   // lanes per key feature
        static_assert(LPF == 8, "eight neighbouring lanes share a key feature");
        const int d = threadIdx.x / LPF, part = threadIdx.x % LPF;       // each takes D / LPF = 8 of the row
        float dv8[8], sh[8], sl[8], acc = 0.f;
        load_hidden<8>(dhT, hdt, bh * D * D + (int64_t)d * D + part * 8, dv8);
        unpack8(ld8(Sh + d * LS + part * 8), sh);
        unpack8(ld8(Sl + d * LS + part * 8), sl);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += dv8[e] * (sh[e] + sl[e]);
        acc += dpp_f32<kDppQuadXor1>(acc);
        acc += dpp_f32<kDppQuadXor2>(acc);
        acc += dpp_f32<kDppRowHalfMirror>(acc);
        if (part == 0) {
            float *lp = qdq + seq + (int64_t)(reverse ? 0 : T_len - 1) * rowstride + d;
            *lp += acc;
        }
    }
}

template <typename TO, int C, int D>
static int launch_dq2(hipStream_t st, int B, int T_len, int H, int reverse, int hdt, const void *h0, const float *g,
                      const void *v, const void *k, const void *q, const void *dhT, const void *dout, void *dq,
                      float *qdq)
{
    typedef BT T;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    const size_t lds = ((size_t)(4 * C + 2 * D + (sizeof(TO) == 4 ? C : 0)) * LS + (size_t)(C / 8) * 2 * 16 * XS) *
                           sizeof(T) +
                       (size_t)(C / 16) * D * sizeof(float);
    auto kern = recurrent_stream_dq2_kernel<TO, C, D>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(H, B), block(C * 8);
    hipLaunchKernelGGL(kern, grid, block, lds, st, h0, g, (const T *)v, (const T *)k, (const T *)q,
                       dhT, (const TO *)dout, (T *)dq, qdq, T_len, H, reverse, hdt);
    return launch_status();
}

// ---------------------------------------------------------------------------------------------------
// sweep 2: dk, dv, dh0 and d(log_fgate), dS in accumulator registers (formulas: gla_recurrent_stream_bwd.hip).
// A wave holds the 32 key features fo.. of its 16 rows for everything elementwise and for dk, the 32 value
// features fo.. for dv.  The scores A = Q~ K~^T contract over the key features: each wave forms them on its
// slice and the two waves of a sub-block add their halves through LDS (one more barrier per block).
// ---------------------------------------------------------------------------------------------------
template <typename TO, int C, int D>
__global__ __launch_bounds__(C * 8) void recurrent_stream_rev2_kernel(
    const float *__restrict__ g, const BT *__restrict__ v, const BT *__restrict__ k, const BT *__restrict__ q,
    const void *__restrict__ dhT, const TO *__restrict__ dout, void *__restrict__ dh0,
    float *__restrict__ dg, BT *__restrict__ dv, BT *__restrict__ dk, int T_len, int H, int reverse, int hdt)
{
    typedef BT T;
    constexpr int NB = C / 16, NW = 2 * NB, KS = D / 32, NT = D / 16;
    static_assert(D == 64 && KS == 2, "a wave takes one 32-feature slice of two");
    static_assert(NT * NT == 2 * NW, "two state tiles per wave");
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    typedef FragTypes<T>::d8 D8;
    typedef FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *tO = reinterpret_cast<T *>(smem);           // [C][LS]  dout
    T *Vn = tO + C * LS;                           // [C][LS]  value
    T *Qh = Vn + C * LS;                           // [C][LS]  q * exp(l_i), bf16 head
    T *Ql = Qh + C * LS;                           // [C][LS]  ... and remainder
    T *KTh = Ql + C * LS;                          // [C][LS]  k * exp(Lend - L_j), head
    T *KTl = KTh + C * LS;                         // [C][LS]  ... and remainder
    T *DTh = KTl + C * LS;                         // [D][LS]  dS' as [dv][dk], head
    T *DTl = DTh + D * LS;                         // [D][LS]  ... and remainder
    T *xs = DTl + D * LS;                          // [NW][2][16][XS] per-wave scratch
    float *rtab = reinterpret_cast<float *>(xs + NW * 2 * 16 * XS);   // [NB][D] exp(tau_m)
    float *dltab = rtab + NB * D;                  // [NB][D] sub-block sums of q*dq - k*dk
    float *runtab = dltab + NB * D;                // [2][D]  sum over the later blocks, double-buffered
    f32x4 *xch = reinterpret_cast<f32x4 *>(runtab + 2 * D);          // [NW][NB][64] score blocks of a slice
    constexpr bool kSplitDout = sizeof(TO) == 4;   // an fp32 dout enters the products as bf16 head + remainder
    T *tOl = reinterpret_cast<T *>(xch + NW * NB * 64);               // [C][LS]  the remainder of dout (fp32 dout only)

    const int lane = threadIdx.x & 63;
    const int W = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int J0 = W < NB ? W : NW - 1 - W;        // the wave's sub-block
    const int fo = W < NB ? 0 : 32;                // ... and its first feature
    const int PW = NW - 1 - W;                     // the wave with the other half of the sub-block
    const int r = lane & 15, c = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y;
    const int64_t seq = ((int64_t)b * T_len * H + h) * D;
    const int64_t rowstride = (int64_t)H * D;
    const int64_t bh = (int64_t)b * H + h;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const TrLane<T> Lx = make_tr_lane<T>(XS);
    const int ptl = plain_tr_lane<T>(LS);
    const int wrow = 16 * J0 * LS + L.nat;
    T *xh = xs + (2 * W) * 16 * XS, *xl = xh + 16 * XS;
    const int N = (T_len + C - 1) / C;
    const int td = W % NB, nt0 = 2 * (W / NB);     // the wave's state tiles: key tile td, value tiles nt0, nt0 + 1
    // the wave with the longer chains of the two on a SIMD goes first when both are ready
    if (J0 < NB / 2) __builtin_amdgcn_s_setprio(1);

    // dS: DS[j][e] = dS[dk = 16 td + 4c + e][dv = 16(nt0 + j) + r]
    f32x4 DS[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            DS[j][e] = load_hidden1(dhT, hdt, bh * D * D + (int64_t)(16 * td + 4 * c + e) * D + 16 * (nt0 + j) + r);
    auto publish = [&]() {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            T4 hi, lo;
            split4<T>(DS[j], hi, lo);
            const int off = (16 * (nt0 + j) + r) * LS + 16 * td + 4 * c;
            *reinterpret_cast<T4 *>(DTh + off) = hi;
            *reinterpret_cast<T4 *>(DTl + off) = lo;
        }
    };
    publish();
    for (int d = threadIdx.x; d < 2 * D; d += C * 8) runtab[d] = 0.f;

    // Memory traffic is spread over the block as in sweep 1: the next block's rows are requested in four pieces
    // (gates; q, k; sweep 1's q*dq; v, dout) and a block's results are stored one block late, in three pieces.
    f32x8 gN, qdqN;
    D8 qN, kN, vN;
    DoutRow<TO> dN;
    bool validN;
    int64_t rowN;
    auto fetch_g = [&](int n) {
        const int s = n * C + 16 * J0 + r;
        validN = s < T_len;
        const int sc = validN ? s : T_len - 1;
        rowN = seq + (int64_t)(reverse ? T_len - 1 - sc : sc) * rowstride + fo + 8 * c;
        gN = ld8(g + rowN);
    };
    auto fetch_qk = [&]() {
        qN = ld8(q + rowN);
        kN = ld8(k + rowN);
    };
    auto fetch_qdq = [&]() { qdqN = ld8(dg + rowN); };
    auto fetch_vo = [&]() {
        vN = ld8(v + rowN);
        dN.load(dout + rowN);
    };
    fetch_g(N - 1);
    fetch_qk();
    fetch_qdq();
    fetch_vo();
    D8 dv_late, dk_late;
    f32x8 dg_late;
    int64_t row_late = 0;
    bool valid_late = false;

#pragma unroll 1
    for (int n = N - 1; n >= 0; --n) {
        const bool valid = validN;
        const int64_t row = rowN;            // element offset of the lane's 8 features of its row
        float p[8], sv[8], a[8], bq[8], kt[8];   // l_i; tau - l_i; q; k; k e^{tau - l_i}
        bool one_anchor;
        {
            if ((n + 1) * C > T_len && !valid) {   // only the last block can hold padded steps
                float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                gN = pack8<float>(z);
                qN = kN = vN = pack8<T>(z);
                dN.zero();
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e] = gN.v[e] * kLog2e;
            unpack8(qN, a);
            unpack8(kN, bq);
            if (!valid) {
                float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                qdqN = pack8<float>(z);
            }
            st8(tO + wrow + fo, dN.operand());
            if constexpr (kSplitDout) st8(tOl + wrow + fo, dN.remainder());
            st8(Vn + wrow + fo, vN);

            float *rt = rtab + J0 * D + fo + 8 * c;
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e] = prefix_sum_rows(p[e]);
            if (r == 15) st8(rt, pack8<float>(p));
            asm volatile("" ::: "memory");
            const f32x8 tau = ld8(rt);
            float span = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sv[e] = tau.v[e] - p[e];
                span = fmaxf(span, fmaxf(fabsf(p[e]), fabsf(sv[e])));
            }
            one_anchor = wave_all_below(span, kOneAnchorSpan);
            if (__builtin_expect(!one_anchor, false)) {
                // hard gates: l_i and tau - l_i from the sibling hierarchy (see sweep 1)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    p[e] = gN.v[e] * kLog2e;
                    sv[e] = 0.f;
                }
                hier_step<1>(p, sv, (r & 1) != 0);
                hier_step<2>(p, sv, (r & 2) != 0);
                hier_step<4>(p, sv, (r & 4) != 0);
                hier_step<8>(p, sv, (r & 8) != 0);
            }
            float qe[8], rw[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                qe[e] = a[e] * fast_exp2(p[e]);
                kt[e] = bq[e] * fast_exp2(sv[e]);
                rw[e] = fast_exp2(p[e] + sv[e]);
            }
            D8 h8, l8;
            split8<T>(qe, h8, l8);
            st8(Qh + wrow + fo, h8);
            st8(Ql + wrow + fo, l8);
            asm volatile("" ::: "memory");
            if (r == 0) st8(rt, pack8<float>(rw));
        }
        float qdq[8];                        // q*dq of the rows (sweep 1 left it in the d(log_fgate) buffer)
#pragma unroll
        for (int e = 0; e < 8; ++e) qdq[e] = qdqN.v[e];
        lds_barrier();                       // tiles of this block and the published dS' are in place
        const bool more = n > 0;
        if (valid_late) st8(dv + row_late, dv_late);
        if (more) fetch_g(n - 1);
        __builtin_amdgcn_sched_barrier(0);

        // ---- products that contract over all value features (operands from the tiles), the own sub-block ----
        D8 vf[KS];
        float dko[8];                        // the own sub-block's part of dk
        f32x4 Aown = {0.f, 0.f, 0.f, 0.f};   // this slice's share of the scores A[i = 4c+e][j = r] of the own sub-block
        {
            D8 dof[KS];
            f32x4 dAn = {0.f, 0.f, 0.f, 0.f}, dAt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                dof[k2] = ld8(tO + wrow + 32 * k2);
                vf[k2] = ld8(Vn + wrow + 32 * k2);
            }
            if constexpr (kSplitDout) {
#pragma unroll
                for (int k2 = 0; k2 < KS; ++k2) {
                    const D8 dofl = ld8(tOl + wrow + 32 * k2);
                    dAn = mma_d(dofl, vf[k2], dAn);
                    dAt = mma_d(vf[k2], dofl, dAt);
                }
            }
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                dAn = mma_d(dof[k2], vf[k2], dAn);
                dAt = mma_d(vf[k2], dof[k2], dAt);
            }
            float dd = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
            dd = reduce_over_cgroups(dd);
            float dot = 0.f;
            if (__builtin_expect(one_anchor, true)) {
                f32x4 low;
                T4 lowh, lowl;               // dA of the own sub-block below the diagonal
#pragma unroll
                for (int e = 0; e < 4; ++e) low[e] = (4 * c + e > r) ? dAn[e] : 0.f;
                split4<T>(low, lowh, lowl);
                float qo[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    dot += a[e] * bq[e];
                    dko[e] = dd * a[e];
                    qo[e] = a[e] * fast_exp2(-sv[e]);
                }
                D8 oh, ol, kh, kl;
                split8<T>(qo, oh, ol);
                split8<T>(kt, kh, kl);
                const f32x4 G = mma_d_split(oh, ol, kh, kl, f32x4{0.f, 0.f, 0.f, 0.f});
                // own link of dk: H'^T[dk][j] = sum_{i > j} (q e^{-s})_i[dk] dA_ij, through the wave's scratch
                st8(xh + Lx.nat, oh);
                st8(xl + Lx.nat, ol);
                asm volatile("" ::: "memory");
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    f32x4 hk = {0.f, 0.f, 0.f, 0.f};
                    hk = mma_t_split(lds_tr4(xh + Lx.k4 + 4 * tt, XS), lds_tr4(xl + Lx.k4 + 4 * tt, XS), lowh, lowl, hk);
#pragma unroll
                    for (int e = 0; e < 4; ++e) dko[4 * tt + e] += hk[e] * fast_exp2(sv[4 * tt + e]);
                }
                asm volatile("" ::: "memory");
#pragma unroll
                for (int e = 0; e < 4; ++e) Aown[e] = (4 * c + e > r) ? G[e] : 0.f;
            } else {
                const f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
                const HardSliceRev hs = hard_slice_rev<XS, false>(
                    g + row, q + row, k + row, valid ? 1.f : 0.f, dd, dAt, dAn, z4, z4, z4, z4, 0.f, (LdsBT)xh, (LdsBT)xl,
                    Lx.nat, Lx.k4, (LdsF32) nullptr, (LdsBT) nullptr, (LdsBT) nullptr);
                dot = hs.dot;
#pragma unroll
                for (int e = 0; e < 8; ++e) dko[e] = hs.dk8[e];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int o = 4 * c + e;
                    float acc = 0.f;
#pragma unroll
                    for (int l = 0; l < 4; ++l) {
                        const int h_ = 1 << l;
                        const bool ok = ((o ^ r) < 2 * h_) && (o & h_) && !(r & h_);
                        acc += ok ? hs.G[l][e] : 0.f;
                    }
                    Aown[e] = acc;
                }
            }
            dot = reduce_over_cgroups(dot);
#pragma unroll
            for (int e = 0; e < 4; ++e) Aown[e] += (4 * c + e == r) ? dot : 0.f;   // A_ii = q_i.k_i (gla.py:983)
        }

        __builtin_amdgcn_sched_barrier(0);
        if (valid_late) st8(dk + row_late, dk_late);
        if (more) fetch_qk();
        __builtin_amdgcn_sched_barrier(0);
        // ---- score blocks of the later sub-blocks: this slice's share of A_Ij (key side walked up by r_I), dA_Ij
        T4 dAh[NB], dAl[NB];
        xch[(W * NB + J0) * 64 + lane] = Aown;
        {
            float kch[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) kch[e] = kt[e];
#pragma unroll
            for (int I = 1; I < NB; ++I) {
                dAh[I] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
                dAl[I] = dAh[I];
                if (I > J0) {
                    f32x4 as = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
                    D8 kh, kl;
                    split8<T>(kch, kh, kl);
                    as = mma_d_split(ld8(Qh + L.nat + 16 * I * LS + fo), ld8(Ql + L.nat + 16 * I * LS + fo), kh, kl, as);
#pragma unroll
                    for (int k2 = 0; k2 < KS; ++k2) {
                        if constexpr (kSplitDout) da = mma_d(ld8(tOl + L.nat + 16 * I * LS + 32 * k2), vf[k2], da);
                        da = mma_d(ld8(tO + L.nat + 16 * I * LS + 32 * k2), vf[k2], da);
                    }
                    f32x8 rr = ld8(rtab + I * D + fo + 8 * c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) kch[e] *= rr.v[e];
                    xch[(W * NB + I) * 64 + lane] = as;
                    split4<T>(da, dAh[I], dAl[I]);
                }
            }
            D8 kh, kl;                       // k e^{Lend - L_j} of the slice: operand of the dv state term of both halves
            split8<T>(kch, kh, kl);
            st8(KTh + wrow + fo, kh);
            st8(KTl + wrow + fo, kl);
        }
        lds_barrier();                       // both halves of every score block and of K~ are in place
        if (valid_late) st8(dg + row_late, dg_late);
        if (more) fetch_qdq();
        __builtin_amdgcn_sched_barrier(0);

        T4 Ach[NB], Acl[NB];                 // [0]: the own sub-block; [I]: the later ones
        {
            f32x4 t = xch[(W * NB + J0) * 64 + lane], u = xch[(PW * NB + J0) * 64 + lane];
#pragma unroll
            for (int e = 0; e < 4; ++e) t[e] += u[e];
            split4<T>(t, Ach[0], Acl[0]);
#pragma unroll
            for (int I = 1; I < NB; ++I) {
                Ach[I] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
                Acl[I] = Ach[I];
                if (I > J0) {
                    f32x4 t2 = xch[(W * NB + I) * 64 + lane], u2 = xch[(PW * NB + I) * 64 + lane];
#pragma unroll
                    for (int e = 0; e < 4; ++e) t2[e] += u2[e];
                    split4<T>(t2, Ach[I], Acl[I]);
                }
            }
        }

        // -- dv of the slice: dS'^T K~ first, then the own and the later sub-blocks
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                const D8 Kth = ld8(KTh + wrow + 32 * k2), Ktl = ld8(KTl + wrow + 32 * k2);
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    acc[tt] = mma_d_split(ld8(DTh + L.own + (fo + 4 * tt) * LS + 32 * k2),
                                          ld8(DTl + L.own + (fo + 4 * tt) * LS + 32 * k2), Kth, Ktl, acc[tt]);
            }
#pragma unroll
            for (int I = 0; I < NB; ++I) {
                if (I >= J0) {
                    const T4 bh4 = I == J0 ? Ach[0] : Ach[I], bl4 = I == J0 ? Acl[0] : Acl[I];
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
                        const T4 oa = lds_tr4(tO + L.k4 + fo + 4 * tt + 16 * I * LS, LS);
                        acc[tt] = mma_t(oa, bl4, acc[tt]);
                        if constexpr (kSplitDout)
                            acc[tt] = mma_t(lds_tr4(tOl + L.k4 + fo + 4 * tt + 16 * I * LS, LS), bh4, acc[tt]);
                        acc[tt] = mma_t(oa, bh4, acc[tt]);
                    }
                }
            }
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = acc[e >> 2][e & 3];
            dv_late = pack8<T>(o);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (more) fetch_vo();
        __builtin_amdgcn_sched_barrier(0);
        // -- dk of the slice: dS' v first, then the later sub-blocks in descending order
        {
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            // (dS' v)[dk][j] = sum_dv dS'[dk][dv] v_j[dv]: 16 dv rows per step, read transposed.  Step (k2, half)
            // contracts over dv = 32 k2 + 8 c + 4 half + m, which is what lane (j, c) holds of v_j.
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const T4 vb = half ? __builtin_shufflevector(vf[k2], vf[k2], 4, 5, 6, 7)
                                       : __builtin_shufflevector(vf[k2], vf[k2], 0, 1, 2, 3);
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
                        acc[tt] = mma_t(lds_tr4(DTl + L.k8 + (32 * k2 + 4 * half) * LS + fo + 4 * tt, LS), vb, acc[tt]);
                        acc[tt] = mma_t(lds_tr4(DTh + L.k8 + (32 * k2 + 4 * half) * LS + fo + 4 * tt, LS), vb, acc[tt]);
                    }
                }
            }
#pragma unroll
            for (int I = NB - 1; I >= 1; --I) {
                if (I > J0) {
                    f32x8 rr = ld8(rtab + I * D + fo + 8 * c);
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[tt][e] *= rr.v[4 * tt + e];
                        acc[tt] = mma_t_split(lds_tr4(Qh + L.k4 + fo + 4 * tt + 16 * I * LS, LS),
                                              lds_tr4(Ql + L.k4 + fo + 4 * tt + 16 * I * LS, LS), dAh[I], dAl[I],
                                              acc[tt]);
                    }
                }
            }
            float o[8];
            f32x8 sfx;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                o[e] = fast_exp2(sv[e]) * acc[e >> 2][e & 3] + dko[e];
                // q*dq - k*dk of the row, then its reverse running sum inside the sub-block
                sfx.v[e] = suffix_sum_rows(qdq[e] - bq[e] * o[e]);
                qdq[e] = sfx.v[e];
            }
            dk_late = pack8<T>(o);
            if (r == 0) st8(dltab + J0 * D + fo + 8 * c, sfx);
        }

        // ---- dS <- dS r_I + (q e^{l})_I^T dO_I over the sub-blocks, last first ---------------------------
#pragma unroll
        for (int I = NB - 1; I >= 0; --I) {
            const f32x4 rr = *reinterpret_cast<const f32x4 *>(rtab + I * D + 16 * td + 4 * c);
            const T4 qah = lds_tr4(Qh + ptl + 16 * I * LS + 16 * td, LS);
            const T4 qal = lds_tr4(Ql + ptl + 16 * I * LS + 16 * td, LS);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 4; ++e) DS[j][e] *= rr[e];
                const T4 ob = lds_tr4(tO + ptl + 16 * I * LS + 16 * (nt0 + j), LS);
                DS[j] = mma_t(qal, ob, DS[j]);
                if constexpr (kSplitDout) DS[j] = mma_t(qah, lds_tr4(tOl + ptl + 16 * I * LS + 16 * (nt0 + j), LS), DS[j]);
                DS[j] = mma_t(qah, ob, DS[j]);
            }
        }
        lds_barrier();                       // sub-block sums complete; every wave is done with the tiles
        {
            f32x8 o, tot = ld8(runtab + (n & 1) * D + fo + 8 * c);
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] = qdq[e] + tot.v[e];
#pragma unroll
            for (int m = 0; m < NB; ++m) {
                f32x8 t = ld8(dltab + m * D + fo + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    o.v[e] += m > J0 ? t.v[e] : 0.f;
                    tot.v[e] += t.v[e];
                }
            }
            if (J0 == 0 && r == 0) st8(runtab + ((n & 1) ^ 1) * D + fo + 8 * c, tot);
            dg_late = o;
            row_late = row;
            valid_late = valid;
        }
        publish();
    }
    if (valid_late) {
        st8(dv + row_late, dv_late);
        st8(dk + row_late, dk_late);
        st8(dg + row_late, dg_late);
    }

#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            store_hidden1(dh0, hdt, bh * D * D + (int64_t)(16 * td + 4 * c + e) * D + 16 * (nt0 + j) + r, DS[j][e]);
}

template <typename TO, int C, int D>
static int launch_rev2(hipStream_t st, int B, int T_len, int H, int reverse, int hdt, const float *g, const void *v,
                       const void *k, const void *q, const void *dhT, const void *dout, void *dh0, float *dg,
                       void *dv, void *dk)
{
    typedef BT T;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    constexpr int NB = C / 16, NW = 2 * NB;
    const size_t lds = ((size_t)(6 * C + 2 * D + (sizeof(TO) == 4 ? C : 0)) * LS + (size_t)NW * 2 * 16 * XS) * sizeof(T) +
                       (size_t)(2 * NB + 2) * D * sizeof(float) + (size_t)NW * NB * 64 * sizeof(f32x4);
    auto kern = recurrent_stream_rev2_kernel<TO, C, D>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(H, B), block(C * 8);
    hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)v, (const T *)k, (const T *)q, dhT,
                       (const TO *)dout, dh0, dg, (T *)dv, (T *)dk, T_len, H, reverse, hdt);
    return launch_status();
}

int launch_recurrent_stream_rev2(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                                 const float *g, const void *v, const void *k, const void *q, const void *dhT,
                                 const void *dout, void *dh0, float *dg, void *dv, void *dk)
{
    if (D == 64 && dout_f32)
        return launch_rev2<float, 64, 64>(st, B, T_len, H, reverse, hdt, g, v, k, q, dhT, dout, dh0, dg, dv, dk);
    if (D == 64) return launch_rev2<BT, 64, 64>(st, B, T_len, H, reverse, hdt, g, v, k, q, dhT, dout, dh0, dg, dv, dk);
    return GLA_ERR_UNSUPPORTED;
}

int launch_recurrent_stream_dq2(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                                const void *h0, const float *g, const void *v, const void *k, const void *q,
                                const void *dhT, const void *dout, void *dq, float *qdq)
{
    if (D == 64 && dout_f32)
        return launch_dq2<float, 64, 64>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, dhT, dout, dq, qdq);
    if (D == 64) return launch_dq2<BT, 64, 64>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, dhT, dout, dq, qdq);
    return GLA_ERR_UNSUPPORTED;
}

}  // namespace gla
