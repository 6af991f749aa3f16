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
template <int C, int D>
__global__ __launch_bounds__(C * 8) void recurrent_stream_dq2_kernel(
    const BT *__restrict__ h0, const float *__restrict__ g, const BT *__restrict__ v, const BT *__restrict__ k,
    const BT *__restrict__ q, const BT *__restrict__ dhT, const BT *__restrict__ dout, BT *__restrict__ dq,
    float *__restrict__ qdq, int T_len, int H, int reverse)
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

    // state: S[j][e] = state[dk = 16(nt0 + j) + r][dv = 16 tv + 4c + e]
    f32x4 S[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        float t4[4];
        load_vec<T, 4>(h0 + bh * D * D + (int64_t)(16 * (nt0 + j) + r) * D + 16 * tv + 4 * c, t4);
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
    D8 qN, kN, vN, dN;
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
        dN = ld8(dout + rowN);
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
                qN = kN = vN = dN = pack8<T>(z);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e] = gN.v[e] * kLog2e;
            qf = qN;
            unpack8(kN, bq);
            st8(Vn + wrow + fo, vN);
            st8(tO + wrow + fo, dN);

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
            D8 dof[KS], vf[KS], vJ[NJ][KS], sLo[KS][2], sHi[KS][2];
            f32x8 rr[NJ];
            T4 kh[NJ][2], kl[NJ][2], kho[2], klo[2];
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                dof[k2] = ld8(tO + wrow + 32 * k2);
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
            for (int k2 = 0; k2 < KS; ++k2) dAt = mma_d(vf[k2], dof[k2], dAt);
            // the state term of the slice
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    acc[tt] = mma_d(sLo[k2][tt], dof[k2], acc[tt]);
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
                for (int k2 = 0; k2 < KS; ++k2) da = mma_d(vJ[J][k2], dof[k2], da);
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
                for (int k2 = 0; k2 < KS; ++k2) dAn = mma_d(dof[k2], vf[k2], dAn);
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
        unpack8(ld8(dhT + bh * D * D + (int64_t)d * D + part * 8), dv8);
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

template <int C, int D>
static int launch_dq2(hipStream_t st, int B, int T_len, int H, int reverse, const void *h0, const float *g,
                      const void *v, const void *k, const void *q, const void *dhT, const void *dout, void *dq,
                      float *qdq)
{
    typedef BT T;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    const size_t lds = ((size_t)(4 * C + 2 * D) * LS + (size_t)(C / 8) * 2 * 16 * XS) * sizeof(T) +
                       (size_t)(C / 16) * D * sizeof(float);
    auto kern = recurrent_stream_dq2_kernel<C, D>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(H, B), block(C * 8);
    hipLaunchKernelGGL(kern, grid, block, lds, st, (const T *)h0, g, (const T *)v, (const T *)k, (const T *)q,
                       (const T *)dhT, (const T *)dout, (T *)dq, qdq, T_len, H, reverse);
    return launch_status();
}

int launch_recurrent_stream_dq2(hipStream_t st, int B, int T_len, int H, int D, int reverse, const void *h0,
                                const float *g, const void *v, const void *k, const void *q, const void *dhT,
                                const void *dout, void *dq, float *qdq)
{
    if (D == 64) return launch_dq2<64, 64>(st, B, T_len, H, reverse, h0, g, v, k, q, dhT, dout, dq, qdq);
    return GLA_ERR_UNSUPPORTED;
}

}  // namespace gla
