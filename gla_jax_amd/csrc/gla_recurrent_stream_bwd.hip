// recurrent_gla backward for bf16 inputs on the matrix cores: the two sweeps of gla.py:271-360 with the
// rank-1 updates of C consecutive timesteps applied together (see gla_recurrent_stream.hip for the block
// form of the recurrence).  Neither sweep stores a hidden state:
//   sweep 1 runs along the forward's direction with the state S in accumulator registers and writes
//           dq_t = S_t do_t and, in fp32 into the d(log_fgate) buffer, q_t * dq_t;
//   sweep 2 runs against it with dS in accumulator registers and writes dk_t = dS_t v_t, dv_t = dS_t^T k_t,
//           dh0, and d(log_fgate)_t = sum_{s>=t} (q_s*dq_s - k_s*dk_s) + sum_v dhT*hT   (gla.py:263).
// Every product whose operand is a rescaled (hence rounded) quantity takes it as bf16 head + remainder,
// so the gradients carry fp32-grade products like the vector kernels they replace; this also makes the
// plain difference q*dq - k*dk accurate enough for the gate gradient.
//
// Block form, for query row i of sub-block I and key row j of sub-block J of a block (l = gate prefix in the
// sub-block, tau_m = sub-block totals, r_m = e^{tau_m}, s = tau - l):
//   dq_i = e^{l_i} ((((S_in do_i) r_0 + G_0) r_1 + G_1) ... r_{I-1} + G_{I-1}) + e^{-s_i} G_I' + dA_ii k_i
//          G_J = sum_{j in J} dA_ij (k e^{s})_j,  G_I' the same over j < i of the own sub-block,  dA = dO V^T
// with the dyadic levels of the reference replacing the G_I' term when the gates of the sub-block are hard.
#include "gla_recurrent_stream_bwd.hpp"
#include "gla_recurrent_stream.hpp"

namespace gla {

typedef __bf16 BT;

// ---------------------------------------------------------------------------------------------------
// sweep 1
// ---------------------------------------------------------------------------------------------------
// WIDE: dq is a float array (head dimension 256 adds two such runs and rounds once, gla_split.hip)
template <typename TO, int C, int D, bool WIDE>
__global__ __launch_bounds__(C * 4) void recurrent_stream_dq_kernel(
    const void *__restrict__ h0, const float *__restrict__ g, const BT *__restrict__ v, const BT *__restrict__ k,
    const BT *__restrict__ q, const void *__restrict__ dhT, const TO *__restrict__ dout,
    std::conditional_t<WIDE, float, BT> *__restrict__ dq, float *__restrict__ qdq, int T_len, int H, int reverse,
    int hdt)
{
    typedef BT T;
    typedef std::conditional_t<WIDE, float, BT> TG;
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4, NT = D / 16, RT = NT / NB;
    static_assert(NT % NB == 0, "every wave owns the same number of state row tiles");
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    typedef FragTypes<T>::d8 D8;
    typedef FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *Vn = reinterpret_cast<T *>(smem);           // [C][LS]  value
    T *Kh = Vn + C * LS;                           // [C][LS]  k * exp(tau_J - l_j), bf16 head
    T *Kl = Kh + C * LS;                           // [C][LS]  ... and remainder
    T *Sh = Kl + C * LS;                           // [D][LS]  state at the start of the block, [dk][dv], head
    T *Sl = Sh + D * LS;                           // [D][LS]  ... and remainder
    T *xs = Sl + D * LS;                           // [NB][2][16][XS] per-wave scratch (hard gates only)
    float *rtab = reinterpret_cast<float *>(xs + NB * 2 * 16 * XS);   // [NB][D] exp(tau_m)
    constexpr bool kSplitDout = sizeof(TO) == 4;   // an fp32 dout enters the products as bf16 head + remainder

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, c = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y;
    const int64_t seq = ((int64_t)b * T_len * H + h) * D;
    const int64_t rowstride = (int64_t)H * D;
    const int64_t bh = (int64_t)b * H + h;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const TrLane<T> Lx = make_tr_lane<T>(XS);
    const int ptl = plain_tr_lane<T>(LS);
    const int wrow = 16 * w * LS + L.nat;
    T *xh = xs + (2 * w) * 16 * XS, *xl = xh + 16 * XS;
    const int N = (T_len + C - 1) / C;

    // state: S[i][nt][e] = state[dk = 16nt + r][dv = 16(w + i NB) + 4c + e]
    f32x4 S[RT][NT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float t4[4];
            load_hidden<4>(h0, hdt, bh * D * D + (int64_t)(16 * nt + r) * D + 16 * (w + i * NB) + 4 * c, t4);
            S[i][nt] = f32x4{t4[0], t4[1], t4[2], t4[3]};
        }
    auto publish_state = [&]() {
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                T4 hi, lo;
                split4<T>(S[i][nt], hi, lo);
                const int off = (16 * nt + r) * LS + 16 * (w + i * NB) + 4 * c;
                *reinterpret_cast<T4 *>(Sh + off) = hi;
                *reinterpret_cast<T4 *>(Sl + off) = lo;
            }
    };
    publish_state();

    f32x8 gN[KS];
    D8 qN[KS], kN[KS], vN[KS];
    DoutRow<TO> dN[KS];
    bool validN;
    int64_t rowN;
    auto fetch = [&](int n) {
        const int s = n * C + 16 * w + r;
        validN = s < T_len;
        const int sc = validN ? s : T_len - 1;
        rowN = seq + (int64_t)(reverse ? T_len - 1 - sc : sc) * rowstride;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            gN[ks] = ld8(g + rowN + 32 * ks + 8 * c);
            qN[ks] = ld8(q + rowN + 32 * ks + 8 * c);
            kN[ks] = ld8(k + rowN + 32 * ks + 8 * c);
            vN[ks] = ld8(v + rowN + 32 * ks + 8 * c);
            dN[ks].load(dout + rowN + 32 * ks + 8 * c);
        }
    };
    fetch(0);

#pragma unroll 1
    for (int n = 0; n < N; ++n) {
        const bool valid = validN;
        const int64_t row = rowN;
        float p[NV], dqo[NV];                // l_i; the own sub-block's part of dq (already scaled)
        D8 qf[KS], kf[KS], dof[KS], dofl[KS];   // dofl: what the bf16 rounding of an fp32 dout row leaves over
        T4 lowTh, lowTl;                     // dA^T of the own sub-block below the diagonal (one anchor)
        bool one_anchor;
        {
            D8 vf[KS];
            if ((n + 1) * C > T_len && !valid) {   // only the last block can hold padded steps
                float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    gN[ks] = pack8<float>(z);
                    qN[ks] = kN[ks] = vN[ks] = pack8<T>(z);
                    dN[ks].zero();
                }
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) p[8 * ks + e] = gN[ks].v[e] * kLog2e;
                qf[ks] = qN[ks];
                kf[ks] = kN[ks];
                vf[ks] = vN[ks];
                dof[ks] = dN[ks].operand();
                if constexpr (kSplitDout) dofl[ks] = dN[ks].remainder();
                st8(Vn + wrow + 32 * ks, vf[ks]);
            }

            // dAt[e] = dA[i = r][j = 4c+e], dAn[e] = dA[i = 4c+e][j = r]  (dA = dO V^T: exact products of bf16)
            f32x4 dAn = {0.f, 0.f, 0.f, 0.f}, dAt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if constexpr (kSplitDout) {
                    dAn = mma_d(dofl[ks], vf[ks], dAn);
                    dAt = mma_d(vf[ks], dofl[ks], dAt);
                }
                dAn = mma_d(dof[ks], vf[ks], dAn);
                dAt = mma_d(vf[ks], dof[ks], dAt);
            }
            float dd = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
            dd = reduce_over_cgroups(dd);

            // gate prefix, totals through the wave's table row, one anchor or not
            float *rt = rtab + w * D;
#pragma unroll
            for (int i = 0; i < NV; ++i) p[i] = prefix_sum_rows(p[i]);
            if (r == 15) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) st8(rt + 32 * ks + 8 * c, pack8<float>(p + 8 * ks));
            }
            asm volatile("" ::: "memory");
            float span = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 tau = ld8(rt + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    span = fmaxf(span, fmaxf(fabsf(p[8 * ks + e]), fabsf(tau.v[e] - p[8 * ks + e])));
            }
            one_anchor = wave_all_below(span, kOneAnchorSpan);

            if (one_anchor) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    f32x8 tau = ld8(rt + 32 * ks + 8 * c);
                    float bq[8];
                    unpack8(kf[ks], bq);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        dqo[8 * ks + e] = dd * bq[e];                       // diagonal term (gla.py:1181-1185)
                        bq[e] *= fast_exp2(tau.v[e] - p[8 * ks + e]);
                    }
                    D8 kh, kl;
                    split8<T>(bq, kh, kl);
                    st8(Kh + wrow + 32 * ks, kh);
                    st8(Kl + wrow + 32 * ks, kl);
                }
                asm volatile("" ::: "memory");
                if (r == 0) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        f32x8 tau = ld8(rt + 32 * ks + 8 * c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) tau.v[e] = fast_exp2(tau.v[e]);
                        st8(rt + 32 * ks + 8 * c, tau);
                    }
                }
                f32x4 lowT;
#pragma unroll
                for (int e = 0; e < 4; ++e) lowT[e] = (4 * c + e < r) ? dAt[e] : 0.f;
                split4<T>(lowT, lowTh, lowTl);
            } else {
                // hard gates: the dyadic levels, 32 features at a time, inputs fetched again
                const float live = valid ? 1.f : 0.f;
#pragma unroll 1
                for (int ks = 0; ks < KS; ++ks) {
                    const HardSliceDq hs = hard_slice_dq<XS>(
                        g + row + 32 * ks + 8 * c, q + row + 32 * ks + 8 * c, k + row + 32 * ks + 8 * c, live, dd, dAt, dAn,
                        (LdsBT)xh, (LdsBT)xl, Lx.nat, Lx.k4, (LdsF32)(rt + 32 * ks + 8 * c), (LdsBT)(Kh + wrow + 32 * ks),
                        (LdsBT)(Kl + wrow + 32 * ks));
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        p[8 * ks + e] = hs.p8[e];
                        dqo[8 * ks + e] = hs.dq8[e];
                    }
                }
                lowTh = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
                lowTl = lowTh;
            }
        }
        __syncthreads();                     // tiles of this block and the published state are in place

        // dA^T of the pairs with the earlier sub-blocks, [j][i] = v_j . do_i: they do not depend on the feature
        T4 dah[NB], dal[NB];
#pragma unroll
        for (int J = 0; J < NB - 1; ++J) {
            f32x4 da = {0.f, 0.f, 0.f, 0.f};
            if (J < w) {
#pragma unroll
                for (int k2 = 0; k2 < KS; ++k2) {
                    const D8 vj = ld8(Vn + L.nat + 16 * J * LS + 32 * k2);
                    if constexpr (kSplitDout) da = mma_d(vj, dofl[k2], da);
                    da = mma_d(vj, dof[k2], da);
                }
            }
            split4<T>(da, dah[J], dal[J]);
        }

        // ---- dq chain: state term, then the earlier sub-blocks in ascending order, then the own one --------
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int fo = 32 * ks;
            if (KS > 2) __builtin_amdgcn_sched_barrier(0);   // one slice's operands at a time (register pressure)
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    acc[tt] = mma_d(ld8(Sl + L.own + (fo + 4 * tt) * LS + 32 * k2), dof[k2], acc[tt]);
                    const D8 sh = ld8(Sh + L.own + (fo + 4 * tt) * LS + 32 * k2);
                    if constexpr (kSplitDout) acc[tt] = mma_d(sh, dofl[k2], acc[tt]);
                    acc[tt] = mma_d(sh, dof[k2], acc[tt]);
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
                        acc[tt] = mma_t_split(lds_tr4(Kh + L.k4 + fo + 4 * tt + 16 * J * LS, LS),
                                              lds_tr4(Kl + L.k4 + fo + 4 * tt + 16 * J * LS, LS), dah[J], dal[J],
                                              acc[tt]);
                    }
                }
            }
            f32x4 gq[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            if (one_anchor) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    gq[tt] = mma_t_split(lds_tr4(Kh + L.k4 + fo + 4 * tt + 16 * w * LS, LS),
                                         lds_tr4(Kl + L.k4 + fo + 4 * tt + 16 * w * LS, LS), lowTh, lowTl, gq[tt]);
            }
            float o[8], a[8];
            f32x8 rw = ld8(rtab + w * D + fo + 8 * c);       // e^{tau}: e^{-s} = e^{l} / e^{tau}
            unpack8(qf[ks], a);
            f32x8 prod;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float el = fast_exp2(p[8 * ks + e]);
                const float es = one_anchor ? el * __builtin_amdgcn_rcpf(rw.v[e]) : 0.f;
                o[e] = el * acc[e >> 2][e & 3] + es * gq[e >> 2][e & 3] + dqo[8 * ks + e];
                prod.v[e] = a[e] * o[e];
            }
            if (valid) {
                st8(dq + row + fo + 8 * c, pack8<TG>(o));
                st8(qdq + row + fo + 8 * c, prod);
            }
        }

        // the next block's rows are requested only here (see sweep 2)
        if (n + 1 < N) fetch(n + 1);

        // ---- state update: S <- S e^{tau_J} + V_J^T (k e^{tau_J - l})_J over the sub-blocks in order ------
#pragma unroll
        for (int J = 0; J < NB; ++J) {
            float rr[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) rr[nt] = rtab[J * D + 16 * nt + r];
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                auto va = lds_tr4(Vn + ptl + 16 * J * LS + 16 * (w + i * NB), LS);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) S[i][nt][e] *= rr[nt];
                    S[i][nt] = mma_t(va, lds_tr4(Kl + ptl + 16 * J * LS + 16 * nt, LS), S[i][nt]);
                    S[i][nt] = mma_t(va, lds_tr4(Kh + ptl + 16 * J * LS + 16 * nt, LS), S[i][nt]);
                }
            }
        }
        __syncthreads();
        publish_state();
    }

    // The last term of gla.py:263, sum_v dhT * hT per key feature, from the state this sweep ends with (just
    // published as bf16 head + remainder: 16 bits of mantissa, where the stored hidden_final has 8).  Every
    // d(log_fgate)_t is a sum over the steps s >= t, so the term is added to q*dq of the LAST step and
    // reaches all of them through sweep 2's running sum.
    __syncthreads();           // the published state and every q*dq row are in place
    {
        constexpr int LPF = C * 4 / D;                                   // lanes per key feature: 4 or 2
        static_assert(LPF == 4 || LPF == 2, "a quad or a pair of lanes shares a key feature");
        const int d = threadIdx.x / LPF, part = threadIdx.x % LPF;       // each takes D / LPF of the row
        const int64_t dpo = bh * D * D + (int64_t)d * D + part * (D / LPF);
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < D / LPF; j += 8) {
            float dv8[8], sh[8], sl[8];
            load_hidden<8>(dhT, hdt, dpo + j, dv8);
            unpack8(ld8(Sh + d * LS + part * (D / LPF) + j), sh);
            unpack8(ld8(Sl + d * LS + part * (D / LPF) + j), sl);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc += dv8[e] * (sh[e] + sl[e]);
        }
        acc += dpp_f32<kDppQuadXor1>(acc);
        if (LPF == 4) acc += dpp_f32<kDppQuadXor2>(acc);
        if (part == 0) {
            float *lp = qdq + seq + (int64_t)(reverse ? 0 : T_len - 1) * rowstride + d;
            *lp += acc;
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// sweep 2: against the forward's direction, dS in accumulator registers.  For key row j of sub-block J:
//   dv_j = sum_{i >= j} A_ij do_i + dS'^T (k e^{Lend - L})_j
//   dk_j = e^{s_j} ((((dS' v_j) r_{NB-1} + H_{NB-1}) r_{NB-2} + ...) r_{J+1} + H_{J+1}) + e^{s_j} H_J' + dA_jj q_j
//          H_I = sum_{i in I} dA_ij (q e^{l})_i,  H_J' = sum_{i > j, own sub-block} dA_ij q_i e^{-s_i}
//   dS_in = diag(e^{Lend}) dS' + sum_i (q e^{L})_i do_i^T     (a Horner chain over the sub-blocks, last first)
// dS' is the gradient w.r.t. the state after the block.
// ---------------------------------------------------------------------------------------------------
// WIDE: dv and dk are float arrays (see sweep 1)
template <typename TO, int C, int D, bool WIDE>
__global__ __launch_bounds__(C * 4) void recurrent_stream_rev_kernel(
    const float *__restrict__ g, const BT *__restrict__ v, const BT *__restrict__ k, const BT *__restrict__ q,
    const void *__restrict__ dhT, const TO *__restrict__ dout, void *__restrict__ dh0,
    float *__restrict__ dg, std::conditional_t<WIDE, float, BT> *__restrict__ dv,
    std::conditional_t<WIDE, float, BT> *__restrict__ dk, int T_len, int H, int reverse, int hdt)
{
    typedef BT T;
    typedef std::conditional_t<WIDE, float, BT> TG;
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4, NT = D / 16, RT = NT / NB;
    static_assert(NT % NB == 0, "every wave owns the same number of state row tiles");
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    typedef FragTypes<T>::d8 D8;
    typedef FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *tO = reinterpret_cast<T *>(smem);           // [C][LS]  dout
    T *Qh = tO + C * LS;                           // [C][LS]  q * exp(l_i), bf16 head
    T *Ql = Qh + C * LS;                           // [C][LS]  ... and remainder
    // dS' is kept in ONE orientation, [dv][dk] (head / remainder): the product that contracts over dk reads its
    // rows, the one that contracts over dv reads it transposed, 16 dv rows per MFMA.
    T *DTh = Ql + C * LS;                          // [D][LS]
    T *DTl = DTh + D * LS;
    T *xs = DTl + D * LS;                          // [NB][2][16][XS] per-wave scratch
    float *rtab = reinterpret_cast<float *>(xs + NB * 2 * 16 * XS);   // [NB][D] exp(tau_m)
    float *dltab = rtab + NB * D;                  // [NB][D] sub-block sums of q*dq - k*dk
    float *runtab = dltab + NB * D;                // [2][D]  sum over the later blocks of q*dq - k*dk, double-buffered
    constexpr bool kSplitDout = sizeof(TO) == 4;   // an fp32 dout enters the products as bf16 head + remainder
    T *tOl = reinterpret_cast<T *>(runtab + 2 * D);   // [C][LS]  the remainder of dout (fp32 dout only)

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, c = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y;
    const int64_t seq = ((int64_t)b * T_len * H + h) * D;
    const int64_t rowstride = (int64_t)H * D;
    const int64_t bh = (int64_t)b * H + h;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const TrLane<T> Lx = make_tr_lane<T>(XS);
    const int ptl = plain_tr_lane<T>(LS);
    const int wrow = 16 * w * LS + L.nat;
    T *xh = xs + (2 * w) * 16 * XS, *xl = xh + 16 * XS;
    const int N = (T_len + C - 1) / C;

    // dS: DS[i][nt][e] = dS[dk = 16(w + i NB) + 4c + e][dv = 16nt + r]
    f32x4 DS[RT][NT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                DS[i][nt][e] = load_hidden1(dhT, hdt, bh * D * D + (int64_t)(16 * (w + i * NB) + 4 * c + e) * D + 16 * nt + r);
    auto publish = [&]() {
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                T4 hi, lo;
                split4<T>(DS[i][nt], hi, lo);
                const int dk0 = 16 * (w + i * NB) + 4 * c, dvc = 16 * nt + r;
                *reinterpret_cast<T4 *>(DTh + dvc * LS + dk0) = hi;
                *reinterpret_cast<T4 *>(DTl + dvc * LS + dk0) = lo;
            }
    };
    publish();
    // the running sum over the later blocks is the same for all rows: it lives in LDS, block n reads buffer
    // n & 1 and wave 0 writes the other one, so readers and the writer never meet between two barriers
    for (int d = threadIdx.x; d < 2 * D; d += C * 4) runtab[d] = 0.f;

    f32x8 gN[KS];
    D8 qN[KS], kN[KS], vN[KS];
    DoutRow<TO> dN[KS];
    bool validN;
    int64_t rowN;
    auto fetch = [&](int n) {
        const int s = n * C + 16 * w + r;
        validN = s < T_len;
        const int sc = validN ? s : T_len - 1;
        rowN = seq + (int64_t)(reverse ? T_len - 1 - sc : sc) * rowstride;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            gN[ks] = ld8(g + rowN + 32 * ks + 8 * c);
            qN[ks] = ld8(q + rowN + 32 * ks + 8 * c);
            kN[ks] = ld8(k + rowN + 32 * ks + 8 * c);
            vN[ks] = ld8(v + rowN + 32 * ks + 8 * c);
            dN[ks].load(dout + rowN + 32 * ks + 8 * c);
        }
    };
    fetch(N - 1);

#pragma unroll 1
    for (int n = N - 1; n >= 0; --n) {
        const bool valid = validN;
        const int64_t row = rowN;
        float sv[NV], dko[NV], kt[NV], qdq[NV];  // tau - l_i; own sub-block's part of dk; k e^{s}; q*dq
        D8 qf[KS], kf[KS], vf[KS], dof[KS];
        f32x4 Aown = {0.f, 0.f, 0.f, 0.f};       // scores A[i = 4c+e][j = r] of the own sub-block
        T4 lowh, lowl;                           // dA of the own sub-block below the diagonal (one anchor)
        f32x4 dAn = {0.f, 0.f, 0.f, 0.f}, dAt = {0.f, 0.f, 0.f, 0.f};
        bool one_anchor;
        float dd = 0.f;
        {
            float p[NV];
            if ((n + 1) * C > T_len && !valid) {   // only the last block can hold padded steps
                float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    gN[ks] = pack8<float>(z);
                    qN[ks] = kN[ks] = vN[ks] = pack8<T>(z);
                    dN[ks].zero();
                }
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    p[8 * ks + e] = gN[ks].v[e] * kLog2e;
                }
                qf[ks] = qN[ks];
                kf[ks] = kN[ks];
                vf[ks] = vN[ks];
                dof[ks] = dN[ks].operand();
                st8(tO + wrow + 32 * ks, dof[ks]);
                if constexpr (kSplitDout) {
                    const D8 dofl = dN[ks].remainder();
                    st8(tOl + wrow + 32 * ks, dofl);
                    dAn = mma_d(dofl, vf[ks], dAn);
                    dAt = mma_d(vf[ks], dofl, dAt);
                }
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                dAn = mma_d(dof[ks], vf[ks], dAn);
                dAt = mma_d(vf[ks], dof[ks], dAt);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
            dd = reduce_over_cgroups(dd);

            float *rt = rtab + w * D;
#pragma unroll
            for (int i = 0; i < NV; ++i) p[i] = prefix_sum_rows(p[i]);
            if (r == 15) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) st8(rt + 32 * ks + 8 * c, pack8<float>(p + 8 * ks));
            }
            asm volatile("" ::: "memory");
            float span = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 tau = ld8(rt + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    sv[8 * ks + e] = tau.v[e] - p[8 * ks + e];
                    span = fmaxf(span, fmaxf(fabsf(p[8 * ks + e]), fabsf(sv[8 * ks + e])));
                }
            }
            one_anchor = wave_all_below(span, kOneAnchorSpan);

            float dot = 0.f;
            if (one_anchor) {
                asm volatile("" ::: "memory");
                if (r == 0) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        f32x8 tau = ld8(rt + 32 * ks + 8 * c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) tau.v[e] = fast_exp2(tau.v[e]);
                        st8(rt + 32 * ks + 8 * c, tau);
                    }
                }
                f32x4 low;
#pragma unroll
                for (int e = 0; e < 4; ++e) low[e] = (4 * c + e > r) ? dAn[e] : 0.f;
                split4<T>(low, lowh, lowl);
                f32x4 G = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    float a[8], bq[8], qo[8], qe[8];
                    unpack8(qf[ks], a);
                    unpack8(kf[ks], bq);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        dot += a[e] * bq[e];
                        dko[8 * ks + e] = dd * a[e];
                        qo[e] = a[e] * fast_exp2(-sv[8 * ks + e]);
                        qe[e] = a[e] * fast_exp2(p[8 * ks + e]);
                        kt[8 * ks + e] = bq[e] * fast_exp2(sv[8 * ks + e]);
                    }
                    D8 h8, l8, oh, ol, kh, kl;
                    split8<T>(qe, h8, l8);
                    st8(Qh + wrow + 32 * ks, h8);
                    st8(Ql + wrow + 32 * ks, l8);
                    split8<T>(qo, oh, ol);
                    split8<T>(kt + 8 * ks, kh, kl);
                    G = mma_d_split(oh, ol, kh, kl, G);
                    // own link of dk: H'^T[dk][j] = sum_{i > j} (q e^{-s})_i[dk] dA_ij, through the wave's scratch
                    st8(xh + Lx.nat, oh);
                    st8(xl + Lx.nat, ol);
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
                        f32x4 hk = {0.f, 0.f, 0.f, 0.f};
                        hk = mma_t_split(lds_tr4(xh + Lx.k4 + 4 * tt, XS), lds_tr4(xl + Lx.k4 + 4 * tt, XS), lowh, lowl,
                                         hk);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            dko[8 * ks + 4 * tt + e] += hk[e] * fast_exp2(sv[8 * ks + 4 * tt + e]);
                    }
                    asm volatile("" ::: "memory");
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) Aown[e] = (4 * c + e > r) ? G[e] : 0.f;
            } else {
                const float live = valid ? 1.f : 0.f;
                f32x4 Gl[4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll 1
                for (int ks = 0; ks < KS; ++ks) {
                    const HardSliceRev hs = hard_slice_rev<XS>(
                        g + row + 32 * ks + 8 * c, q + row + 32 * ks + 8 * c, k + row + 32 * ks + 8 * c, live, dd, dAt, dAn,
                        Gl[0], Gl[1], Gl[2], Gl[3], dot, (LdsBT)xh, (LdsBT)xl, Lx.nat, Lx.k4,
                        (LdsF32)(rt + 32 * ks + 8 * c), (LdsBT)(Qh + wrow + 32 * ks), (LdsBT)(Ql + wrow + 32 * ks));
#pragma unroll
                    for (int l = 0; l < 4; ++l) Gl[l] = hs.G[l];
                    dot = hs.dot;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        sv[8 * ks + e] = hs.s8[e];
                        dko[8 * ks + e] = hs.dk8[e];
                        kt[8 * ks + e] = hs.kt8[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int o = 4 * c + e;
                    float acc = 0.f;
#pragma unroll
                    for (int l = 0; l < 4; ++l) {
                        const int h_ = 1 << l;
                        const bool ok = ((o ^ r) < 2 * h_) && (o & h_) && !(r & h_);
                        acc += ok ? Gl[l][e] : 0.f;
                    }
                    Aown[e] = acc;
                }
                lowh = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
                lowl = lowh;
            }
            dot = reduce_over_cgroups(dot);
#pragma unroll
            for (int e = 0; e < 4; ++e) Aown[e] += (4 * c + e == r) ? dot : 0.f;   // A_ii = q_i.k_i (gla.py:983)
        }
        __syncthreads();                     // tiles of this block and the published dS' are in place
        // q*dq of the block's rows (sweep 1 left it in the d(log_fgate) buffer) is requested here, not with the
        // rest of the block: it is needed last, and is not held through the work above
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 t = ld8(dg + row + 32 * ks + 8 * c);
#pragma unroll
            for (int e = 0; e < 8; ++e) qdq[8 * ks + e] = valid ? t.v[e] : 0.f;
        }

        // ---- score blocks of the later sub-blocks: A_Ij (key side walked up by r_I) and dA_Ij ----------
        T4 Ach[NB], Acl[NB], dAh[NB], dAl[NB];
        D8 Kth[KS], Ktl[KS];                 // k e^{Lend - L_j}, head and remainder
        {
            float kch[NV];
#pragma unroll
            for (int i = 0; i < NV; ++i) kch[i] = kt[i];
#pragma unroll
            for (int I = 1; I < NB; ++I) {
                Ach[I] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
                Acl[I] = Ach[I];
                dAh[I] = Ach[I];
                dAl[I] = Ach[I];
                if (I > w) {
                    f32x4 a = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        D8 kh, kl;
                        split8<T>(kch + 8 * ks, kh, kl);
                        a = mma_d_split(ld8(Qh + L.nat + 16 * I * LS + 32 * ks), ld8(Ql + L.nat + 16 * I * LS + 32 * ks),
                                        kh, kl, a);
                        if constexpr (kSplitDout) da = mma_d(ld8(tOl + L.nat + 16 * I * LS + 32 * ks), vf[ks], da);
                        da = mma_d(ld8(tO + L.nat + 16 * I * LS + 32 * ks), vf[ks], da);
                        f32x8 rr = ld8(rtab + I * D + 32 * ks + 8 * c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) kch[8 * ks + e] *= rr.v[e];
                    }
                    split4<T>(a, Ach[I], Acl[I]);
                    split4<T>(da, dAh[I], dAl[I]);
                }
            }
            split4<T>(Aown, Ach[0], Acl[0]);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) split8<T>(kch + 8 * ks, Kth[ks], Ktl[ks]);
        }

#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int fo = 32 * ks;
            // -- dv slice: dS'^T K~ first, then the own and the later sub-blocks
            {
                f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
                for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt)
                        acc[tt] = mma_d_split(ld8(DTh + L.own + (fo + 4 * tt) * LS + 32 * k2),
                                              ld8(DTl + L.own + (fo + 4 * tt) * LS + 32 * k2), Kth[k2], Ktl[k2], acc[tt]);
                }
#pragma unroll
                for (int I = 0; I < NB; ++I) {
                    if (I >= w) {
                        const T4 bh4 = I == w ? Ach[0] : Ach[I], bl4 = I == w ? Acl[0] : Acl[I];
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
                if (valid) st8(dv + row + fo + 8 * c, pack8<TG>(o));
            }
            // -- dk slice: dS' v first, then the later sub-blocks in descending order
            {
                f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
                // (dS' v)[dk][j] = sum_dv dS'[dk][dv] v_j[dv]: 16 dv rows per step, read transposed.  Step (k2,
                // half) contracts over dv = 32 k2 + 8 c + 4 half + m, which is what lane (j, c) holds of v_j.
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
                    if (I > w) {
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
                float o[8], kk[8];
                unpack8(kf[ks], kk);
                f32x8 sfx;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    o[e] = fast_exp2(sv[8 * ks + e]) * acc[e >> 2][e & 3] + dko[8 * ks + e];
                    // q*dq - k*dk of the row, then its reverse running sum inside the sub-block
                    sfx.v[e] = suffix_sum_rows(qdq[8 * ks + e] - kk[e] * o[e]);
                    qdq[8 * ks + e] = sfx.v[e];
                }
                if (valid) st8(dk + row + fo + 8 * c, pack8<TG>(o));
                if (r == 0) st8(dltab + w * D + fo + 8 * c, sfx);
            }
        }

        // The next block's rows are requested only here: the registers that receive them are not held through
        // the chains above, and the update below is long enough for them to arrive.
        if (n > 0) fetch(n - 1);

        // ---- dS <- dS r_I + (q e^{l})_I^T dO_I over the sub-blocks, last first ---------------------------
#pragma unroll
        for (int I = NB - 1; I >= 0; --I) {
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const f32x4 rr = *reinterpret_cast<const f32x4 *>(rtab + I * D + 16 * (w + i * NB) + 4 * c);
                const T4 qah = lds_tr4(Qh + ptl + 16 * I * LS + 16 * (w + i * NB), LS);
                const T4 qal = lds_tr4(Ql + ptl + 16 * I * LS + 16 * (w + i * NB), LS);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) DS[i][nt][e] *= rr[e];
                    const T4 ob = lds_tr4(tO + ptl + 16 * I * LS + 16 * nt, LS);
                    DS[i][nt] = mma_t(qal, ob, DS[i][nt]);
                    if constexpr (kSplitDout)
                        DS[i][nt] = mma_t(qah, lds_tr4(tOl + ptl + 16 * I * LS + 16 * nt, LS), DS[i][nt]);
                    DS[i][nt] = mma_t(qah, ob, DS[i][nt]);
                }
            }
        }
        __syncthreads();                     // sub-block sums complete; every wave is done with the tiles
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 o, tot = ld8(runtab + (n & 1) * D + 32 * ks + 8 * c);
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] = qdq[8 * ks + e] + tot.v[e];
#pragma unroll
            for (int m = 0; m < NB; ++m) {
                f32x8 t = ld8(dltab + m * D + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    o.v[e] += m > w ? t.v[e] : 0.f;
                    tot.v[e] += t.v[e];
                }
            }
            if (w == 0 && r == 0) st8(runtab + ((n & 1) ^ 1) * D + 32 * ks + 8 * c, tot);
            if (valid) st8(dg + row + 32 * ks + 8 * c, o);
        }
        publish();
    }

#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                store_hidden1(dh0, hdt, bh * D * D + (int64_t)(16 * (w + i * NB) + 4 * c + e) * D + 16 * nt + r, DS[i][nt][e]);
}

template <typename TO, int C, int D, bool WIDE>
static int launch_dq(hipStream_t st, int B, int T_len, int H, int reverse, int hdt, const void *h0, const float *g,
                     const void *v, const void *k, const void *q, const void *dhT, const void *dout, void *dq,
                     float *qdq)
{
    typedef BT T;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    const size_t lds = ((size_t)(3 * C + 2 * D) * LS + (size_t)(C / 16) * 2 * 16 * XS) * sizeof(T) +
                       (size_t)(C / 16) * D * sizeof(float);
    auto kern = recurrent_stream_dq_kernel<TO, C, D, WIDE>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, h0, g, (const T *)v, (const T *)k, (const T *)q,
                       dhT, (const TO *)dout, (std::conditional_t<WIDE, float, T> *)dq, qdq, T_len, H, reverse, hdt);
    return launch_status();
}

template <typename TO, int C, int D, bool WIDE>
static int launch_rev(hipStream_t st, int B, int T_len, int H, int reverse, int hdt, const float *g, const void *v,
                      const void *k, const void *q, const void *dhT, const void *dout, void *dh0,
                      float *dg, void *dv, void *dk)
{
    typedef BT T;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int XS = 32 + 16 / (int)sizeof(T);
    const size_t lds = ((size_t)(3 * C + 2 * D + (sizeof(TO) == 4 ? C : 0)) * LS + (size_t)(C / 16) * 2 * 16 * XS) *
                           sizeof(T) +
                       (size_t)(2 * (C / 16) + 2) * D * sizeof(float);
    auto kern = recurrent_stream_rev_kernel<TO, C, D, WIDE>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)v, (const T *)k, (const T *)q,
                       dhT, (const TO *)dout, dh0, dg, (std::conditional_t<WIDE, float, T> *)dv,
                       (std::conditional_t<WIDE, float, T> *)dk, T_len, H, reverse, hdt);
    return launch_status();
}

int launch_recurrent_stream_rev(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                                const float *g, const void *v, const void *k, const void *q, const void *dhT,
                                const void *dout, void *dh0, float *dg, void *dv, void *dk, int wide)
{
    if (D == 64 && !wide)
        return launch_recurrent_stream_rev2(st, B, T_len, H, D, reverse, hdt, dout_f32, g, v, k, q, dhT, dout, dh0, dg,
                                            dv, dk);
    if (D != 128) return GLA_ERR_UNSUPPORTED;
    if (wide)
        return dout_f32
                   ? launch_rev<float, 64, 128, true>(st, B, T_len, H, reverse, hdt, g, v, k, q, dhT, dout, dh0, dg, dv, dk)
                   : launch_rev<BT, 64, 128, true>(st, B, T_len, H, reverse, hdt, g, v, k, q, dhT, dout, dh0, dg, dv, dk);
    return dout_f32 ? launch_rev<float, 64, 128, false>(st, B, T_len, H, reverse, hdt, g, v, k, q, dhT, dout, dh0, dg, dv, dk)
                    : launch_rev<BT, 64, 128, false>(st, B, T_len, H, reverse, hdt, g, v, k, q, dhT, dout, dh0, dg, dv, dk);
}

int launch_recurrent_stream_dq(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                               const void *h0, const float *g, const void *v, const void *k, const void *q,
                               const void *dhT, const void *dout, void *dq, float *qdq, int wide)
{
    if (D == 64 && !wide)
        return launch_recurrent_stream_dq2(st, B, T_len, H, D, reverse, hdt, dout_f32, h0, g, v, k, q, dhT, dout, dq,
                                           qdq);
    if (D != 128) return GLA_ERR_UNSUPPORTED;
    if (wide)
        return dout_f32
                   ? launch_dq<float, 64, 128, true>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, dhT, dout, dq, qdq)
                   : launch_dq<BT, 64, 128, true>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, dhT, dout, dq, qdq);
    return dout_f32 ? launch_dq<float, 64, 128, false>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, dhT, dout, dq, qdq)
                    : launch_dq<BT, 64, 128, false>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, dhT, dout, dq, qdq);
}

}  // namespace gla
