// The gated causal scores of ONE 16-token sub-block (one wave), forward side, and the rescaled operands
// the rest of a chunk needs from it (gla.py:964-1029 restricted to a leaf of 16 tokens).
//
// With l_i the inclusive gate sum inside the sub-block (log2 units) and tau its total, the wave produces
//   accD[e]  = A[i = r][j = 4c+e] transposed, i.e. element (key j = 4c+e, query i = r) of the sub-block's
//              scores A_ij = sum_d q_id k_jd e^{l_id - l_jd} (j < i), the plain dot q_i.k_i on the diagonal;
//   qh       = q_i e^{l_i}          (fp32, row layout), the query operand against earlier sub-blocks / the state;
//   kh row   = k_j e^{tau - l_j}    (element type, written to the lane's row of an LDS tile; kl row, if asked
//              for, receives what that rounding leaves over, again in the element type);
//   rt       = e^{tau}              (fp32, the wave's row of a table in LDS).
// Mild gates take ONE anchor (the end of the sub-block), harder ones the dyadic levels 16/8/4/2 of the
// reference; see kOneAnchorSpan.
#pragma once

#include "gla_chunk_common.hpp"

namespace gla {

// Head and remainder of 8 values in the element type: x = hi + lo up to 16 bits of mantissa for bf16.
template <typename T>
__device__ __forceinline__ void split8(const float *x, typename FragTypes<T>::d8 &hi, typename FragTypes<T>::d8 &lo)
{
    float h[8];
    hi = pack8<T>(x);
    unpack8(hi, h);
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = x[e] - h[e];
    lo = pack8<T>(h);
}
// a b^T with both operands given as head + remainder (the remainder x remainder term is dropped)
template <typename D8> __device__ __forceinline__ f32x4 mma_d_split(D8 ah, D8 al, D8 bh, D8 bl, f32x4 acc)
{
    acc = mma_d(al, bh, acc);
    acc = mma_d(ah, bl, acc);
    return mma_d(ah, bh, acc);
}

// The same for 4 accumulator values (a score block as the B operand of a token contraction).
template <typename T>
__device__ __forceinline__ void split4(f32x4 x, typename FragTypes<T>::t4 &hi, typename FragTypes<T>::t4 &lo)
{
    hi = pack4<T>(x);
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] -= (float)hi[e];
    lo = pack4<T>(x);
}
template <typename T4> __device__ __forceinline__ f32x4 mma_t_split(T4 ah, T4 al, T4 bh, T4 bl, f32x4 acc)
{
    acc = mma_t(al, bh, acc);
    acc = mma_t(ah, bl, acc);
    return mma_t(ah, bh, acc);
}

// Hard gates (a sub-block whose gate sums span 48 powers of two or more) are rare, and the dyadic levels need
// more registers than the one-anchor path.  Inlined, they count towards the registers of the whole kernel; as a
// real call, the registers they clobber are saved and restored around the call only, on the path that takes it.
// That pays where the kernel is not held to a register budget of its own (a budget binds the callee too, and
// the saves then land on the common path: the 128-register output kernel of chunk_gla went from 35 to 57 us).
struct HardSliceFwd {
    f32x4 G[4];
    float dot, qh8[8];
};
// One 32-feature slice of a hard sub-block, the loop body of the inlined form in subblock_forward: the levels'
// scores (added to G, one block per level), q.k (added to dot), e^{tau} of the slice into the table row (lane
// r == 0), the rescaled key rows into the tiles (LDS); returns q e^{l_i}.  The pointers are those of the lane's 8
// features of the slice.
template <typename T, bool PRECISE>
__device__ __attribute__((noinline)) HardSliceFwd hard_slice_fwd(
    const float *gp, const T *qp, const T *kp, float live, f32x4 G0, f32x4 G1, f32x4 G2, f32x4 G3, float dot,
    __attribute__((address_space(3))) float *rt3, __attribute__((address_space(3))) T *kh3, bool write_kh,
    __attribute__((address_space(3))) T *kl3, bool write_kl)
{
    typedef typename FragTypes<T>::d8 D8;
    const int r = threadIdx.x & 15;
    HardSliceFwd out;
    out.G[0] = G0; out.G[1] = G1; out.G[2] = G2; out.G[3] = G3;
    float p8[8], s8[8], a[8], bq[8];
    {
        f32x8 gg = ld8(gp);
        unpack8(ld8(qp), a);
        unpack8(ld8(kp), bq);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            p8[e] = gg.v[e] * kLog2e * live;
            s8[e] = 0.f;
            a[e] *= live;
            bq[e] *= live;
        }
    }
    auto level = [&](auto hc, auto lc) {
        constexpr int h_ = decltype(hc)::value, L_ = decltype(lc)::value;
        const bool upper = (r & h_) != 0;
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (upper ? a[e] : bq[e]) * fast_exp2(upper ? p8[e] : s8[e]);
        if constexpr (PRECISE) {
            D8 Xh, Xl;
            split8<T>(x, Xh, Xl);
            out.G[L_] = mma_d_split(Xh, Xl, Xh, Xl, out.G[L_]);
        } else {
            D8 X = pack8<T>(x);
            out.G[L_] = mma_d(X, X, out.G[L_]);
        }
        hier_step<h_>(p8, s8, upper);
    };
    level(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
    level(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
    level(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
    level(std::integral_constant<int, 8>{}, std::integral_constant<int, 3>{});
    // p8 = l_i, s8 = tau - l_i
    if (r == 0) {
        f32x8 t;
#pragma unroll
        for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(p8[e] + s8[e]);
        st8((float *)rt3, t);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        dot += a[e] * bq[e];
        out.qh8[e] = a[e] * fast_exp2(p8[e]);
        bq[e] *= fast_exp2(s8[e]);
    }
    out.dot = dot;
    D8 kh, kl;
    split8<T>(bq, kh, kl);
    if (write_kh) st8((T *)kh3, kh);
    if (write_kl) st8((T *)kl3, kl);
    return out;
}

// PRECISE: the score products take their operands as head + remainder, for callers that promise fp32
// arithmetic on bf16 inputs; kl_row must be given then.
// SCANNED: p already holds the inclusive prefix sums over the rows (the caller ran prefix_sum_rows).
// CALL_HARD: the hard-gate path is a call of hard_slice_fwd per slice instead of inlined code.
template <typename T, int D, bool PRECISE = false, bool SCANNED = false, bool CALL_HARD = false>
__device__ __forceinline__ void subblock_forward(float (&p)[D / 4],
                                                 const typename FragTypes<T>::d8 (&qf)[D / 32],
                                                 const typename FragTypes<T>::d8 (&kf)[D / 32],
                                                 const float *g_row, const T *q_row, const T *k_row, bool valid,
                                                 float *rt, T *kh_row, bool write_kh, T *kl_row, int r, int c,
                                                 f32x4 &accD,
                                                 float (&qh)[D / 4])
{
    constexpr int KS = D / 32, NV = D / 4;
    typedef typename FragTypes<T>::d8 D8;
    // p = l_i; the totals travel through the wave's own table row (same-wave LDS accesses execute in order)
    if constexpr (!SCANNED) {
#pragma unroll
        for (int i = 0; i < NV; ++i) p[i] = prefix_sum_rows(p[i]);
    }
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
    const bool one_anchor = wave_all_below(span, kOneAnchorSpan);

    // the hint keeps the register saves that the other branch needs out of this one (chunk_gla's output kernel,
    // held to 128 registers: 35.5 -> 33 us)
    if (__builtin_expect(one_anchor, true)) {
        float dot = 0.f;
        f32x4 G = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 tau = ld8(rt + 32 * ks + 8 * c);
            float a[8], bq[8], qo[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float s = tau.v[e] - p[8 * ks + e];
                dot += a[e] * bq[e];
                qo[e] = a[e] * fast_exp2(-s);
                qh[8 * ks + e] = a[e] * fast_exp2(p[8 * ks + e]);
                bq[e] *= fast_exp2(s);
            }
            D8 kh, kl;
            split8<T>(bq, kh, kl);
            if (write_kh) st8(kh_row + 32 * ks, kh);
            if (kl_row) st8(kl_row + 32 * ks, kl);
            if constexpr (PRECISE) {
                D8 oh, ol;
                split8<T>(qo, oh, ol);
                G = mma_d_split(kh, kl, oh, ol, G);
            } else {
                G = mma_d(kh, pack8<T>(qo), G);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        dot = reduce_over_cgroups(dot);
#pragma unroll
        for (int e = 0; e < 4; ++e) accD[e] = (4 * c + e < r) ? G[e] : ((4 * c + e == r) ? dot : 0.f);
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
    } else {
        // At level 2h rows in the upper half of their group carry q e^{prefix over the half}, rows in the
        // lower half k e^{suffix over the half}; one MFMA of that mixed tile with itself yields every block
        // of the level.  Walked 32 features at a time (the level's scores add up over the slices) with the
        // inputs fetched again, to keep the register footprint of this rare path small.
        f32x4 Gl[4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        float dot = 0.f;
        const float live = valid ? 1.f : 0.f;
        constexpr int kInlined = CALL_HARD ? 0 : KS;
        if constexpr (CALL_HARD) {
            typedef __attribute__((address_space(3))) T *LdsT;
#pragma unroll 1
            for (int ks = 0; ks < KS; ++ks) {
                const int fo = 32 * ks + 8 * c;
                const HardSliceFwd hs = hard_slice_fwd<T, PRECISE>(
                    g_row + fo, q_row + fo, k_row + fo, live, Gl[0], Gl[1], Gl[2], Gl[3], dot,
                    (__attribute__((address_space(3))) float *)(rt + fo), (LdsT)(kh_row + 32 * ks), write_kh,
                    (LdsT)(kl_row + 32 * ks), kl_row != nullptr);
#pragma unroll
                for (int l = 0; l < 4; ++l) Gl[l] = hs.G[l];
                dot = hs.dot;
#pragma unroll
                for (int e = 0; e < 8; ++e) qh[8 * ks + e] = hs.qh8[e];
            }
        }
#pragma unroll
        for (int ks = 0; ks < kInlined; ++ks) {
            float p8[8], s8[8], a[8], bq[8];
            {
                f32x8 gg = ld8(refetch(g_row) + 32 * ks + 8 * c);
                unpack8(ld8(refetch(q_row) + 32 * ks + 8 * c), a);
                unpack8(ld8(refetch(k_row) + 32 * ks + 8 * c), bq);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    p8[e] = gg.v[e] * kLog2e * live;
                    s8[e] = 0.f;
                    a[e] *= live;
                    bq[e] *= live;
                }
            }
            auto level = [&](auto hc, auto lc) {
                constexpr int h_ = decltype(hc)::value, L_ = decltype(lc)::value;
                const bool upper = (r & h_) != 0;
                float x[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (upper ? a[e] : bq[e]) * fast_exp2(upper ? p8[e] : s8[e]);
                if constexpr (PRECISE) {
                    D8 Xh, Xl;
                    split8<T>(x, Xh, Xl);
                    Gl[L_] = mma_d_split(Xh, Xl, Xh, Xl, Gl[L_]);
                } else {
                    D8 X = pack8<T>(x);
                    Gl[L_] = mma_d(X, X, Gl[L_]);
                }
                hier_step<h_>(p8, s8, upper);
            };
            level(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
            level(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
            level(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
            level(std::integral_constant<int, 8>{}, std::integral_constant<int, 3>{});
            // p8 = l_i, s8 = tau - l_i
            if (r == 0) {
                f32x8 t;
#pragma unroll
                for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(p8[e] + s8[e]);
                st8(rt + 32 * ks + 8 * c, t);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                dot += a[e] * bq[e];
                qh[8 * ks + e] = a[e] * fast_exp2(p8[e]);
                bq[e] *= fast_exp2(s8[e]);
            }
            {
                D8 kh, kl;
                split8<T>(bq, kh, kl);
                if (write_kh) st8(kh_row + 32 * ks, kh);
                if (kl_row) st8(kl_row + 32 * ks, kl);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        dot = reduce_over_cgroups(dot);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = 4 * c + e;
            float acc = (j == r) ? dot : 0.f;                      // plain fp32 dot on the diagonal (gla.py:983)
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                const int h_ = 1 << l;
                const bool ok = ((j ^ r) < 2 * h_) && (r & h_) && !(j & h_);
                acc += ok ? Gl[l][e] : 0.f;
            }
            accD[e] = acc;
        }
    }
}

}  // namespace gla
