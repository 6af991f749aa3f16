// Pieces shared by the recurrent_gla backward kernels (gla_recurrent_stream_bwd.hip: one wave per 16-step
// sub-block; gla_recurrent_stream_bwd2.hip: two waves per sub-block, each with half of the features): the dyadic
// levels of a sub-block with hard gates, one 32-feature slice at a time.
#pragma once

#include "gla_subblock.hpp"

namespace gla {

typedef __bf16 BT;

// Eight consecutive elements of a `dout` row on their way from memory to the bf16 tile the products read.  TO is
// the element type of `dout`: bf16 for recurrent_gla; float for the recurrent_gla_naive flavour, whose `out` is
// fp32 (gla.py:37) and so is its cotangent.  There the row enters every product as bf16 head + remainder (a second
// tile), like the other operands that are not bf16 numbers to begin with: with the head alone dvalue came out at
// 1.5 x its storage rounding.
template <typename TO> struct DoutRow;
template <> struct DoutRow<BT> {
    bf16x8 raw;
    __device__ __forceinline__ void load(const BT *p) { raw = ld8(p); }
    __device__ __forceinline__ void zero() { const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}; raw = pack8<BT>(z); }
    __device__ __forceinline__ bf16x8 operand() const { return raw; }
    __device__ __forceinline__ bf16x8 remainder() const { return raw; }   // never used: a bf16 row has none
};
template <> struct DoutRow<float> {
    f32x8 raw;
    __device__ __forceinline__ void load(const float *p) { raw = ld8(p); }
    __device__ __forceinline__ void zero() { const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}; raw = pack8<float>(z); }
    __device__ __forceinline__ bf16x8 operand() const { return pack8<BT>(raw.v); }
    __device__ __forceinline__ bf16x8 remainder() const
    {
        float lo[8];
        unpack8(pack8<BT>(raw.v), lo);
#pragma unroll
        for (int e = 0; e < 8; ++e) lo[e] = raw.v[e] - lo[e];
        return pack8<BT>(lo);
    }
};

// One level (half-width H) of the dyadic recursion of a 16-token sub-block on a 32-feature slice: the mixed
// tile X (upper rows q e^{prefix}, lower rows k e^{suffix}) goes through the wave's scratch, dX = (M + M^T) X
// with M the level's masked dA block; adds the query part (upper rows) to dq8 and/or the key part (lower
// rows) to dk8, and (WANT_G) the slice's share of the level's scores X X^T to G.  p8 / s8 are advanced to
// the next level.
template <int H, int XS, bool WANT_Q, bool WANT_K, bool WANT_G = false>
__device__ __forceinline__ void bwd_level(float (&p8)[8], float (&s8)[8], const float (&a)[8], const float (&bq)[8],
                                          f32x4 dAt, f32x4 dAn, BT *xh, BT *xl, int xnat, int xk4, int r, int c,
                                          float (&dq8)[8], float (&dk8)[8], f32x4 *G = nullptr)
{
    typedef FragTypes<BT>::d8 D8;
    typedef FragTypes<BT>::t4 T4;
    const bool upper = (r & H) != 0;
    f32x4 sym;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int o = 4 * c + e;                       // the other row
        const bool same = (o ^ r) < 2 * H;
        const bool o_up = (o & H) != 0;
        sym[e] = (same && upper && !o_up) ? dAt[e] : ((same && o_up && !upper) ? dAn[e] : 0.f);
    }
    T4 sh, sl;
    split4<BT>(sym, sh, sl);
    float fac[8], x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        fac[e] = fast_exp2(upper ? p8[e] : s8[e]);
        x[e] = (upper ? a[e] : bq[e]) * fac[e];
    }
    D8 Xh, Xl;
    split8<BT>(x, Xh, Xl);
    if (WANT_G) *G = mma_d_split(Xh, Xl, Xh, Xl, *G);
    st8(xh + xnat, Xh);
    st8(xl + xnat, Xl);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
        f32x4 dx = {0.f, 0.f, 0.f, 0.f};
        dx = mma_t_split(lds_tr4(xh + xk4 + 4 * tt, XS), lds_tr4(xl + xk4 + 4 * tt, XS), sh, sl, dx);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float z = dx[e] * fac[4 * tt + e];
            if (WANT_Q) dq8[4 * tt + e] += upper ? z : 0.f;
            if (WANT_K) dk8[4 * tt + e] += upper ? 0.f : z;
        }
    }
    asm volatile("" ::: "memory");
    hier_step<H>(p8, s8, upper);
}

// Hard gates are rare (a sub-block whose gate sums span 48 powers of two), and the dyadic levels need ~150
// registers more than the one-anchor path.  Inlined, they set the register count of the whole kernel; as a
// real call, the registers they clobber are saved and restored around the call only, on the path that takes it.
typedef __attribute__((address_space(3))) BT *LdsBT;
typedef __attribute__((address_space(3))) float *LdsF32;

struct HardSliceDq {
    float p8[8], dq8[8];
};
// One 32-feature slice of the own sub-block of sweep 1: dyadic levels (query part), e^{tau} of the slice into
// the table row (lane r == 0), the rescaled key rows into the tiles; returns l_i and the sub-block's part of dq.
// WRITE = false leaves the table and the tiles alone (the caller has filled them from the plain row scan).
template <int XS, bool WRITE = true>
__device__ __attribute__((noinline)) HardSliceDq hard_slice_dq(const float *gp, const BT *qp, const BT *kp, float live,
                                                               float dd, f32x4 dAt, f32x4 dAn, LdsBT xh3, LdsBT xl3,
                                                               int xnat, int xk4, LdsF32 rt3, LdsBT kh3, LdsBT kl3)
{
    typedef FragTypes<BT>::d8 D8;
    const int lane = threadIdx.x & 63, r = lane & 15, c = lane >> 4;
    BT *xh = (BT *)xh3, *xl = (BT *)xl3;
    HardSliceDq out;
    float s8[8], a[8], bq[8], dk8[8];
    f32x8 gg = ld8(gp);
    unpack8(ld8(qp), a);
    unpack8(ld8(kp), bq);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        out.p8[e] = gg.v[e] * kLog2e * live;
        s8[e] = 0.f;
        a[e] *= live;
        bq[e] *= live;
        out.dq8[e] = dd * bq[e];
    }
    bwd_level<1, XS, true, false>(out.p8, s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, out.dq8, dk8);
    bwd_level<2, XS, true, false>(out.p8, s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, out.dq8, dk8);
    bwd_level<4, XS, true, false>(out.p8, s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, out.dq8, dk8);
    bwd_level<8, XS, true, false>(out.p8, s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, out.dq8, dk8);
    // p8 = l_i, s8 = tau - l_i
    if constexpr (WRITE) {
        if (r == 0) {
            f32x8 t;
#pragma unroll
            for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(out.p8[e] + s8[e]);
            st8((float *)rt3, t);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) bq[e] *= fast_exp2(s8[e]);
        D8 kh, kl;
        split8<BT>(bq, kh, kl);
        st8((BT *)kh3, kh);
        st8((BT *)kl3, kl);
    }
    return out;
}

struct HardSliceRev {
    float s8[8], dk8[8], kt8[8];
    f32x4 G[4];
    float dot;
};
// The same for sweep 2: key part of the levels, the levels' scores (added to G, one block per level), q.k
// (added to dot), e^{tau} of the slice into the table row, the rescaled query rows (head, remainder) into the tiles;
// returns tau - l_i, the sub-block's part of dk and k e^{tau - l_i}.  WRITE = false leaves the table and the
// tiles alone.
template <int XS, bool WRITE = true>
__device__ __attribute__((noinline)) HardSliceRev hard_slice_rev(const float *gp, const BT *qp, const BT *kp, float live,
                                                                 float dd, f32x4 dAt, f32x4 dAn, f32x4 G0, f32x4 G1,
                                                                 f32x4 G2, f32x4 G3, float dot, LdsBT xh3, LdsBT xl3,
                                                                 int xnat, int xk4, LdsF32 rt3, LdsBT qh3, LdsBT ql3)
{
    typedef FragTypes<BT>::d8 D8;
    const int lane = threadIdx.x & 63, r = lane & 15, c = lane >> 4;
    BT *xh = (BT *)xh3, *xl = (BT *)xl3;
    HardSliceRev out;
    out.G[0] = G0; out.G[1] = G1; out.G[2] = G2; out.G[3] = G3;
    out.dot = dot;
    float p8[8], a[8], bq[8], dq8[8];
    f32x8 gg = ld8(gp);
    unpack8(ld8(qp), a);
    unpack8(ld8(kp), bq);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        p8[e] = gg.v[e] * kLog2e * live;
        out.s8[e] = 0.f;
        a[e] *= live;
        bq[e] *= live;
        out.dk8[e] = dd * a[e];
        out.dot += a[e] * bq[e];
    }
    bwd_level<1, XS, false, true, true>(p8, out.s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, dq8, out.dk8, &out.G[0]);
    bwd_level<2, XS, false, true, true>(p8, out.s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, dq8, out.dk8, &out.G[1]);
    bwd_level<4, XS, false, true, true>(p8, out.s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, dq8, out.dk8, &out.G[2]);
    bwd_level<8, XS, false, true, true>(p8, out.s8, a, bq, dAt, dAn, xh, xl, xnat, xk4, r, c, dq8, out.dk8, &out.G[3]);
    if constexpr (WRITE) {
        if (r == 0) {
            f32x8 t;
#pragma unroll
            for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(p8[e] + out.s8[e]);
            st8((float *)rt3, t);
        }
    }
    float qe[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        qe[e] = a[e] * fast_exp2(p8[e]);
        out.kt8[e] = bq[e] * fast_exp2(out.s8[e]);
    }
    if constexpr (WRITE) {
        D8 h8, l8;
        split8<BT>(qe, h8, l8);
        st8((BT *)qh3, h8);
        st8((BT *)ql3, l8);
    }
    return out;
}


}  // namespace gla
