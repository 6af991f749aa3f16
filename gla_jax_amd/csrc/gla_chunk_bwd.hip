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

// inclusive suffix sum over the 16 token rows of the wave (lane r receives sum over rows >= r)
__device__ __forceinline__ float suffix_sum_rows(float x)
{
    x += dpp_f32<0x101>(x);   // row_shl:1, lanes past the row end read 0
    x += dpp_f32<0x102>(x);
    x += dpp_f32<0x104>(x);
    x += dpp_f32<0x108>(x);
    return x;
}

template <typename T, int C, int D>
__global__ __launch_bounds__(C * 4) void chunk_grad_kernel(
    const float *__restrict__ g, const T *__restrict__ v, const T *__restrict__ k,
    const T *__restrict__ q, const T *__restrict__ dout, const T *__restrict__ states,
    const T *__restrict__ dstates, const float *__restrict__ decay, float *__restrict__ dg,
    T *__restrict__ dv, T *__restrict__ dk, T *__restrict__ dq, int T_len, int H)
{
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4, NT = D / 16;
    constexpr int LS = TileGeom<T, D>::kStride;
    constexpr int TR = C > D ? C : D;   // rows of one LDS tile
    typedef typename FragTypes<T>::d8 D8;
    extern __shared__ __align__(16) unsigned char smem[];
    T *tile0 = reinterpret_cast<T *>(smem);
    T *tile1 = tile0 + TR * LS;
    T *tile2 = tile1 + TR * LS;
    T *xs = tile2 + TR * LS;                                   // [NB][16][LS] per-wave scratch
    float *rtab = reinterpret_cast<float *>(xs + NB * 16 * LS);   // [NB][D] e^{tau_m}
    float *dltab = rtab + NB * D;                              // [NB][D] sub-block sums of q*dq - k*dk
    float *lbar = dltab + NB * D;                              // [D] chunk-level gate gradient

    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int r = lane & 15, c = lane >> 4;
    const int n = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int N = T_len / C;
    const int64_t tok = (int64_t)b * T_len + (int64_t)n * C + 16 * w + r;
    const int64_t rowoff = (tok * H + h) * D;
    const int64_t bhn = ((int64_t)b * H + h) * N + n;
    T *xw = xs + w * 16 * LS;

    float p[NV], s[NV];
    D8 qf[KS], kf[KS], vf[KS], dof[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * c;
        f32x8 gg = ld8(g + rowoff + d0);
#pragma unroll
        for (int e = 0; e < 8; ++e) { p[8 * ks + e] = gg.v[e] * kLog2e; s[8 * ks + e] = 0.f; }
        qf[ks] = ld8(q + rowoff + d0);
        kf[ks] = ld8(k + rowoff + d0);
        vf[ks] = ld8(v + rowoff + d0);
        dof[ks] = ld8(dout + rowoff + d0);
    }
    if (threadIdx.x < D) lbar[threadIdx.x] = 0.f;

    // ---- the wave's own sub-block ----------------------------------------------------------------
    // dAn[e] = dA[i = 4c+e][j = r],  dAt[e] = dA[i = r][j = 4c+e]   (dA = dO V^T)
    f32x4 dAn = {0.f, 0.f, 0.f, 0.f}, dAt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        dAn = mma_d(dof[ks], vf[ks], dAn);
        dAt = mma_d(vf[ks], dof[ks], dAt);
    }
    f32x4 Aown = {0.f, 0.f, 0.f, 0.f};   // scores A[i = 4c+e][j = r] of the own sub-block
    float dqa[NV], dka[NV];             // sub-block parts of dq, dk (row layout)
    // Gradient w.r.t. the gate cumsum L of this row.  Every term dA_ij * q~_i * k~_j enters row i with +
    // and row j with -; both sides are formed from the SAME rounded operands (the values the MFMAs
    // consume), so the two copies cancel exactly in the reverse cumsum (gla.py:1077-1087 asks for this).
    float dlm[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) { dqa[i] = 0.f; dka[i] = 0.f; dlm[i] = 0.f; }

    auto level = [&](auto hc) {
        constexpr int h_ = decltype(hc)::value;
        const bool upper = (r & h_) != 0;
        float fac[NV];
        D8 Xf[KS];
        f32x4 G = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], bq[8], x[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                fac[8 * ks + e] = fast_exp2(upper ? p[8 * ks + e] : s[8 * ks + e]);
                x[e] = (upper ? a[e] : bq[e]) * fac[8 * ks + e];
            }
            Xf[ks] = pack8<T>(x);
            G = mma_d(Xf[ks], Xf[ks], G);
            st8(xw + r * LS + 32 * ks + 8 * c, Xf[ks]);
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
        __syncthreads();
        auto b4 = pack4<T>(sym);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float xr[8];
            unpack8(Xf[ks], xr);
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const int t = 2 * ks + tt;
                const PiCols pc = pi_cols(t);
                f32x4 dx = {0.f, 0.f, 0.f, 0.f};
                dx = mma_t(lds_tr4(xw, LS, 4 * c, pc.seg, pc.own), b4, dx);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float z = dx[e] * fac[4 * t + e];
                    dqa[4 * t + e] += upper ? z : 0.f;
                    dka[4 * t + e] += upper ? 0.f : z;
                    const float y = dx[e] * xr[4 * tt + e];
                    dlm[4 * t + e] += upper ? y : -y;
                }
            }
        }
        hier_step<h_>(p, s, upper);
        __syncthreads();
    };
    level(std::integral_constant<int, 1>{});
    level(std::integral_constant<int, 2>{});
    level(std::integral_constant<int, 4>{});
    level(std::integral_constant<int, 8>{});

    // diagonal entries, rescaled key tile, table of e^{tau}
    {
        float dd = 0.f, dot = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) dd += (4 * c + e == r) ? dAt[e] : 0.f;
        dd = reduce_over_cgroups(dd);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], bq[8], kh[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                dot += a[e] * bq[e];
                dqa[8 * ks + e] += dd * bq[e];
                dka[8 * ks + e] += dd * a[e];
                kh[e] = bq[e] * fast_exp2(s[8 * ks + e]);
            }
            const int d0 = 32 * ks + 8 * c;
            st8(tile1 + (16 * w + r) * LS + d0, pack8<T>(kh));
            st8(tile0 + (16 * w + r) * LS + d0, vf[ks]);
        }
        dot = reduce_over_cgroups(dot);
#pragma unroll
        for (int e = 0; e < 4; ++e) Aown[e] += (4 * c + e == r) ? dot : 0.f;
        if (r == 0) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 t;
#pragma unroll
                for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(p[8 * ks + e] + s[8 * ks + e]);
                st8(rtab + w * D + 32 * ks + 8 * c, t);
            }
        }
        const T *sp = states + bhn * D * D;
        for (int idx = threadIdx.x; idx < D * D / 8; idx += C * 4) {
            const int row = idx / (D / 8), c8 = (idx % (D / 8)) * 8;
            st8(tile2 + row * LS + c8, ld8(sp + row * D + c8));
        }
    }
    __syncthreads();

    // ---- row-owner role: dq ----------------------------------------------------------------------
    {
        f32x4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const PiCols pc = pi_cols(t);
                auto a = join4(lds_tr4(tile2, LS, 32 * ks + 8 * c, pc.seg, pc.own),
                               lds_tr4(tile2, LS, 32 * ks + 8 * c + 4, pc.seg, pc.own));
                acc[t] = mma_d(a, dof[ks], acc[t]);
            }
        }
#pragma unroll
        for (int J = 0; J < NB - 1; ++J) {
            if (J < w) {
                f32x4 dAT = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    f32x8 rr = ld8(rtab + J * D + 32 * ks + 8 * c);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc[2 * ks][e] *= rr.v[e];
                        acc[2 * ks + 1][e] *= rr.v[4 + e];
                    }
                    dAT = mma_d(ld8(tile0 + (16 * J + r) * LS + 32 * ks + 8 * c), dof[ks], dAT);
                }
                auto b4 = pack4<T>(dAT);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const PiCols pc = pi_cols(t);
                    acc[t] = mma_t(lds_tr4(tile1, LS, 16 * J + 4 * c, pc.seg, pc.own), b4, acc[t]);
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], o[8], qr[8];
            unpack8(qf[ks], a);
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] *= fast_exp2(p[8 * ks + e]);
            unpack8(pack8<T>(a), qr);                    // q e^{l} as the MFMAs of the key side see it
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float hacc = e < 4 ? acc[2 * ks][e] : acc[2 * ks + 1][e - 4];
                o[e] = fast_exp2(p[8 * ks + e]) * hacc + dqa[8 * ks + e];
                dlm[8 * ks + e] += qr[e] * hacc;
            }
            st8(dq + rowoff + 32 * ks + 8 * c, pack8<T>(o));
        }
    }
    __syncthreads();

    // ---- second set of tiles: dO, q e^{l}, dS'^T; chunk-level term sum_v S*dS' ---------------------
    {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8];
            unpack8(qf[ks], a);
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] *= fast_exp2(p[8 * ks + e]);
            const int d0 = 32 * ks + 8 * c;
            st8(tile1 + (16 * w + r) * LS + d0, pack8<T>(a));
            st8(tile0 + (16 * w + r) * LS + d0, dof[ks]);
        }
        const T *dsp = dstates + bhn * D * D;
        float part[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) part[e] = 0.f;
        const int c8 = (threadIdx.x % (D / 8)) * 8;
        for (int idx = threadIdx.x; idx < D * D / 8; idx += C * 4) {
            const int row = idx / (D / 8);
            D8 dsv = ld8(dsp + row * D + c8);
            float a[8], bq[8];
            unpack8(ld8(tile2 + row * LS + c8), a);
            unpack8(dsv, bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) part[e] += a[e] * bq[e];
            st8(tile2 + row * LS + c8, dsv);
        }
        f32x8 dec = ld8(decay + bhn * D + c8);
#pragma unroll
        for (int e = 0; e < 8; ++e) atomicAdd(lbar + c8 + e, part[e] * dec.v[e]);
    }
    __syncthreads();

    // ---- column-owner role: scores, dv ------------------------------------------------------------
    float kch[NV];   // k e^{tau_J - l_j}, walked up to k e^{L_end - L_j}
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        float bq[8];
        unpack8(kf[ks], bq);
#pragma unroll
        for (int e = 0; e < 8; ++e) kch[8 * ks + e] = bq[e] * fast_exp2(s[8 * ks + e]);
    }
    {
        f32x4 Ab[NB];
#pragma unroll
        for (int I = 1; I < NB; ++I) {
            Ab[I] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (I > w) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    Ab[I] = mma_d(ld8(tile1 + (16 * I + r) * LS + 32 * ks + 8 * c), pack8<T>(kch + 8 * ks), Ab[I]);
                    f32x8 rr = ld8(rtab + I * D + 32 * ks + 8 * c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) kch[8 * ks + e] *= rr.v[e];
                }
            }
        }
        Ab[0] = f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            D8 kb = pack8<T>(kch + 8 * ks);
#pragma unroll
            for (int t = 0; t < NT; ++t)
                acc[t] = mma_d(ld8(tile2 + pi_cols(t).own * LS + 32 * ks + 8 * c), kb, acc[t]);
        }
#pragma unroll
        for (int I = 0; I < NB; ++I) {
            if (I >= w) {
                auto b4 = pack4<T>(I == w ? Aown : Ab[I]);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const PiCols pc = pi_cols(t);
                    acc[t] = mma_t(lds_tr4(tile0, LS, 16 * I + 4 * c, pc.seg, pc.own), b4, acc[t]);
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float o[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[e] = acc[2 * ks][e]; o[4 + e] = acc[2 * ks + 1][e]; }
            st8(dv + rowoff + 32 * ks + 8 * c, pack8<T>(o));
        }
    }

    // ---- column-owner role: dk, then dlog_fgate ----------------------------------------------------
    {
        f32x4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const PiCols pc = pi_cols(t);
                auto a = join4(lds_tr4(tile2, LS, 32 * ks + 8 * c, pc.seg, pc.own),
                               lds_tr4(tile2, LS, 32 * ks + 8 * c + 4, pc.seg, pc.own));
                acc[t] = mma_d(a, vf[ks], acc[t]);
            }
        }
        // chunk-level gate gradient, key part: sum_j (k e^{L_end - L_j}) * (V dS'^T)_j
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float z = reduce_over_rows(kch[4 * t + e] * acc[t][e]);
                if (r == 0) atomicAdd(lbar + 32 * (t >> 1) + 8 * c + 4 * (t & 1) + e, z);
            }
        }
#pragma unroll
        for (int I = NB - 1; I >= 1; --I) {
            if (I > w) {
                f32x4 dAI = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    f32x8 rr = ld8(rtab + I * D + 32 * ks + 8 * c);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc[2 * ks][e] *= rr.v[e];
                        acc[2 * ks + 1][e] *= rr.v[4 + e];
                    }
                    dAI = mma_d(ld8(tile0 + (16 * I + r) * LS + 32 * ks + 8 * c), vf[ks], dAI);
                }
                auto b4 = pack4<T>(dAI);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const PiCols pc = pi_cols(t);
                    acc[t] = mma_t(lds_tr4(tile1, LS, 16 * I + 4 * c, pc.seg, pc.own), b4, acc[t]);
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float bq[8], o[8], kr[8];
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) bq[e] *= fast_exp2(s[8 * ks + e]);
            unpack8(pack8<T>(bq), kr);                   // k e^{tau-l} as the MFMAs of the query side see it
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float hacc = e < 4 ? acc[2 * ks][e] : acc[2 * ks + 1][e - 4];
                o[e] = fast_exp2(s[8 * ks + e]) * hacc + dka[8 * ks + e];
                dlm[8 * ks + e] -= kr[e] * hacc;
            }
            st8(dk + rowoff + 32 * ks + 8 * c, pack8<T>(o));
        }
    }
    // reverse cumsum inside the chunk (gla.py:616-617)
#pragma unroll
    for (int i = 0; i < NV; ++i) dlm[i] = suffix_sum_rows(dlm[i]);
    if (r == 0) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 t;
#pragma unroll
            for (int e = 0; e < 8; ++e) t.v[e] = dlm[8 * ks + e];
            st8(dltab + w * D + 32 * ks + 8 * c, t);
        }
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * c;
        f32x8 o = ld8(lbar + d0);
#pragma unroll
        for (int e = 0; e < 8; ++e) o.v[e] += dlm[8 * ks + e];
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
    constexpr int TR = C > D ? C : D, NB = C / 16;
    const size_t lds = (size_t)(3 * TR + NB * 16) * LS * sizeof(T) + (size_t)(2 * NB + 1) * D * sizeof(float);
    auto kern = chunk_grad_kernel<T, C, D>;
    if (int e = allow_lds((const void *)kern, lds)) return e;
    dim3 grid(T_len / C, H, B), block(C * 4);
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
