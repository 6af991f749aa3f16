// chunk_gla forward, output kernel: one workgroup per chunk computes
//     out_i = sum_{j<=i} A_ij v_j  +  (q_i * exp(L_i))^T S_n            (gla.py:792-855, 724-725)
// with A_ij = sum_d q_id k_jd exp(L_id - L_jd) the gated causal scores of gla.py:964-1029.
//
// Secondary chunking.  The chunk is cut into 16-token sub-blocks, one per wave.  With l_i the
// inclusive gate sum inside the sub-block and tau_m the total of sub-block m:
//   * sub-block pair (I > J):  A_ij = sum_d [q_i e^{l_i} prod_{J<m<I} e^{tau_m}]_d [k_j e^{tau_J - l_j}]_d
//     every factor is <= 1; the q side is walked down J = I-1..0 by one multiply per step, and after the
//     last step it is q_i e^{L_i}, the operand of the inter-chunk product;
//   * inside a sub-block the dyadic anchors of the reference are kept (levels 16, 8, 4, 2 of
//     gla.py:1000-1027): at level 2h rows in the upper half of their group carry q e^{prefix over
//     the half}, rows in the lower half carry k e^{suffix over the half}, both <= 1, and ONE
//     16x16xD MFMA of that mixed tile with itself yields every block of the level (masked);
//   * the diagonal is the plain fp32 dot q_i.k_i (gla.py:983).
// Scores are produced transposed (key token x query token) so that the accumulator registers are
// directly the B operand of the (feature x token) product with V.
#include "gla_chunk_common.hpp"
#include "gla_chunk_kernels.hpp"

namespace gla {

template <typename T, int C, int D>
__global__ __launch_bounds__(C * 4) void chunk_out_kernel(const float *__restrict__ g,
                                                          const T *__restrict__ v,
                                                          const T *__restrict__ k,
                                                          const T *__restrict__ q,
                                                          const T *__restrict__ states,
                                                          T *__restrict__ out, int T_len, int H)
{
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4, NT = D / 16;
    constexpr int LS = TileGeom<T, D>::kStride;
    typedef typename FragTypes<T>::d8 D8;
    extern __shared__ __align__(16) unsigned char smem[];
    T *Kh = reinterpret_cast<T *>(smem);           // [C][LS]  k * exp(tau_J - l_j)
    T *Vn = Kh + C * LS;                           // [C][LS]  value
    T *St = Vn + C * LS;                           // [D][LS]  chunk-start state, [dv][dk]
    float *rtab = reinterpret_cast<float *>(St + D * LS);   // [NB][D] exp(tau_m)

    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int r = lane & 15, c = lane >> 4;
    // heads vary fastest over the grid: workgroups that run together touch the same DRAM pages of the
    // [B, T, H, D] arrays (a token's H rows are contiguous)
    const int h = blockIdx.x % H, n = blockIdx.x / H, b = blockIdx.y;
    const int N = T_len / C;
    const int64_t tok = (int64_t)b * T_len + (int64_t)n * C + 16 * w + r;
    const int64_t rowoff = (tok * H + h) * D;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const int wrow = 16 * w * LS + L.nat;          // this lane's row of a [token][feature] tile

    float p[NV], s[NV];
    D8 qf[KS], kf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * c;
        f32x8 gg = ld8(g + rowoff + d0);
#pragma unroll
        for (int e = 0; e < 8; ++e) p[8 * ks + e] = gg.v[e] * kLog2e;
        qf[ks] = ld8(q + rowoff + d0);
        kf[ks] = ld8(k + rowoff + d0);
        st8(Vn + wrow + 32 * ks, ld8(v + rowoff + d0));
    }
    {
        const T *sp = states + (((int64_t)b * H + h) * N + n) * D * D;
        for (int idx = threadIdx.x; idx < D * D / 8; idx += C * 4) {
            const int row = idx / (D / 8), c8 = (idx % (D / 8)) * 8;
            st8(St + row * LS + c8, ld8(sp + row * D + c8));
        }
    }

    // ---- gate prefix of the sub-block; can the whole sub-block share ONE anchor? ------------------
    // p = l_i (inclusive prefix over the 16 rows, log2 units), s = tau - l_i.  The totals travel through
    // the wave's own row of rtab (same-wave LDS accesses execute in order).
#pragma unroll
    for (int i = 0; i < NV; ++i) p[i] = prefix_sum_rows(p[i]);
    if (r == 15) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) st8(rtab + w * D + 32 * ks + 8 * c, pack8<float>(p + 8 * ks));
    }
    asm volatile("" ::: "memory");
    float span = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        f32x8 tau = ld8(rtab + w * D + 32 * ks + 8 * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            s[8 * ks + e] = tau.v[e] - p[8 * ks + e];
            span = fmaxf(span, fmaxf(fabsf(p[8 * ks + e]), fabsf(s[8 * ks + e])));
        }
    }
    asm volatile("" ::: "memory");
    const bool one_anchor = wave_all_below(span, kOneAnchorSpan);

    f32x4 accD = {0.f, 0.f, 0.f, 0.f};   // transposed scores of the diagonal sub-block: [j = 4c+e][i = r]
    if (one_anchor) {
        // Gates this mild need no recursion: with the anchor at the end of the sub-block,
        // A_ij = [q_i e^{l_i - tau}] . [k_j e^{tau - l_j}], both factors are finite (at most 2^span) and carry
        // the same relative rounding as the dyadic form.  The key factor is the operand of the other
        // sub-blocks as well.
        f32x4 G = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], bq[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                a[e] *= fast_exp2(-s[8 * ks + e]);
                bq[e] *= fast_exp2(s[8 * ks + e]);
            }
            G = mma_d(pack8<T>(bq), pack8<T>(a), G);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) accD[e] = (4 * c + e < r) ? G[e] : 0.f;
    } else {
        // ---- the dyadic levels 2, 4, 8, 16 of the reference ------------------------------------------
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 gg = ld8(refetch(g + rowoff) + 32 * ks + 8 * c);
#pragma unroll
            for (int e = 0; e < 8; ++e) { p[8 * ks + e] = gg.v[e] * kLog2e; s[8 * ks + e] = 0.f; }
        }
        auto level = [&](auto hc) {
            constexpr int h_ = decltype(hc)::value;
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
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = 4 * c + e;
                const bool ok = ((j ^ r) < 2 * h_) && upper && !(j & h_);
                accD[e] += ok ? G[e] : 0.f;
            }
            hier_step<h_>(p, s, upper);
        };
        level(std::integral_constant<int, 1>{});
        level(std::integral_constant<int, 2>{});
        level(std::integral_constant<int, 4>{});
        level(std::integral_constant<int, 8>{});
    }

    // p = l_i (inclusive, log2 units), s = tau - l_i.  Rescaled operands, diagonal, table of exp(tau).
    float qh[NV];
    {
        float dot = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float a[8], bq[8], kh[8];
            unpack8(qf[ks], a);
            unpack8(kf[ks], bq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                dot += a[e] * bq[e];
                qh[8 * ks + e] = a[e] * fast_exp2(p[8 * ks + e]);
                kh[e] = bq[e] * fast_exp2(s[8 * ks + e]);
            }
            st8(Kh + wrow + 32 * ks, pack8<T>(kh));
        }
        dot = reduce_over_cgroups(dot);
#pragma unroll
        for (int e = 0; e < 4; ++e) accD[e] += (4 * c + e == r) ? dot : 0.f;
        if (r == 0) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                f32x8 t;
#pragma unroll
                for (int e = 0; e < 8; ++e) t.v[e] = fast_exp2(p[8 * ks + e] + s[8 * ks + e]);
                st8(rtab + w * D + 32 * ks + 8 * c, t);
            }
        }
    }
    __syncthreads();

    // ---- earlier sub-blocks J < w, walking the q side down ---------------------------------------
    f32x4 accT[NB];
#pragma unroll
    for (int J = NB - 2; J >= 0; --J) {
        accT[J] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (J < w) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                D8 qb = pack8<T>(qh + 8 * ks);
                D8 ka = ld8(Kh + L.nat + 16 * J * LS + 32 * ks);
                accT[J] = mma_d(ka, qb, accT[J]);
                f32x8 rr = ld8(rtab + J * D + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) qh[8 * ks + e] *= rr.v[e];
            }
        }
    }
    accT[NB - 1] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- out^T[dv][i]: state term, then the score blocks ----------------------------------------
    f32x4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        D8 qb = pack8<T>(qh + 8 * ks);   // q * exp(L_i)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            D8 sa = ld8(St + L.own + own_const(t, 32 * ks, LS));
            acc[t] = mma_d(sa, qb, acc[t]);
        }
    }
#pragma unroll
    for (int J = 0; J < NB; ++J) {
        if (J <= w) {
            auto b4 = pack4<T>(J == w ? accD : accT[J]);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                auto a4 = lds_tr4(Vn + L.k4 + tr_const(16 * J, t, LS), LS);
                acc[t] = mma_t(a4, b4, acc[t]);
            }
        }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        float o[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) { o[e] = acc[2 * ks][e]; o[4 + e] = acc[2 * ks + 1][e]; }
        st8(out + rowoff + 32 * ks + 8 * c, pack8<T>(o));
    }
}

template <typename T, int C, int D>
int launch_chunk_out(hipStream_t st, int B, int T_len, int H, const float *g, const void *v, const void *k,
                     const void *q, const void *states, void *out)
{
    constexpr int LS = TileGeom<T, D>::kStride;
    const size_t lds = (size_t)(2 * C + D) * LS * sizeof(T) + (size_t)(C / 16) * D * sizeof(float);
    auto kern = chunk_out_kernel<T, C, D>;
    if (int e = allow_lds((const void *)kern, lds)) return e;
    dim3 grid(T_len / C * H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)v, (const T *)k, (const T *)q,
                       (const T *)states, (T *)out, T_len, H);
    return launch_status();
}

#define GLA_INST_OUT(T, C, D)                                                                          \
    template int launch_chunk_out<T, C, D>(hipStream_t, int, int, int, const float *, const void *,   \
                                           const void *, const void *, const void *, void *);
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_OUT)

}  // namespace gla
