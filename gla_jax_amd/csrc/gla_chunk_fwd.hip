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
#include "gla_subblock.hpp"
#include "gla_chunk_kernels.hpp"

namespace gla {

// Resources: two tiles (keys of all but the last sub-block, values), 32 staged state rows and a table
// fit twice into a CU's LDS, and the register budget is held to what lets two workgroups share a CU, so
// that one loads while the other computes.
// WIDE: `out` is a float array (the sum of two such runs is rounded once: head dimension 256, gla_split.hip).
template <typename T, int C, int D, int DM, bool WIDE>
__global__ __launch_bounds__(C * 4) __attribute__((amdgpu_waves_per_eu(C / 32, C / 32))) void chunk_out_kernel(
    const float *__restrict__ g, const T *__restrict__ v, const T *__restrict__ k, const T *__restrict__ q,
    const T *__restrict__ states, int slots, std::conditional_t<WIDE, float, T> *__restrict__ out, int T_len, int H)
{
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4;
    constexpr int LS = TileGeom<T, D>::kStride;
    typedef typename FragTypes<T>::d8 D8;
    typedef typename FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *Vn = reinterpret_cast<T *>(smem);           // [C][LS]       value
    T *Kh = Vn + C * LS;                           // [C - 16][LS]  k * exp(tau_J - l_j), sub-blocks 0 .. NB-2
    T *St = Kh + (C - 16) * LS;                    // [32][LS]      32 rows of the chunk-start state [dv][dk] (fp32 data)
    // 16-bit data: the slab [all dk][32 dv] of the tiled state, as it lies in memory ([dk][SS]); the products read
    // it transposed
    constexpr bool kTiled = sizeof(T) == 2;
    constexpr int SS = 32;                         // row stride of the slab: the rows as they lie in a tile
    static_assert(!kTiled || D * SS <= 32 * LS, "the slab fits where the 32 staged rows were");
    const TrLane<T> Ls = make_tr_lane<T>(SS);
    float *rtab = reinterpret_cast<float *>(St + 32 * LS);   // [NB][D] exp(tau_m)

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, c = lane >> 4;
    // heads vary fastest over the grid: workgroups that run together touch the same DRAM pages of the
    // [B, T, H, D] arrays (a token's H rows are contiguous)
    const int h = blockIdx.x % H, n = blockIdx.x / H, b = blockIdx.y;
    const int N = T_len / C;
    const int64_t tok = (int64_t)b * T_len + (int64_t)n * C + 16 * w + r;
    const int64_t rowoff = (tok * H + h) * DM;     // DM features per row in memory (DM < D: see RowMap)
    const TrLane<T> L = make_tr_lane<T>(LS);
    const int wrow = 16 * w * LS + L.nat;          // this lane's row of a [token][feature] tile

    // 32 rows of the state per slice of the output's features, through registers, one slice ahead
    constexpr int kPieces = 32 * D / 8;                       // 8-element pieces of a slice
    constexpr int kPer = (kPieces + C * 4 - 1) / (C * 4);     // pieces per thread
    D8 pf[kPer];
    const T *sp = states + (((int64_t)b * H + h) * slots + n) * D * D;
    auto stage_fetch = [&](int slice) {
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int idx = threadIdx.x + u * C * 4;
            if (kPieces % (C * 4) == 0 || idx < kPieces) {
                if constexpr (kTiled)      // tiles (i, slice), i = idx / 128: 2 KB each, read as they lie
                    pf[u] = ld8(sp + (((idx >> 7) * (D / 32) + slice) << 10) + (idx & 127) * 8);
                else
                    pf[u] = ld8(sp + (32 * slice + idx / (D / 8)) * D + (idx % (D / 8)) * 8);
            }
        }
    };
    auto stage_store = [&]() {
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int idx = threadIdx.x + u * C * 4;
            if (kPieces % (C * 4) == 0 || idx < kPieces) {
                if constexpr (kTiled)
                    st8(St + (32 * (idx >> 7) + ((idx & 127) >> 2)) * SS + 8 * (idx & 3), pf[u]);
                else
                    st8(St + (idx / (D / 8)) * LS + (idx % (D / 8)) * 8, pf[u]);
            }
        }
    };

    f32x4 accD = {0.f, 0.f, 0.f, 0.f};   // transposed scores of the diagonal sub-block: [j = 4c+e][i = r]
    float qh[NV];                        // q * exp(l_i), walked down the earlier sub-blocks below
    {
        float p[NV];
        D8 qf[KS], kf[KS];
        // The gates come first and are scanned before q and k are requested: with all three in flight at
        // once the 128 registers that let two workgroups share a CU do not suffice, and the spill of a
        // freshly loaded row makes the wave wait for every request it has out.
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            f32x8 gg = ld8_row<D, DM>(g + rowoff + 32 * ks, c);
#pragma unroll
            for (int e = 0; e < 8; ++e) p[8 * ks + e] = gg.v[e] * kLog2e;
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) p[i] = prefix_sum_rows(p[i]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qf[ks] = ld8_row<D, DM>(q + rowoff + 32 * ks, c);
            kf[ks] = ld8_row<D, DM>(k + rowoff + 32 * ks, c);
        }

        // (the hard-gate path reads the rows again at row + 8c: the row pointers are shifted so that a padded lane
        // lands on its row's first features, and `valid` zeroes what it reads there)
        const int shift = RowMap<D, DM>::col(c) - 8 * c;
        subblock_forward<T, D, false, true>(p, qf, kf, g + rowoff + shift, q + rowoff + shift, k + rowoff + shift,
                                            RowMap<D, DM>::live(c), rtab + w * D, Kh + wrow, w < NB - 1, nullptr, r, c,
                                            accD, qh);
    }
    // Values and the first state rows are requested only now: the registers above are free again, and
    // the other workgroup on the CU covers the wait.
    {
        D8 vf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) vf[ks] = ld8_row<D, DM>(v + rowoff + 32 * ks, c);
        stage_fetch(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) st8(Vn + wrow + 32 * ks, vf[ks]);
    }
    stage_store();
    __syncthreads();
    if (KS > 1) stage_fetch(1);

    // ---- earlier sub-blocks J < w, walking the q side down; scores kept as packed MFMA operands ----
    T4 sc[NB];
#pragma unroll
    for (int J = NB - 2; J >= 0; --J) {
        f32x4 a = {0.f, 0.f, 0.f, 0.f};
        if (J < w) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                D8 qb = pack8<T>(qh + 8 * ks);
                D8 ka = ld8(Kh + L.nat + 16 * J * LS + 32 * ks);
                a = mma_d(ka, qb, a);
                f32x8 rr = ld8(rtab + J * D + 32 * ks + 8 * c);
#pragma unroll
                for (int e = 0; e < 8; ++e) qh[8 * ks + e] *= rr.v[e];
            }
        }
        sc[J] = pack4<T>(a);
    }
    sc[NB - 1] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
    // The own sub-block's scores enter the product with V as head + remainder: next to the diagonal the gated
    // scores are the largest of a row, and under strong decay they carry most of the output.
    T4 scD, scDl;
    split4<T>(accD, scD, scDl);
    D8 qb[KS];                           // q * exp(L_i): operand of the state term
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qb[ks] = pack8<T>(qh + 8 * ks);

    // ---- out^T[dv][i] in slices of 32 output features: state term, then the score blocks ------------
#pragma unroll 1
    for (int ks = 0; ks < KS; ++ks) {
        const int fo = 32 * ks;
        f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int k2 = 0; k2 < KS; ++k2) {
            if constexpr (kTiled) {
                // step (k2, half) contracts over dk = 32 k2 + 8c + 4 half + m, which is what lane (i, c) holds of
                // (q e^{L})_i; 16 key features per product, the slab read transposed
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const T4 qh4 = half ? __builtin_shufflevector(qb[k2], qb[k2], 4, 5, 6, 7)
                                        : __builtin_shufflevector(qb[k2], qb[k2], 0, 1, 2, 3);
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt)
                        acc[tt] = mma_t(lds_tr4(St + Ls.k8 + (32 * k2 + 4 * half) * SS + 4 * tt, SS), qh4, acc[tt]);
                }
            } else {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    acc[tt] = mma_d(ld8(St + L.own + 4 * tt * LS + 32 * k2), qb[k2], acc[tt]);
            }
        }
#pragma unroll
        for (int J = 0; J < NB; ++J) {
            if (J <= w) {
                const T4 b4 = J == w ? scD : sc[J];
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    const T4 va = lds_tr4(Vn + L.k4 + fo + 4 * tt + 16 * J * LS, LS);
                    if constexpr (sizeof(T) == 2) {
                        if (J == w) acc[tt] = mma_t(va, scDl, acc[tt]);
                    }
                    acc[tt] = mma_t(va, b4, acc[tt]);
                }
            }
        }
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = acc[e >> 2][e & 3];
        st8_row_once<D, DM>(out + rowoff + fo, c, pack8<std::conditional_t<WIDE, float, T>>(o));
        if (ks + 1 < KS) {
            __syncthreads();             // every wave is done with the staged rows
            stage_store();
            __syncthreads();
            if (ks + 2 < KS) stage_fetch(ks + 2);
        }
    }
}

template <typename T, int C, int D, int DM, bool WIDE>
int launch_chunk_out(hipStream_t st, int B, int T_len, int H, const float *g, const void *v, const void *k,
                     const void *q, const void *states, int slots, void *out)
{
    constexpr int LS = TileGeom<T, D>::kStride;
    const size_t lds = (size_t)(2 * C - 16 + 32) * LS * sizeof(T) + (size_t)(C / 16) * D * sizeof(float);
    auto kern = chunk_out_kernel<T, C, D, DM, WIDE>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(T_len / C * H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)v, (const T *)k, (const T *)q,
                       (const T *)states, slots, (std::conditional_t<WIDE, float, T> *)out, T_len, H);
    return launch_status();
}

#define GLA_INST_OUT_AS(T, C, D, DM, WIDE)                                                                   \
    template int launch_chunk_out<T, C, D, DM, WIDE>(hipStream_t, int, int, int, const float *, const void *, \
                                                     const void *, const void *, const void *, int, void *);
#define GLA_INST_OUT(T, C, D, DM) GLA_INST_OUT_AS(T, C, D, DM, false)
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_OUT)
GLA_INST_OUT_AS(__bf16, 128, 128, 128, true)
GLA_INST_OUT_AS(__bf16, 64, 128, 128, true)
GLA_INST_OUT_AS(__bf16, 32, 128, 128, true)

}  // namespace gla
