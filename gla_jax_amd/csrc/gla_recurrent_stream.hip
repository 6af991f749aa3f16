// recurrent_gla forward for bf16 inputs on the matrix cores: one workgroup streams over the sequence of
// one (batch, head) pair with the [DK,DV] state in fp32 accumulator registers; no hidden state ever
// touches HBM (gla.py:50-96 keeps the state of a program in registers the same way).
//
// The rank-1 updates of C consecutive timesteps are applied together.  With L_t the gate sum from the
// start of the block of C steps to t and Lend its total,
//     o_t  = (q_t e^{L_t})^T S_in + sum_{j<=t} A_tj v_j ,        A_tj = sum_d q_td k_jd e^{L_td - L_jd}
//     S_out = diag(e^{Lend}) S_in + sum_j (k_j e^{Lend - L_j}) v_j^T
// which is the recurrence S_t = diag(e^{g_t}) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t written out for C steps
// (gla.py:35-37).  The block is cut into 16-step sub-blocks, one per wave; scores inside a sub-block and
// the rescaled operands come from subblock_forward (every exponent <= 0, or bounded, see there), pairs
// of sub-blocks multiply the query side down by e^{tau_m} per step, and the state update is a Horner chain
// over the sub-blocks: S <- S * e^{tau_J} + V_J^T (k e^{tau_J - l})_J, so nothing is rescaled by a factor
// above 1; the rescaled keys enter it as bf16 head + remainder, so the update is as exact as the fp32
// rank-1 updates of the reference.  The state enters the output product as a pair of bf16 numbers (head + remainder, 16 bits of
// mantissa), so the fp32 state of the reference (gla.py:89) is not rounded where it is used.
//
// Steps past the end of the sequence are padded with g = 0, k = v = q = 0 (they leave the state alone and
// are not stored), so any T works.  `reverse` walks the sequence from its end (gla.py:421-438).
#include "gla_subblock.hpp"
#include "gla_recurrent_stream.hpp"

namespace gla {

template <typename TO> struct OutPack;
template <> struct OutPack<__bf16> {
    static __device__ __forceinline__ void store(__bf16 *p, const float *o) { st8(p, pack8<__bf16>(o)); }
};
template <> struct OutPack<float> {
    static __device__ __forceinline__ void store(float *p, const float *o) { st8(p, pack8<float>(o)); }
};

// STATE: only hidden_final is wanted (a segment's own contribution to the state, or to its cotangent, when a
// sequence runs as segments side by side): the scores of earlier sub-blocks, the output products and the stores
// of `out` are left out, and so is the copy of the state that those products read.
template <typename TO, int C, int D, bool STATE = false>
__global__ __launch_bounds__(C * 4, STATE ? 2 : 1) void recurrent_stream_fwd_kernel(
    const void *__restrict__ h0, const float *__restrict__ g, const __bf16 *__restrict__ v,
    const __bf16 *__restrict__ k, const __bf16 *__restrict__ q, void *__restrict__ hT,
    TO *__restrict__ out, int T_len, int H, int reverse, int hdt, int g_shift, float *__restrict__ gate_sums)
{
    typedef __bf16 T;
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4, NT = D / 16;
    // The NT x NT state tiles are split evenly over the waves: a wave owns RT tile rows (dv) and NTW of the
    // NT tile columns (dk).  With more waves than tile rows, G waves share a row and split its columns.
    constexpr int G = NB > NT ? NB / NT : 1, RT = NB > NT ? 1 : NT / NB, NTW = NT / G, NDV = NB / G;
    static_assert(NT * NT % NB == 0 && NDV * RT == NT && NTW * G == NT, "the state tiles split evenly over the waves");
    constexpr int LS = TileGeom<T, D>::kStride;
    typedef typename FragTypes<T>::d8 D8;
    typedef typename FragTypes<T>::t4 T4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *Vn = reinterpret_cast<T *>(smem);           // [C][LS]  value
    T *Kh = Vn + C * LS;                           // [C][LS]  k * exp(tau_J - l_j)
    T *Kl = Kh + C * LS;                           // [C][LS]  what the bf16 rounding of Kh leaves over
    T *St = Kl + C * LS;                           // [D][LS]  state at the start of the block, [dv][dk]: bf16 head
    T *Sl = St + D * LS;                           // [D][LS]  ... and the bf16 of what the head leaves over
    float *rtab = reinterpret_cast<float *>(STATE ? St : Sl + D * LS);   // [NB][D] exp(tau_m)
    float *gsum = rtab + NB * D;                   // [NB][D] (STATE with gate_sums) every wave's share of the sequence's gate sums

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, c = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y;
    const int64_t seq = ((int64_t)b * T_len * H + h) * D;      // element offset of (b, t = 0, h)
    const int64_t rowstride = (int64_t)H * D;
    const int64_t bh = (int64_t)b * H + h;
    const TrLane<T> L = make_tr_lane<T>(LS);
    const int ptl = plain_tr_lane<T>(LS);
    const int wrow = 16 * w * LS + L.nat;          // this lane's row of a [token][feature] tile
    const int N = (T_len + C - 1) / C;
    const int wv = w % NDV, nt0 = (w / NDV) * NTW;   // the wave's tile rows are wv + i NDV, its tile columns nt0 + j

    // state: S[i][j][e] = state[dk = 16(nt0 + j) + r][dv = 16(wv + i NDV) + 4c + e]  (accumulator layout of a
    // (dv x dk) product tile)
    f32x4 S[RT][NTW];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            float t4[4] = {0.f, 0.f, 0.f, 0.f};     // no initial state given: zeros (the lean pass of a segment)
            if (h0) load_hidden<4>(h0, hdt, bh * D * D + (int64_t)(16 * (nt0 + nt) + r) * D + 16 * (wv + i * NDV) + 4 * c, t4);
            S[i][nt] = f32x4{t4[0], t4[1], t4[2], t4[3]};
        }
    // A lane's four values of a tile lie in four rows of the [dv][dk] copy.  The four lanes of a quad exchange them
    // (a 4 x 4 transpose in two steps across lanes 1 and 2 apart), after which lane 4a + j holds the key features
    // 4a..4a+3 of row 4c + j: one 8-byte store per tile and precision instead of four 2-byte ones.
    auto publish_state = [&]() {
        const int j = r & 3;
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                f32x4 x = S[i][nt], y;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float other = dpp_f32<kDppQuadXor1>(x[e ^ 1]);
                    y[e] = ((j ^ e) & 1) ? other : x[e];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float other = dpp_f32<kDppQuadXor2>(y[e ^ 2]);
                    x[e] = ((j ^ e) & 2) ? other : y[e];
                }
                T4 hi, lo;
                split4<T>(x, hi, lo);
                const int off = (16 * (wv + i * NDV) + 4 * c + j) * LS + 16 * (nt0 + nt) + (r & 12);
                *reinterpret_cast<T4 *>(St + off) = hi;
                *reinterpret_cast<T4 *>(Sl + off) = lo;
            }
    };
    if constexpr (!STATE) publish_state();
    if constexpr (STATE) {
        if (gate_sums)
            for (int d = threadIdx.x; d < NB * D; d += C * 4) gsum[d] = 0.f;
        __syncthreads();                             // a wave adds to its row before the loop's first barrier
    }

    // inputs of the wave's 16 steps of a block, one block ahead
    f32x8 gN[KS];
    D8 qN[KS], kN[KS], vN[KS];
    bool validN;
    int64_t rowN, growN;
    auto fetch = [&](int n) {
        const int s = n * C + 16 * w + r;                      // logical step
        validN = s < T_len;
        const int sc = validN ? s : T_len - 1;
        const int at = reverse ? T_len - 1 - sc : sc;
        rowN = seq + (int64_t)at * rowstride;
        growN = rowN;
        if constexpr (STATE) {
            // g_shift: a step takes the gate of the row g_shift rows further on in the array (the sequences of a
            // launch lie one behind the other).  Where the array ends the nearest row stands in: that step is the
            // first of its sequence, and its gate scales the zeros, or the initial state, it starts from.
            int64_t gr = (int64_t)b * T_len + at + g_shift;
            const int64_t last = (int64_t)gridDim.y * T_len - 1;
            gr = gr < 0 ? 0 : (gr > last ? last : gr);
            growN = (gr * H + h) * D;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            gN[ks] = ld8(g + growN + 32 * ks + 8 * c);
            kN[ks] = ld8(k + rowN + 32 * ks + 8 * c);
            if constexpr (!STATE) qN[ks] = ld8(q + rowN + 32 * ks + 8 * c);
            else qN[ks] = kN[ks];                             // nothing uses the query side of a lean pass
            vN[ks] = ld8(v + rowN + 32 * ks + 8 * c);
        }
    };
    fetch(0);

#pragma unroll 1
    for (int n = 0; n < N; ++n) {
        const bool valid = validN;
        const int64_t row = rowN, grow = growN;
        f32x4 accD = {0.f, 0.f, 0.f, 0.f};   // transposed scores of the own sub-block: [j = 4c+e][i = r]
        float qh[NV];                        // q * exp(l_i), walked down the earlier sub-blocks below
        {
            float p[NV];
            D8 qf[KS], kf[KS];
            if ((n + 1) * C > T_len && !valid) {   // only the last block can hold padded steps
                float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    gN[ks] = pack8<float>(z);
                    qN[ks] = kN[ks] = vN[ks] = pack8<T>(z);
                }
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) p[8 * ks + e] = gN[ks].v[e] * kLog2e;
                qf[ks] = qN[ks];
                kf[ks] = kN[ks];
                st8(Vn + wrow + 32 * ks, vN[ks]);
            }
            subblock_forward<T, D, true, false, D == 64>(p, qf, kf, g + grow, q + row, k + row, valid, rtab + w * D, Kh + wrow, true,
                                   Kl + wrow, r, c, accD, qh);
            if constexpr (STATE) {
                // the sequence's gate sums (what the scan over segments decays a state by): p now holds the sums
                // over the sub-block's rows up to the lane's own, in powers of two, so its last row holds the
                // sub-block's total (padded steps add zeros).  Every wave keeps a row of its own, added up in wave
                // order at the end: the same bits whenever the same call runs again
                if (gate_sums && r == 15) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        f32x8 t = ld8(gsum + w * D + 32 * ks + 8 * c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) t.v[e] += p[8 * ks + e];
                        st8(gsum + w * D + 32 * ks + 8 * c, t);
                    }
                }
            }
        }
        __syncthreads();                     // tiles of this block and the published state are in place

        if constexpr (!STATE) {
        // ---- earlier sub-blocks J < w, walking the q side down; scores kept as packed MFMA operands ----
        // (operands and scores as bf16 head + remainder: the products keep 16 bits of mantissa)
        T4 sc[NB], sl[NB];
#pragma unroll
        for (int J = NB - 2; J >= 0; --J) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            if (J < w) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    D8 qbh, qbl;
                    split8<T>(qh + 8 * ks, qbh, qbl);
                    a = mma_d_split(ld8(Kh + L.nat + 16 * J * LS + 32 * ks), ld8(Kl + L.nat + 16 * J * LS + 32 * ks),
                                    qbh, qbl, a);
                    f32x8 rr = ld8(rtab + J * D + 32 * ks + 8 * c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) qh[8 * ks + e] *= rr.v[e];
                }
            }
            split4<T>(a, sc[J], sl[J]);
        }
        sc[NB - 1] = pack4<T>(f32x4{0.f, 0.f, 0.f, 0.f});
        sl[NB - 1] = sc[NB - 1];
        T4 scD, slD;
        split4<T>(accD, scD, slD);
        D8 qb[KS], ql[KS];                   // q * exp(L_i), operand of the state term: bf16 head and remainder
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float hi[8], lo[8];
            qb[ks] = pack8<T>(qh + 8 * ks);
            unpack8(qb[ks], hi);
#pragma unroll
            for (int e = 0; e < 8; ++e) lo[e] = qh[8 * ks + e] - hi[e];
            ql[ks] = pack8<T>(lo);
        }

        // ---- out^T[dv][i] in slices of 32 output features: state term, then the score blocks --------
        // (a real loop at D = 128: one slice's temporaries live at a time.  The fully unrolled form was also
        // WRONG there: the slices at features 32 and 64 lost the key features 96..127 of the state term,
        // with the published state intact and every immediate offset of the reads in range; the cause was
        // not found, so the unrolled form stays out for D = 128.)
        constexpr int kSliceUnroll = KS > 2 ? 1 : KS;
#pragma unroll kSliceUnroll
        for (int ks = 0; ks < KS; ++ks) {
            const int fo = 32 * ks;
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    const D8 sh = ld8(St + L.own + (fo + 4 * tt) * LS + 32 * k2);
                    acc[tt] = mma_d(ld8(Sl + L.own + (fo + 4 * tt) * LS + 32 * k2), qb[k2], acc[tt]);
                    acc[tt] = mma_d(sh, ql[k2], acc[tt]);
                    acc[tt] = mma_d(sh, qb[k2], acc[tt]);
                }
            }
#pragma unroll
            for (int J = 0; J < NB; ++J) {
                if (J <= w) {
                    const T4 b4 = J == w ? scD : sc[J], l4 = J == w ? slD : sl[J];
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) {
                        const T4 va = lds_tr4(Vn + L.k4 + fo + 4 * tt + 16 * J * LS, LS);
                        acc[tt] = mma_t(va, l4, acc[tt]);
                        acc[tt] = mma_t(va, b4, acc[tt]);
                    }
                }
            }
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = acc[e >> 2][e & 3];
            if (valid) OutPack<TO>::store(out + row + fo + 8 * c, o);
        }
        }   // !STATE

        // The next block's rows are requested only here: the registers that receive them are not held through
        // the score and output phases above, and the update below is long enough for them to arrive.
        if (n + 1 < N) fetch(n + 1);

        // ---- state update: S <- S e^{tau_J} + V_J^T (k e^{tau_J - l})_J over the sub-blocks in order ------
#pragma unroll
        for (int J = 0; J < NB; ++J) {
            float rr[NTW];
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) rr[nt] = rtab[J * D + 16 * (nt0 + nt) + r];
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                auto va = lds_tr4(Vn + ptl + 16 * J * LS + 16 * (wv + i * NDV), LS);
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) S[i][nt][e] *= rr[nt];
                    S[i][nt] = mma_t(va, lds_tr4(Kl + ptl + 16 * J * LS + 16 * (nt0 + nt), LS), S[i][nt]);
                    S[i][nt] = mma_t(va, lds_tr4(Kh + ptl + 16 * J * LS + 16 * (nt0 + nt), LS), S[i][nt]);
                }
            }
        }
        __syncthreads();                     // every wave is done with the tiles and the old state
        if constexpr (!STATE) publish_state();
    }

    if constexpr (STATE) {
        // (the loop's last barrier is behind every wave's additions)
        if (gate_sums && threadIdx.x < D) {
            float t = 0.f;
#pragma unroll
            for (int m = 0; m < NB; ++m) t += gsum[m * D + threadIdx.x];
            gate_sums[bh * D + threadIdx.x] = t * (1.f / kLog2e);
        }
    }
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            float t4[4] = {S[i][nt][0], S[i][nt][1], S[i][nt][2], S[i][nt][3]};
            store_hidden<4>(hT, hdt, bh * D * D + (int64_t)(16 * (nt0 + nt) + r) * D + 16 * (wv + i * NDV) + 4 * c, t4);
        }
}

template <typename TO, int C, int D, bool STATE = false>
static int launch_one(hipStream_t st, int B, int T_len, int H, int reverse, int hdt, const void *h0, const float *g,
                      const void *v, const void *k, const void *q, void *hT, void *out, int g_shift = 0,
                      float *gate_sums = nullptr)
{
    typedef __bf16 T;
    constexpr int LS = TileGeom<T, D>::kStride;
    // (the lean form has no copy of the state in LDS; its table of decays moves up to where that copy would start)
    const size_t lds = (size_t)(3 * C + (STATE ? 0 : 2 * D)) * LS * sizeof(T) +
                       (size_t)(C / 16) * (STATE ? 2 : 1) * D * sizeof(float);
    auto kern = recurrent_stream_fwd_kernel<TO, C, D, STATE>;
    static LdsGrant grant;
    if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
    dim3 grid(H, B), block(C * 4);
    hipLaunchKernelGGL(kern, grid, block, lds, st, h0, g, (const T *)v, (const T *)k, (const T *)q, hT, (TO *)out,
                       T_len, H, reverse, hdt, g_shift, gate_sums);
    return launch_status();
}

template <typename TO>
int launch_recurrent_stream_fwd(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt,
                                const void *h0, const float *g, const void *v, const void *k, const void *q,
                                void *hT, void *out)
{
    if (D == 64) return launch_one<TO, 128, 64>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, hT, out);
    if (D == 128) return launch_one<TO, 64, 128>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, hT, out);
    return GLA_ERR_UNSUPPORTED;
}

int launch_recurrent_stream_state(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, const void *h0,
                                 const float *g, const void *v, const void *k, const void *q, void *hT, int g_shift,
                                 float *gate_sums)
{
    if (g_shift < -1 || g_shift > 1 || (g_shift && gate_sums)) return GLA_ERR_SHAPE;
    if (D == 64)
        return launch_one<__bf16, 128, 64, true>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, hT, nullptr, g_shift,
                                                 gate_sums);
    if (D == 128)
        return launch_one<__bf16, 64, 128, true>(st, B, T_len, H, reverse, hdt, h0, g, v, k, q, hT, nullptr, g_shift,
                                                 gate_sums);
    return GLA_ERR_UNSUPPORTED;
}

template int launch_recurrent_stream_fwd<__bf16>(hipStream_t, int, int, int, int, int, int, const void *,
                                                 const float *, const void *, const void *, const void *,
                                                 void *, void *);
template int launch_recurrent_stream_fwd<float>(hipStream_t, int, int, int, int, int, int, const void *,
                                                const float *, const void *, const void *, const void *,
                                                void *, void *);

}  // namespace gla
