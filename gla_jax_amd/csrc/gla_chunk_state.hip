// Inter-chunk state path of chunk_gla (gla.py:695-729 forward, gla.py:731-790 backward):
//
//   chunk_outer_kernel   per chunk n:  P_n^T[dv][dk] = sum_j X[j][dv] * Y~[j][dk]     (bf16 MFMA, fp32 out)
//        forward:  X = value, Y~ = key   * exp(L_end - L_j)   -> kv_n      (gla.py:705-708)
//        backward: X = dout,  Y~ = query * exp(L_j)           -> dstate_n  (gla.py:748-750)
//     and the chunk decay exp(L_end) per feature.
//   chunk_scan_kernel    over chunks:  S_{n+1} = decay_n * S_n + P_n  (ops.py:286-297 combine op), written
//     as the chunk-START states the output kernel needs (gla.py:720-723); run backwards it is the
//     reverse scan of gla.py:759-765 and yields the gradient w.r.t. every chunk-END state.  Both
//     orientations of the state are written, each consumer reads the one whose rows it contracts.
//
// L is the within-chunk inclusive cumsum of log_fgate (gla.py:509), never written to memory: each
// wave scans its 16 tokens across lanes, block totals go through a small LDS table.
// States are consumed as the A operand of (feature x token) products: [dv][dk] where the product
// contracts over dk, [dk][dv] where it contracts over dv.
#include "gla_chunk_common.hpp"
#include "gla_chunk_kernels.hpp"

namespace gla {

// Two tiles and a table fit twice into a CU's LDS; the register budget is held to what lets two
// workgroups share a CU, so that one loads while the other computes.
template <typename T, int C, int D, int DM, int MODE>
__global__ __launch_bounds__(C * 4) __attribute__((amdgpu_waves_per_eu(C / 32, C / 32))) void chunk_outer_kernel(const float *__restrict__ g,
                                                            const T *__restrict__ x,
                                                            const T *__restrict__ y,
                                                            float *__restrict__ prodT,
                                                            float *__restrict__ decay, int T_len, int H)
{
    constexpr int NB = C / 16, KS = D / 32, NV = D / 4, NT = D / 16;
    constexpr int LS = TileGeom<T, D>::kStride;
    extern __shared__ __align__(16) unsigned char smem[];
    T *Xn = reinterpret_cast<T *>(smem);
    T *Yn = Xn + C * LS;
    float *ttab = reinterpret_cast<float *>(Yn + C * LS);   // [NB][D] tau_m: gate total of sub-block m (log2 units)

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: scalar loop bounds below
    const int r = lane & 15, c = lane >> 4;
    // heads vary fastest over the grid: workgroups that run together touch the same DRAM pages of the
    // [B, T, H, D] arrays (a token's H rows are contiguous)
    const int h = blockIdx.x % H, n = blockIdx.x / H, b = blockIdx.y;
    const int N = T_len / C;
    const int64_t tok = (int64_t)b * T_len + (int64_t)n * C + 16 * w + r;
    const int64_t rowoff = (tok * H + h) * DM;     // DM features per row in memory (DM < D: see RowMap)

    float p[NV];
    typename FragTypes<T>::d8 yf[KS], xf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        f32x8 gg = ld8_row<D, DM>(g + rowoff + 32 * ks, c);
#pragma unroll
        for (int e = 0; e < 8; ++e) p[8 * ks + e] = gg.v[e] * kLog2e;
        yf[ks] = ld8_row<D, DM>(y + rowoff + 32 * ks, c);
        xf[ks] = ld8_row<D, DM>(x + rowoff + 32 * ks, c);
    }
    // Gate sums inside the sub-block (log2 units).  The query side needs the inclusive prefix l_i, the key
    // side the sum over the LATER rows, tau - l_j: that one is scanned directly (a suffix scan, then one row
    // down) instead of being formed as a difference, which would cancel against a closed gate (g = -200
    // leaves 3e-5 of absolute error in every later prefix).  The row that ends up with the sub-block total
    // tau (15 for the prefix, 0 for the suffix) publishes it.
#pragma unroll
    for (int i = 0; i < NV; ++i) p[i] = MODE == 0 ? suffix_sum_rows(p[i]) : prefix_sum_rows(p[i]);
    if (r == (MODE == 0 ? 0 : 15)) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) st8(ttab + w * D + 32 * ks + 8 * c, pack8<float>(p + 8 * ks));
    }
    if (MODE == 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) p[i] = dpp_f32<0x101>(p[i]);   // row_shl:1: the next row's sum, 0 past the last
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) st8(Xn + (16 * w + r) * LS + 32 * ks + 8 * c, xf[ks]);
    __syncthreads();
    // The gate sum from a row to the chunk's end (keys) or from its start (queries) adds the totals of the
    // sub-blocks after (before) the wave's own; all sums are <= 0, so ONE exponential per element gives the
    // factor, and the loop bounds are wave-uniform (no per-lane selects).
    const int m_lo = MODE == 0 ? w + 1 : 0, m_hi = MODE == 0 ? NB : w;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * c;
        float sum[8], yv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) sum[e] = p[8 * ks + e];
        for (int m = m_lo; m < m_hi; ++m) {
            f32x8 t = ld8(ttab + m * D + d0);
#pragma unroll
            for (int e = 0; e < 8; ++e) sum[e] += t.v[e];
        }
        unpack8(yf[ks], yv);
#pragma unroll
        for (int e = 0; e < 8; ++e) yv[e] *= fast_exp2(sum[e]);
        st8(Yn + (16 * w + r) * LS + d0, pack8<T>(yv));
    }
    if (w == 0 && r == 0) {
        // chunk decay e^{L_end}: the total over all sub-blocks
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = 32 * ks + 8 * c;
            f32x8 all = ld8(ttab + d0);
            for (int m = 1; m < NB; ++m) {
                f32x8 t = ld8(ttab + m * D + d0);
#pragma unroll
                for (int e = 0; e < 8; ++e) all.v[e] += t.v[e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) all.v[e] = fast_exp2(all.v[e]);
            st8(decay + (((int64_t)b * H + h) * N + n) * D + d0, all);
        }
    }
    __syncthreads();

    float *outp = prodT + (((int64_t)b * H + h) * N + n) * D * D;
    for (int mt = w; mt < NT; mt += NB) {
        f32x4 acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
        const int ptl = plain_tr_lane<T>(LS);
#pragma unroll 2
        for (int J = 0; J < NB; ++J) {
            auto a = lds_tr4(Xn + ptl + 16 * J * LS + 16 * mt, LS);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                auto bb = lds_tr4(Yn + ptl + 16 * J * LS + 16 * nt, LS);
                acc[nt] = mma_t(a, bb, acc[nt]);
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int e = 0; e < 4; ++e) outp[(16 * mt + 4 * c + e) * D + 16 * nt + r] = acc[nt][e];
    }
}

// One thread = a 2x2 patch of the state, one block = one wave = a 16x16 tile (8x8 lanes), walked over the
// chunks in registers.  The running state is written per chunk in BOTH orientations ([dv][dk] for products
// contracting over dk, [dk][dv] for products contracting over dv); with 8x8 lanes of 2x2 patches every
// store instruction fills whole 32-byte sectors either way.  Single-wave blocks spread a state over as many
// CUs as possible: with four-wave blocks the headline shape left a third of the chip with half the work
// (20 -> 18 us), and 8 sequences used 128 CUs (77 -> 60 us).
template <typename T> struct Pair;
template <> struct Pair<__bf16> { typedef bf16x2 type; };
template <> struct Pair<float> { typedef f32x2 type; };

// U = chunks whose inputs are in flight per thread: 4 when the grid fills the machine, 32 when few (b,h)
// pairs leave it to the single thread to keep the memory system busy (long sequences, small batch).
// DM: head dimension of hin / hout in memory (16 when D = 32 stands in for it: rows and columns past DM are zero
// on the way in and are not stored on the way out; the per-chunk buffers are D x D).
template <typename T, int D, int DM, int U>
__global__ __launch_bounds__(64) void chunk_scan_kernel(const void *__restrict__ hin,
                                                         const float *__restrict__ prodT,
                                                         const float *__restrict__ decay,
                                                         T *__restrict__ statesT, T *__restrict__ statesN,
                                                         void *__restrict__ hout, int N, int reverse, int tail,
                                                         int hdt)
{
    typedef typename Pair<T>::type P2;
    constexpr int TPD = D / 32;
    // (b,h) runs along x, the 32x32 tiles along y: workgroups are dealt to the 8 XCDs in x-major order, so when
    // the number of (b,h) pairs is a multiple of 8 all tiles of one state meet in ONE L2.  A tile row is half a
    // 128-byte line of the bf16 states: the halves written by neighbouring tiles are then merged there and
    // leave as whole lines.
    const int bh = blockIdx.x;
    const int tile_v = (blockIdx.y >> 2) / TPD, tile_k = (blockIdx.y >> 2) % TPD;   // 32x32 tile, then its quarter
    const int lane = threadIdx.x, wave = blockIdx.y & 3;
    const int ti = lane >> 3, tj = lane & 7;
    const int dv0 = 32 * tile_v + 16 * (wave >> 1) + 2 * ti;
    const int dk0 = 32 * tile_k + 16 * (wave & 1) + 2 * tj;
    float X[2][2];   // X[i][j] = S[dk0 + j][dv0 + i]
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        // the initial state enters the fp32 running state in its own element type (ops.py:396 takes it uncast,
        // gla.py:711-716); the chunk-start copy of it below is stored in the element type like every other
        // chunk-start state (gla.py:720)
        float t[2] = {0.f, 0.f};
        if (DM == D || (dk0 + j < DM && dv0 < DM))
            load_hidden<2>(hin, hdt, (int64_t)bh * DM * DM + (dk0 + j) * DM + dv0, t);
        X[0][j] = t[0];
        X[1][j] = t[1];
    }
    const float *pp = prodT + (int64_t)bh * N * D * D + dv0 * D + dk0;
    const float *dp = decay + (int64_t)bh * N * D + dk0;
    const int64_t sbase = (int64_t)bh * N * D * D;
    const int64_t sbaseN = (int64_t)bh * (N + tail) * D * D;   // tail: one more slot holds the state after the last chunk
    auto emit = [&](int n) {
        if (statesT) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                P2 t;
                t[0] = X[i][0]; t[1] = X[i][1];
                *reinterpret_cast<P2 *>(statesT + sbase + (int64_t)n * D * D + (dv0 + i) * D + dk0) = t;
            }
        }
        if (statesN) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                P2 t;
                t[0] = X[0][j]; t[1] = X[1][j];
                *reinterpret_cast<P2 *>(statesN + sbaseN + (int64_t)n * D * D + (dk0 + j) * D + dv0) = t;
            }
        }
    };
    int step = 0;
    for (; step + U <= N; step += U) {
        f32x2 pv[U][2], dc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int n = reverse ? N - 1 - (step + u) : step + u;
            pv[u][0] = *reinterpret_cast<const f32x2 *>(pp + (int64_t)n * D * D);
            pv[u][1] = *reinterpret_cast<const f32x2 *>(pp + (int64_t)n * D * D + D);
            dc[u] = *reinterpret_cast<const f32x2 *>(dp + (int64_t)n * D);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int n = reverse ? N - 1 - (step + u) : step + u;
            emit(n);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) X[i][j] = dc[u][j] * X[i][j] + pv[u][i][j];
        }
    }
    for (; step < N; ++step) {
        const int n = reverse ? N - 1 - step : step;
        f32x2 p0 = *reinterpret_cast<const f32x2 *>(pp + (int64_t)n * D * D);
        f32x2 p1 = *reinterpret_cast<const f32x2 *>(pp + (int64_t)n * D * D + D);
        f32x2 dc = *reinterpret_cast<const f32x2 *>(dp + (int64_t)n * D);
        emit(n);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            X[0][j] = dc[j] * X[0][j] + p0[j];
            X[1][j] = dc[j] * X[1][j] + p1[j];
        }
    }
    if (tail && statesN) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            P2 t;
            t[0] = X[0][j]; t[1] = X[1][j];
            *reinterpret_cast<P2 *>(statesN + sbaseN + (int64_t)N * D * D + (dk0 + j) * D + dv0) = t;
        }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const float t[2] = {X[0][j], X[1][j]};
        if (DM == D || (dk0 + j < DM && dv0 < DM))
            store_hidden<2>(hout, hdt, (int64_t)bh * DM * DM + (dk0 + j) * DM + dv0, t);
    }
}

template <typename T, int C, int D, int DM>
int launch_chunk_outer(hipStream_t st, int mode, int B, int T_len, int H, const float *g, const void *x,
                       const void *y, float *prodT, float *decay)
{
    constexpr int LS = TileGeom<T, D>::kStride;
    const size_t lds = (size_t)2 * C * LS * sizeof(T) + (size_t)(C / 16) * D * sizeof(float);
    dim3 grid(T_len / C * H, B), block(C * 4);
    if (mode == 0) {
        auto kern = chunk_outer_kernel<T, C, D, DM, 0>;
        static LdsGrant grant;
        if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
        hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)x, (const T *)y, prodT, decay, T_len, H);
    } else {
        auto kern = chunk_outer_kernel<T, C, D, DM, 1>;
        static LdsGrant grant;
        if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
        hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)x, (const T *)y, prodT, decay, T_len, H);
    }
    return launch_status();
}

template <typename T, int D, int DM>
int launch_chunk_scan(hipStream_t st, int BH, int N, int reverse, int hdt, const void *hin, const float *prodT,
                      const float *decay, void *statesT, void *statesN, void *hout, int tail)
{
    dim3 grid(BH, (D / 16) * (D / 16)), block(64);
    if ((int64_t)grid.y * BH >= 1024) {      // at least a wave per SIMD
        hipLaunchKernelGGL((chunk_scan_kernel<T, D, DM, 4>), grid, block, 0, st, hin, prodT, decay,
                           (T *)statesT, (T *)statesN, hout, N, reverse, tail, hdt);
    } else {
        hipLaunchKernelGGL((chunk_scan_kernel<T, D, DM, 32>), grid, block, 0, st, hin, prodT, decay,
                           (T *)statesT, (T *)statesN, hout, N, reverse, tail, hdt);
    }
    return launch_status();
}

#define GLA_INST_OUTER(T, C, D, DM)                                                                   \
    template int launch_chunk_outer<T, C, D, DM>(hipStream_t, int, int, int, int, const float *, const void *, \
                                                 const void *, float *, float *);
#define GLA_INST_SCAN(T, D, DM)                                                                       \
    template int launch_chunk_scan<T, D, DM>(hipStream_t, int, int, int, int, const void *, const float *, \
                                             const float *, void *, void *, void *, int);
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_OUTER)
GLA_INST_SCAN(__bf16, 32, 16)
GLA_INST_SCAN(__bf16, 32, 32)
GLA_INST_SCAN(__bf16, 64, 64)
GLA_INST_SCAN(__bf16, 128, 128)
GLA_INST_SCAN(__bf16, 256, 256)
GLA_INST_SCAN(float, 32, 16)
GLA_INST_SCAN(float, 32, 32)
GLA_INST_SCAN(float, 64, 64)
GLA_INST_SCAN(float, 128, 128)

}  // namespace gla
