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

// The per-chunk products go from the product kernel to the scan and nowhere else, so their layout and type are
// the library's own.  Layout: the order of the matrix instruction's accumulators, [chunk][tile row mt][tile column
// nt][lane][4]: a lane stores the 4 accumulator values of a 16x16 tile with ONE access, a wave one contiguous
// kilobyte or half of it, and the scan's lane (one wave per tile) reads them back the same way.  Type: float for
// float data; for bf16 data a block floating point of 16-bit mantissas with ONE exponent per tile and key
// feature, i.e. per 16 values P[dv = 16 mt .. + 15][dk]: the exponent is that of the largest of the 16, so nothing
// overflows whatever the size of the inputs, a key feature that is orders of magnitude larger than its neighbours
// (or decays away) does not cost them precision, and every value is off by at most 2^-16 of the largest of its
// 16 (the scan adds the products into an fp32 state, so what counts is the absolute error; plain half precision,
// 2^-12 of each value, left hidden_final of a strongly decaying case at 1.6 x its storage rounding, bf16 products
// cost the headline shape the plain 2e-2 bound).  Exponent 255 marks a group that holds a value that is not finite
// (or beyond 2^124): the scan reads all 16 as NaN.  The exponents (one byte each) travel next to the decays.  Half the bytes of fp32 products, written and read
// once per direction: 100 MB less per step at B4 T4096 H6 D128.
template <typename T> struct Prod;
template <> struct Prod<float> { typedef float type; };
template <> struct Prod<__bf16> { typedef short type; };
typedef __attribute__((ext_vector_type(4))) short i16x4;
typedef __attribute__((ext_vector_type(2))) short i16x2;
constexpr int kProdNotFinite = 255;      // the exponent byte of a group with a value that is not finite

// Two tiles and a table fit twice into a CU's LDS; the register budget is held to what lets two
// workgroups share a CU, so that one loads while the other computes.
template <typename T, int C, int D, int DM, int MODE>
__global__ __launch_bounds__(C * 4) __attribute__((amdgpu_waves_per_eu(C / 32, C / 32))) void chunk_outer_kernel(const float *__restrict__ g,
                                                            const T *__restrict__ x,
                                                            const T *__restrict__ y,
                                                            typename Prod<T>::type *__restrict__ prodT,
                                                            float *__restrict__ decay,
                                                            unsigned char *__restrict__ pexp, int T_len, int H)
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
    if (w == (MODE == 0 ? NB - 1 : 0) && r == 0) {
        // chunk decay e^{L_end}: the total over all sub-blocks, formed by the wave that has no totals to add above
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

    const int64_t bhn = ((int64_t)b * H + h) * N + n;
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
        // acc[nt][e] = P^T[dv = 16 mt + 4c + e][dk = 16 nt + r]: stored in this order, one access per tile and lane
        typename Prod<T>::type *outp = prodT + ((bhn * NT + mt) * NT) * 256 + lane * 4;
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) *reinterpret_cast<f32x4 *>(outp + nt * 256) = acc[nt];
        } else {
            unsigned char *expp = pexp + ((bhn * NT + mt) * NT) * 16 + r;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                // the largest magnitude of the key feature's 16 values (4 here, 4 in each of the lanes r + 16 c'); a NaN
                // counts as infinite
                float m = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float a = fabsf(acc[nt][e]);
                    m = fmaxf(m, a == a ? a : __builtin_inff());
                }
                m = fmaxf(m, shfl_xor_f32(m, 16));
                m = fmaxf(m, shfl_xor_f32(m, 32));
                // m = f 2^(eb - 126) with f in [0.5, 1): times 2^(126 - eb) every value lies in (-1, 1), which the
                // packed conversion maps to 16-bit mantissas (x 32767, rounded).  eb is held to a range in which that
                // scale and its inverse are normal floats: an all-zero group takes the smallest exponent of the
                // range, a group beyond it is marked as not finite.
                int eb = (__float_as_int(m) >> 23) & 0xff;
                eb = eb < 27 ? 27 : (eb > 250 ? kProdNotFinite : eb);
                const float sc = __int_as_float((253 - (eb > 250 ? 250 : eb)) << 23);
                const i16x2 lo = __builtin_amdgcn_cvt_pknorm_i16(acc[nt][0] * sc, acc[nt][1] * sc);
                const i16x2 hi = __builtin_amdgcn_cvt_pknorm_i16(acc[nt][2] * sc, acc[nt][3] * sc);
                *reinterpret_cast<i16x4 *>(outp + nt * 256) = i16x4{lo[0], lo[1], hi[0], hi[1]};
                if (c == 0) expp[nt * 16] = (unsigned char)eb;
            }
        }
    }
}

// One block = one wave = one 16x16 tile of the state, walked over the chunks in registers; lane (r, c) holds
// S[dk = 16 nt + r][dv = 16 mt + 4c .. + 3], which is where the product kernel's accumulators of that tile sit.  The
// running state is written per chunk in BOTH orientations ([dv][dk] for products contracting over dk, [dk][dv] for
// products contracting over dv): [dk][dv] takes the lane's 4 values as they are; for [dv][dk] neighbouring lanes
// swap halves first, so that each stores two rows of two neighbouring dk.  Either way every store instruction fills
// whole 32-byte sectors.  Single-wave blocks spread a state over as many CUs as possible: with four-wave blocks the
// headline shape left a third of the chip with half the work (20 -> 18 us), and 8 sequences used 128 CUs (77 -> 60 us).
template <typename T> struct Pair;
template <> struct Pair<__bf16> { typedef bf16x2 type; };
template <> struct Pair<float> { typedef f32x2 type; };

// U = chunks per batch (two batches of inputs are in flight per thread): 8 when the grid fills the machine, 16 when
// few (b,h) pairs leave it to the single thread to keep the memory system busy (long sequences, small batch).
// DM: head dimension of hin / hout in memory (16 when D = 32 stands in for it: rows and columns past DM are zero
// on the way in and are not stored on the way out; the per-chunk buffers are D x D).
template <typename T, int D, int DM, int U>
__global__ __launch_bounds__(64) void chunk_scan_kernel(const void *__restrict__ hin,
                                                         const typename Prod<T>::type *__restrict__ prodT,
                                                         const float *__restrict__ decay,
                                                         const unsigned char *__restrict__ pexp,
                                                         T *__restrict__ statesT, T *__restrict__ statesN,
                                                         void *__restrict__ hout, int N, int reverse, int tail,
                                                         int hdt, int tiled)
{
    typedef typename Pair<T>::type P2;
    typedef typename FragTypes<T>::t4 T4;
    typedef typename Prod<T>::type P;
    constexpr int TPD = D / 32, NT = D / 16;
    // (b,h) runs along x, the 32x32 tiles along y: workgroups are dealt to the 8 XCDs in x-major order, so when
    // the number of (b,h) pairs is a multiple of 8 all tiles of one state meet in ONE L2.  A tile row is half a
    // 128-byte line of the bf16 states: the halves written by neighbouring tiles are then merged there and
    // leave as whole lines.
    const int bh = blockIdx.x;
    const int tile_v = (blockIdx.y >> 2) / TPD, tile_k = (blockIdx.y >> 2) % TPD;   // 32x32 tile, then its quarter
    const int mt = 2 * tile_v + ((blockIdx.y >> 1) & 1), nt = 2 * tile_k + (blockIdx.y & 1);
    const int lane = threadIdx.x, r = lane & 15, c = lane >> 4;
    const int dv0 = 16 * mt + 4 * c, dk = 16 * nt + r;
    const bool in_mem = DM == D || (dk < DM && dv0 < DM);
    float X[4] = {0.f, 0.f, 0.f, 0.f};   // X[e] = S[dk][dv0 + e]
    // the initial state enters the fp32 running state in its own element type (ops.py:396 takes it uncast,
    // gla.py:711-716); the chunk-start copy of it below is stored in the element type like every other
    // chunk-start state (gla.py:720)
    if (in_mem) load_hidden<4>(hin, hdt, (int64_t)bh * DM * DM + dk * DM + dv0, X);
    const P *pp = prodT + (((int64_t)bh * N * NT + mt) * NT + nt) * 256 + lane * 4;   // + n * D * D
    const float *dp = decay + (int64_t)bh * N * D + dk;                               // + n * D
    const unsigned char *ep = pexp + (((int64_t)bh * N * NT + mt) * NT + nt) * 16 + r;   // + n * D * D / 16
    const int64_t sbase = (int64_t)bh * N * D * D;
    const int64_t sbaseN = (int64_t)bh * (N + tail) * D * D;   // tail: one more slot holds the state after the last chunk
    const bool odd = (r & 1) != 0;
    auto emit_n = [&](int64_t slot) {
        T4 t = pack4<T>(f32x4{X[0], X[1], X[2], X[3]});
        *reinterpret_cast<T4 *>(statesN + sbaseN + slot * D * D + (tiled ? state_offset<T, D>(dk, dv0) : dk * D + dv0)) = t;
    };
    auto emit = [&](int n) {
        if (statesT) {
            // lanes r and r^1 swap halves: the even one ends up with rows dv0, dv0 + 1, the odd one with rows
            // dv0 + 2, dv0 + 3, each for the two neighbouring dk of the pair
            float Y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) Y[e] = dpp_f32<kDppQuadXor1>(X[e]);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                P2 t;
                t[0] = odd ? Y[2 + i] : X[i];
                t[1] = odd ? X[2 + i] : Y[i];
                *reinterpret_cast<P2 *>(statesT + sbase + (int64_t)n * D * D + (dv0 + (odd ? 2 : 0) + i) * D +
                                        (dk & ~1)) = t;
            }
        }
        if (statesN) emit_n(n);
    };
    // what a lane asks for per chunk, kept as it arrives until the chunk is worked through (converting it where it
    // is requested would make the lane wait for it there)
    struct Raw {
        typename std::conditional<sizeof(P) == 4, f32x4, i16x4>::type p;
        int eb;
        float dc;
    };
    auto request = [&](int n, Raw &x) {
        x.p = *reinterpret_cast<const decltype(x.p) *>(pp + (int64_t)n * D * D);
        if constexpr (sizeof(P) == 2) x.eb = ep[(int64_t)n * (D * D / 16)];
        x.dc = dp[(int64_t)n * D];
    };
    auto advance = [&](const Raw &x) {
        if constexpr (sizeof(P) == 4) {
#pragma unroll
            for (int e = 0; e < 4; ++e) X[e] = x.dc * X[e] + x.p[e];
        } else {
            const float sc = x.eb == kProdNotFinite ? __builtin_nanf("")
                                                    : __int_as_float((x.eb + 1) << 23) * (1.f / 32767.f);   // 2^(eb - 126) / 32767
#pragma unroll
            for (int e = 0; e < 4; ++e) X[e] = x.dc * X[e] + (float)x.p[e] * sc;
        }
    };
    // Batches of U chunks, the next batch's inputs requested before the current one is worked through: what hides
    // the latency of the loads is the number of bytes on their way.
    auto chunk_of = [&](int step) { return reverse ? N - 1 - step : step; };
    Raw buf[2][U];
    const int nb = N / U;
    if (nb > 0) {
#pragma unroll
        for (int u = 0; u < U; ++u) request(chunk_of(u), buf[0][u]);
    }
    auto batch = [&](int b, auto cur, auto nxt) {
        constexpr int kc = decltype(cur)::value, kn = decltype(nxt)::value;
        if (b + 1 < nb) {
#pragma unroll
            for (int u = 0; u < U; ++u) request(chunk_of((b + 1) * U + u), buf[kn][u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            emit(chunk_of(b * U + u));
            advance(buf[kc][u]);
        }
    };
    for (int b = 0; b < nb; b += 2) {
        batch(b, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
        if (b + 1 < nb) batch(b + 1, std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
    }
    for (int step = nb * U; step < N; ++step) {
        const int n = chunk_of(step);
        Raw x;
        request(n, x);
        emit(n);
        advance(x);
    }
    if (tail && statesN) emit_n(N);
    if (in_mem) store_hidden<4>(hout, hdt, (int64_t)bh * DM * DM + dk * DM + dv0, X);
}

template <typename T, int C, int D, int DM>
int launch_chunk_outer(hipStream_t st, int mode, int B, int T_len, int H, const float *g, const void *x,
                       const void *y, void *prodT, float *decay, unsigned char *pexp)
{
    typedef typename Prod<T>::type P;
    constexpr int LS = TileGeom<T, D>::kStride;
    const size_t lds = (size_t)2 * C * LS * sizeof(T) + (size_t)(C / 16) * D * sizeof(float);
    dim3 grid(T_len / C * H, B), block(C * 4);
    if (mode == 0) {
        auto kern = chunk_outer_kernel<T, C, D, DM, 0>;
        static LdsGrant grant;
        if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
        hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)x, (const T *)y, (P *)prodT, decay, pexp, T_len,
                           H);
    } else {
        auto kern = chunk_outer_kernel<T, C, D, DM, 1>;
        static LdsGrant grant;
        if (int e = allow_lds(grant, (const void *)kern, lds)) return e;
        hipLaunchKernelGGL(kern, grid, block, lds, st, g, (const T *)x, (const T *)y, (P *)prodT, decay, pexp, T_len,
                           H);
    }
    return launch_status();
}

template <typename T, int D, int DM>
int launch_chunk_scan(hipStream_t st, int BH, int N, int reverse, int hdt, const void *hin, const void *prodT,
                      const float *decay, const unsigned char *pexp, void *statesT, void *statesN, void *hout,
                      int tail, int tiled)
{
    typedef typename Prod<T>::type P;
    dim3 grid(BH, (D / 16) * (D / 16)), block(64);
    constexpr int kFew = 8;
    if ((int64_t)grid.y * BH >= 1024) {      // at least a wave per SIMD
        hipLaunchKernelGGL((chunk_scan_kernel<T, D, DM, kFew>), grid, block, 0, st, hin, (const P *)prodT, decay, pexp,
                           (T *)statesT, (T *)statesN, hout, N, reverse, tail, hdt, tiled);
    } else {
        hipLaunchKernelGGL((chunk_scan_kernel<T, D, DM, 16>), grid, block, 0, st, hin, (const P *)prodT, decay, pexp,
                           (T *)statesT, (T *)statesN, hout, N, reverse, tail, hdt, tiled);
    }
    return launch_status();
}

#define GLA_INST_OUTER(T, C, D, DM)                                                                   \
    template int launch_chunk_outer<T, C, D, DM>(hipStream_t, int, int, int, int, const float *, const void *, \
                                                 const void *, void *, float *, unsigned char *);
#define GLA_INST_SCAN(T, D, DM)                                                                       \
    template int launch_chunk_scan<T, D, DM>(hipStream_t, int, int, int, int, const void *, const void *, \
                                             const float *, const unsigned char *, void *, void *, void *, int, int);
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_OUTER)
GLA_INST_SCAN(__bf16, 32, 16)
GLA_INST_SCAN(__bf16, 32, 32)
GLA_INST_SCAN(__bf16, 64, 64)
GLA_INST_SCAN(__bf16, 128, 128)
GLA_INST_SCAN(float, 32, 16)
GLA_INST_SCAN(float, 32, 32)
GLA_INST_SCAN(float, 64, 64)
GLA_INST_SCAN(float, 128, 128)

}  // namespace gla
