// Stand-alone scans of the reference's ops.py as gfx950 kernels:
//   gla_cumsum_f32    <- cumsum_recursive / cumsum_pallas / cumsum_kernel   (ops.py:152-284)
//   gla_rnn_scan_f32  <- rnn_recursive / rnn_pallas / rnn_kernel            (ops.py:286-456)
// Both are HBM-bound streaming kernels: lanes map to the contiguous inner axis so every wave access
// is a full 256-byte row segment, and the scanned axis is walked by the wave in registers.
#include "gla_common.hpp"

namespace gla {

// One block = one outer index x 64 consecutive inner columns.  The scanned axis is cut into WAVES
// contiguous segments, one per wave: pass 1 sums each segment, the segment totals are prefixed
// through LDS, pass 2 re-reads the segment (L2 hit) and writes the running sum.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void cumsum_kernel(const float *__restrict__ src,
                                                            const float *__restrict__ init,
                                                            float *__restrict__ dst, int64_t t_len,
                                                            int64_t n_inner, int reverse)
{
    __shared__ float totals[WAVES][64];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t col = (int64_t)blockIdx.x * 64 + lane;
    const int64_t outer = blockIdx.y;
    const bool valid = col < n_inner;
    const int64_t seg = (t_len + WAVES - 1) / WAVES;
    const int64_t s0 = wave * seg;
    const int64_t s1 = s0 + seg < t_len ? s0 + seg : t_len;
    const float *base = src + outer * t_len * n_inner + col;
    float *obase = dst + outer * t_len * n_inner + col;

    float sum = 0.f;
    if (valid) {
        int64_t s = s0;
        for (; s + 4 <= s1; s += 4) {
            float a[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int64_t t = reverse ? t_len - 1 - (s + u) : s + u;
                a[u] = base[t * n_inner];
            }
            sum += (a[0] + a[1]) + (a[2] + a[3]);
        }
        for (; s < s1; ++s) {
            int64_t t = reverse ? t_len - 1 - s : s;
            sum += base[t * n_inner];
        }
    }
    totals[wave][lane] = sum;
    __syncthreads();
    if (!valid) return;
    float run = init ? init[outer * n_inner + col] : 0.f;
    for (int w = 0; w < wave; ++w) run += totals[w][lane];
    int64_t s = s0;
    for (; s + 4 <= s1; s += 4) {
        float a[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int64_t t = reverse ? t_len - 1 - (s + u) : s + u;
            a[u] = base[t * n_inner];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int64_t t = reverse ? t_len - 1 - (s + u) : s + u;
            run += a[u];
            obase[t * n_inner] = run;
        }
    }
    for (; s < s1; ++s) {
        int64_t t = reverse ? t_len - 1 - s : s;
        run += base[t * n_inner];
        obase[t * n_inner] = run;
    }
}

// The same with the scanned axis cut finer, for long axes over few columns: a block owns CL columns of one
// outer index, a wave covers 64 / CL segments at once (lane = segment-in-wave x column), the block
// WAVES * 64 / CL segments.  A wave access is 64 / CL row pieces of CL floats.
template <int CL, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void cumsum_tiled_kernel(const float *__restrict__ src,
                                                                  const float *__restrict__ init,
                                                                  float *__restrict__ dst, int64_t t_len,
                                                                  int64_t n_inner, int reverse)
{
    constexpr int TG = 64 / CL, NSEG = WAVES * TG;
    __shared__ float totals[NSEG][CL];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cl = lane % CL, segi = wave * TG + lane / CL;
    const int64_t col = (int64_t)blockIdx.x * CL + cl;
    const int64_t outer = blockIdx.y;
    const bool valid = col < n_inner;
    const int64_t seg = (t_len + NSEG - 1) / NSEG;
    const int64_t s0 = segi * seg < t_len ? segi * seg : t_len;
    const int64_t s1 = s0 + seg < t_len ? s0 + seg : t_len;
    const float *base = src + outer * t_len * n_inner + col;
    float *obase = dst + outer * t_len * n_inner + col;

    float sum = 0.f;
    if (valid) {
        int64_t s = s0;
        for (; s + 8 <= s1; s += 8) {
            float a[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) a[u] = base[(reverse ? t_len - 1 - (s + u) : s + u) * n_inner];
            sum += ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
        }
        for (; s < s1; ++s) sum += base[(reverse ? t_len - 1 - s : s) * n_inner];
    }
    totals[segi][cl] = sum;
    __syncthreads();
    if (!valid) return;
    float run = init ? init[outer * n_inner + col] : 0.f;
    for (int w = 0; w < segi; ++w) run += totals[w][cl];
    int64_t s = s0;
    for (; s + 8 <= s1; s += 8) {
        float a[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) a[u] = base[(reverse ? t_len - 1 - (s + u) : s + u) * n_inner];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            run += a[u];
            obase[(reverse ? t_len - 1 - (s + u) : s + u) * n_inner] = run;
        }
    }
    for (; s < s1; ++s) {
        const int64_t t = reverse ? t_len - 1 - s : s;
        run += base[t * n_inner];
        obase[t * n_inner] = run;
    }
}

// The same for segments of at most SEG rows: a thread keeps its whole segment in registers between the two
// passes, so the source is read once (all SEG requests go out before the first sum) and nothing is re-read.
template <int CL, int WAVES, int SEG>
__global__ __launch_bounds__(WAVES * 64) void cumsum_cached_kernel(const float *__restrict__ src,
                                                                   const float *__restrict__ init,
                                                                   float *__restrict__ dst, int64_t t_len,
                                                                   int64_t n_inner, int reverse)
{
    constexpr int TG = 64 / CL, NSEG = WAVES * TG;
    __shared__ float totals[NSEG][CL];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cl = lane % CL, segi = wave * TG + lane / CL;
    const int64_t col = (int64_t)blockIdx.x * CL + cl;
    const int64_t outer = blockIdx.y;
    const bool valid = col < n_inner;
    const int64_t seg = (t_len + NSEG - 1) / NSEG;            // <= SEG, checked by the launcher
    const int64_t s0 = segi * seg < t_len ? segi * seg : t_len;
    const int len = valid ? (int)((s0 + seg < t_len ? s0 + seg : t_len) - s0) : 0;
    // element u of the segment sits `step` rows after the first one (before it when summing from the far end)
    const int64_t first = reverse ? t_len - 1 - s0 : s0;
    const int64_t step = reverse ? -n_inner : n_inner;
    const float *base = src + outer * t_len * n_inner + first * n_inner + (valid ? col : 0);
    float *obase = dst + outer * t_len * n_inner + first * n_inner + (valid ? col : 0);

    float a[SEG];
#pragma unroll
    for (int u = 0; u < SEG; ++u) a[u] = u < len ? base[u * step] : 0.f;
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < SEG; u += 4) sum += (a[u] + a[u + 1]) + (a[u + 2] + a[u + 3]);
    totals[segi][cl] = sum;
    __syncthreads();
    float run = (init && valid) ? init[outer * n_inner + col] : 0.f;
    for (int w = 0; w < segi; ++w) run += totals[w][cl];
#pragma unroll
    for (int u = 0; u < SEG; ++u) {
        run += a[u];
        if (u < len) obase[u * step] = run;
    }
}

// One thread = one (k, W consecutive v) strip of the state, walked over T in registers; the loads
// of step n do not depend on the recurrence, so UNROLL of them are kept in flight.  W = 4 (one
// 16-byte access per step) when V is a multiple of 4, W = 1 for every other V.
template <int W> struct Strip;
template <> struct Strip<4> { typedef f32x4 type; };
template <> struct Strip<1> { typedef float type; };

template <int UNROLL, int W>
__global__ __launch_bounds__(256) void rnn_scan_kernel(const float *__restrict__ a,
                                                       const float *__restrict__ kv,
                                                       const float *__restrict__ init_a,
                                                       const float *__restrict__ init_kv,
                                                       float *__restrict__ out_a,
                                                       float *__restrict__ out_x, int64_t T, int64_t K,
                                                       int64_t V, int reverse)
{
    typedef typename Strip<W>::type X;
    const int64_t vw = V / W;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= K * vw) return;
    const int64_t b = blockIdx.y;
    const int64_t k = idx / vw, vq = idx % vw;
    const float *ab = a + b * T * K + k;
    const X *xb = reinterpret_cast<const X *>(kv + b * T * K * V + k * V) + vq;
    X *ob = reinterpret_cast<X *>(out_x + b * T * K * V + k * V) + vq;
    float *oab = out_a ? out_a + b * T * K + k : nullptr;
    X x = X{};
    if (init_kv) x = reinterpret_cast<const X *>(init_kv + b * K * V + k * V)[vq];
    float ca = init_a ? init_a[b * K + k] : 0.f;
    int64_t s = 0;
    for (; s + UNROLL <= T; s += UNROLL) {
        float av[UNROLL];
        X bv[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int64_t t = reverse ? T - 1 - (s + u) : s + u;
            av[u] = ab[t * K];
            bv[u] = xb[t * K * vw];
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int64_t t = reverse ? T - 1 - (s + u) : s + u;
            float f = __expf(av[u]);
            x = f * x + bv[u];
            ca += av[u];
            ob[t * K * vw] = x;
            if (oab && vq == 0) oab[t * K] = ca;
        }
    }
    for (; s < T; ++s) {
        int64_t t = reverse ? T - 1 - s : s;
        float av = ab[t * K];
        x = __expf(av) * x + xb[t * K * vw];
        ca += av;
        ob[t * K * vw] = x;
        if (oab && vq == 0) oab[t * K] = ca;
    }
}

}  // namespace gla

extern "C" int gla_cumsum_f32(void *stream, const float *src, const float *init, float *dst,
                              int64_t n_outer, int64_t t_len, int64_t n_inner, int reverse)
{
    if (!src || !dst) return GLA_ERR_NULL;
    if (n_outer <= 0 || t_len <= 0 || n_inner <= 0 || n_outer > 65535) return GLA_ERR_SHAPE;
    dim3 grid((unsigned)((n_inner + 63) / 64), (unsigned)n_outer);
    hipStream_t st = (hipStream_t)stream;
    // long axis over few columns: cut the axis finer so that the grid fills the machine
    if (t_len >= 2048 && (int64_t)grid.x * grid.y < 1024) {
        dim3 fine((unsigned)((n_inner + 15) / 16), (unsigned)n_outer);
        if (t_len <= 64 * 64)       // 64 segments of at most 64 rows: held in registers, read once
            hipLaunchKernelGGL((gla::cumsum_cached_kernel<16, 16, 64>), fine, dim3(1024), 0, st, src, init, dst,
                               t_len, n_inner, reverse);
        else
            hipLaunchKernelGGL((gla::cumsum_tiled_kernel<16, 16>), fine, dim3(1024), 0, st, src, init, dst, t_len,
                               n_inner, reverse);
    } else if (t_len >= 64 && t_len <= 4 * 64)
        hipLaunchKernelGGL((gla::cumsum_cached_kernel<64, 4, 64>), grid, dim3(256), 0, st, src, init, dst, t_len,
                           n_inner, reverse);
    else if (t_len >= 64)
        hipLaunchKernelGGL(gla::cumsum_kernel<4>, grid, dim3(256), 0, st, src, init, dst, t_len, n_inner,
                           reverse);
    else
        hipLaunchKernelGGL(gla::cumsum_kernel<1>, grid, dim3(64), 0, st, src, init, dst, t_len, n_inner,
                           reverse);
    return gla::launch_status();
}

extern "C" int gla_rnn_scan_f32(void *stream, const float *log_fgate, const float *kv,
                                const float *init_log_fgate, const float *init_kv,
                                float *out_log_lambda, float *out_state, int64_t batch, int64_t T,
                                int64_t K, int64_t V, int reverse)
{
    if (!log_fgate || !kv || !out_state) return GLA_ERR_NULL;
    if (batch <= 0 || T <= 0 || K <= 0 || V <= 0 || batch > 65535) return GLA_ERR_SHAPE;
    const bool wide = V % 4 == 0;
    if (wide && (!gla::aligned16(kv) || !gla::aligned16(out_state) || (init_kv && !gla::aligned16(init_kv))))
        return GLA_ERR_ALIGN;
    int64_t n = K * (wide ? V / 4 : V);
    dim3 grid((unsigned)((n + 255) / 256), (unsigned)batch);
    auto kern = wide ? gla::rnn_scan_kernel<8, 4> : gla::rnn_scan_kernel<8, 1>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, log_fgate, kv, init_log_fgate, init_kv,
                       out_log_lambda, out_state, T, K, V, reverse);
    return gla::launch_status();
}
