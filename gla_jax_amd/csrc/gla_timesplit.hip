// recurrent_gla on fewer sequences than the GPU has compute units: a sequence as S segments side by side.
//
// The recurrent kernels walk one (batch, head) pair per workgroup, step after step, so B*H workgroups are all
// the parallelism a call has; with 64 pairs three quarters of the chip idle.  The recurrence is linear in the
// state: with the L steps of segment p applied to a zero state giving loc_p, and a_p the product of its decays,
//     state entering segment p+1 = a_p * (state entering segment p) + loc_p,
// so one pass over all segments at once (zero initial states) yields every loc_p, a scan over the S segments the
// entering states, and a second pass, again over all segments at once, the outputs: a [B,T,H,D] array is a
// [B*S,T/S,H,D] array as it lies, so the segments are batch entries of the same kernels.  The backward needs the
// cotangent of the state at every segment's end as well: it obeys the same kind of recurrence against time, with
// query in the place of key, dout in the place of value and the decays moved by one step (the decay between
// two steps belongs to the later one).  States cross segments in fp32.
// This file holds the small kernels around those passes: the scan over segments, a float array as two bf16 arrays
// (an fp32 dout beside bf16 data) and, for the cases whose first pass is a full kernel (fp32 data, head dimensions 16
// and 32; the lean kernel of the others does these itself), the segments' gate sums, the gates moved by one row and
// a zero fill.
#include "gla_timesplit.hpp"

namespace gla {

namespace {

// One workgroup per (b, p, h): D/4 lanes cover a row (4 floats each), 256/(D/4) rows in flight, LDS for the rest.
template <int D>
__global__ __launch_bounds__(256) void segment_gate_sums_kernel(const float *__restrict__ g, float *__restrict__ sums,
                                                                int L, int H)
{
    constexpr int kLanes = D / 4, kRows = 256 / kLanes;
    __shared__ f32x4 part[kRows][kLanes];
    const int64_t seg = blockIdx.x / H;                 // b*S + p: segments of one batch entry lie one after another
    const int h = blockIdx.x % H;
    const int lane = threadIdx.x % kLanes, r = threadIdx.x / kLanes;
    const float *row = g + ((seg * L + r) * H + h) * (int64_t)D + 4 * lane;
    const int64_t step = (int64_t)kRows * H * D;
    // eight rows requested before the first is added: a workgroup has one wave per SIMD and nothing else to hide
    // the trip behind (one load at a time ran at 2.3 TB/s)
    constexpr int kAhead = 8;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    int t = r;
    for (; t + (kAhead - 1) * kRows < L; t += kAhead * kRows, row += kAhead * step) {
        f32x4 x[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) x[u] = *reinterpret_cast<const f32x4 *>(row + u * step);
#pragma unroll
        for (int u = 0; u < kAhead; ++u) acc += x[u];
    }
    for (; t < L; t += kRows, row += step) acc += *reinterpret_cast<const f32x4 *>(row);
    part[r][lane] = acc;
    __syncthreads();
    if (r == 0) {
#pragma unroll 4
        for (int i = 1; i < kRows; ++i) acc += part[i][lane];
        *reinterpret_cast<f32x4 *>(sums + ((seg * H + h) * (int64_t)D + 4 * lane)) = acc;
    }
}

// dst row t = src row t + dir of the same batch entry, zeros where there is none; 4 floats per thread
__global__ __launch_bounds__(256) void shift_rows_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                         int64_t n4, int64_t T, int64_t row4, int dir)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const int64_t t = i / row4 % T + dir;
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
    if (t >= 0 && t < T) x = *reinterpret_cast<const f32x4 *>(src + (i + dir * row4) * 4);
    *reinterpret_cast<f32x4 *>(dst + i * 4) = x;
}

// One thread per 4 neighbouring value features of a (b, h, dk) state row, a loop over the segments.  The
// contributions may come in pieces: every segment as F consecutive pieces of Lf steps each (S*F pieces per batch
// entry, loc / loc2 / sums indexed by piece); `entering` is stored per segment, before its first piece.
// loc2 (may be null) is a second array of contributions, added to the first.
__global__ __launch_bounds__(256) void segment_scan_kernel(const void *__restrict__ init, const float *__restrict__ loc,
                                                           const float *__restrict__ loc2,
                                                           const float *__restrict__ sums,
                                                           const float *__restrict__ g, float *__restrict__ entering,
                                                           void *__restrict__ final, int64_t n4, int S, int F, int Lf,
                                                           int H, int D, int hdt, int edge_row, int descending)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const int64_t e = i * 4;                            // element of a [B][H][D][D] array
    const int64_t dd = (int64_t)D * D;
    const int64_t b = e / (dd * H);
    const int h = (int)(e / dd % H), dk = (int)(e / D % D);
    const int64_t in_state = e % dd;
    const int P = S * F;
    float x[4];
    load_hidden<4>(init, hdt, e, x);
    // Only x ties one piece to the next; what a piece reads does not depend on it.  Eight pieces' reads are issued
    // before the first of them is used: with few sequences there are few threads here and many pieces, and one
    // piece per memory round trip made this kernel the longest of a call (36 us at 64 pieces of B1 T8192 H2 D64).
    constexpr int kAhead = 8;
    for (int j0 = 0; j0 < P; j0 += kAhead) {
        f32x4 l[kAhead];
        float a[kAhead], w[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int j = j0 + u < P ? j0 + u : P - 1;      // (past the end: the last piece again, not used)
            const int pf = descending ? P - 1 - j : j;      // the piece, in the order the recurrence meets them
            const int64_t piece = b * P + pf;
            const int64_t o = (piece * H + h) * dd + in_state;
            l[u] = *reinterpret_cast<const f32x4 *>(loc + o);
            if (loc2) l[u] += *reinterpret_cast<const f32x4 *>(loc2 + o);
            a[u] = sums[(piece * H + h) * (int64_t)D + dk];
            w[u] = g ? g[((piece * Lf + edge_row) * H + h) * (int64_t)D + dk] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int j = j0 + u;
            if (j < P) {
                const int pf = descending ? P - 1 - j : j;
                if (j % F == 0)
                    *reinterpret_cast<f32x4 *>(entering + (((b * S + pf / F) * H + h) * dd + in_state)) =
                        f32x4{x[0], x[1], x[2], x[3]};
                const float ea = expf(a[u]), ew = expf(w[u]);
#pragma unroll
                for (int c = 0; c < 4; ++c) x[c] = ea * x[c] + ew * l[u][c];
            }
        }
    }
    if (final) store_hidden<4>(final, hdt, e, x);
}

// hi = the bf16 nearest to x, lo = the bf16 nearest to what that leaves over; 8 elements per thread
__global__ __launch_bounds__(256) void head_remainder_kernel(const float *__restrict__ x, __bf16 *__restrict__ hi,
                                                             __bf16 *__restrict__ lo, int64_t n8)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    float a[8], h[8], l[8];
    load_vec<float, 8>(x + i * 8, a);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        h[j] = (float)(__bf16)a[j];
        l[j] = a[j] - h[j];
    }
    store_vec<__bf16, 8>(hi + i * 8, h);
    store_vec<__bf16, 8>(lo + i * 8, l);
}

__global__ __launch_bounds__(256) void zero_fill_kernel(f32x4 *__restrict__ dst, int64_t n16)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) dst[i] = f32x4{0.f, 0.f, 0.f, 0.f};
}

inline bool grid_fits(int64_t threads) { return (threads + 255) / 256 <= 0x7fffffffLL; }
inline dim3 grid_for(int64_t threads) { return dim3((unsigned)((threads + 255) / 256)); }

}  // namespace

int launch_segment_gate_sums(hipStream_t st, int64_t B, int64_t S, int64_t L, int64_t H, int D, const float *g,
                             float *sums)
{
    if (B * S * H > 0x7fffffffLL || L > 0x7fffffffLL) return GLA_ERR_SHAPE;
    const dim3 grid((unsigned)(B * S * H)), block(256);
#define GLA_SUMS_CASE(D_)                                                                                       \
    case D_: hipLaunchKernelGGL(segment_gate_sums_kernel<D_>, grid, block, 0, st, g, sums, (int)L, (int)H); break
    switch (D) {
    GLA_SUMS_CASE(16);
    GLA_SUMS_CASE(32);
    GLA_SUMS_CASE(64);
    GLA_SUMS_CASE(128);
    GLA_SUMS_CASE(256);
    default: return GLA_ERR_SHAPE;
    }
#undef GLA_SUMS_CASE
    return launch_status();
}

int launch_shift_rows(hipStream_t st, int64_t B, int64_t T, int64_t row_len, const float *src, float *dst, int dir)
{
    if (row_len % 4 != 0 || (dir != 1 && dir != -1)) return GLA_ERR_SHAPE;
    const int64_t n4 = B * T * row_len / 4;
    if (!grid_fits(n4)) return GLA_ERR_SHAPE;
    hipLaunchKernelGGL(shift_rows_kernel, grid_for(n4), dim3(256), 0, st, src, dst, n4, T, row_len / 4, dir);
    return launch_status();
}

int launch_segment_scan(hipStream_t st, int64_t B, int64_t S, int64_t F, int64_t Lf, int64_t H, int D, int hdt,
                        const void *init, const float *loc, const float *loc2, const float *sums, const float *g,
                        int edge_row, int descending, float *entering, void *final)
{
    const int64_t n4 = B * H * D * D / 4;
    if (!grid_fits(n4) || S * F > 0x7fffffffLL || Lf > 0x7fffffffLL || F < 1) return GLA_ERR_SHAPE;
    hipLaunchKernelGGL(segment_scan_kernel, grid_for(n4), dim3(256), 0, st, init, loc, loc2, sums, g, entering, final, n4,
                       (int)S, (int)F, (int)Lf, (int)H, D, hdt, edge_row, descending);
    return launch_status();
}

int launch_head_remainder(hipStream_t st, int64_t n, const float *x, void *hi, void *lo)
{
    if (n % 8 != 0 || !grid_fits(n / 8)) return GLA_ERR_SHAPE;
    hipLaunchKernelGGL(head_remainder_kernel, grid_for(n / 8), dim3(256), 0, st, x, (__bf16 *)hi, (__bf16 *)lo, n / 8);
    return launch_status();
}

int launch_zero_fill(hipStream_t st, void *dst, size_t n)
{
    if (n % 16 != 0) return GLA_ERR_SHAPE;
    const int64_t n16 = (int64_t)(n / 16);
    if (!grid_fits(n16)) return GLA_ERR_SHAPE;
    hipLaunchKernelGGL(zero_fill_kernel, grid_for(n16), dim3(256), 0, st, (f32x4 *)dst, n16);
    return launch_status();
}

}  // namespace gla
