// recurrent_gla forward and backward for gfx950: the per-timestep rank-1 state update
//   S_t = exp(g_t)[:,None] * S_{t-1} + k_t v_t^T ,   o_t = S_t^T q_t            (gla.py:35-37, 50-96)
// and its two-sweep gradient (gla.py:271-360, 263).  The [DK,DV] state of one (batch, head) pair
// lives in the registers of one workgroup for the whole sequence; nothing but inputs, outputs and
// the final state touches HBM.  fp32 VALU work throughout (the state is fp32, gla.py:89).
//
// Register tiling: a wave owns 16 columns (forward) or 16 rows (backward) of the state; a lane owns
// a 4-wide strip of that and 1/16 of the other dimension, so per step it needs 4 + R inputs per
// operand, does 3*4*R FMAs and its partial sums are reduced over 16 lanes by xor-shuffles.
#include "gla_common.hpp"
#include "gla_recurrent_stream.hpp"
#include "gla_split.hpp"
#include "gla_timesplit.hpp"

namespace gla {

// N consecutive elements kept in their memory format until used (halves register use for bf16).
template <typename T, int N> struct RawVec;
template <int N> struct RawVec<float, N> {
    float v[N];
    __device__ __forceinline__ void load(const float *p) { load_vec<float, N>(p, v); }
    __device__ __forceinline__ float get(int i) const { return v[i]; }
};
template <int N> struct RawVec<__bf16, N> {
    static constexpr int W = (N + 1) / 2;
    uint32_t v[W];
    __device__ __forceinline__ void load(const __bf16 *p)
    {
        if constexpr (N == 1) {
            v[0] = *reinterpret_cast<const uint16_t *>(p);
        } else if constexpr (N % 8 == 0) {
#pragma unroll
            for (int i = 0; i < W; i += 4) {
                uint4 t = *reinterpret_cast<const uint4 *>(p + 2 * i);
                v[i] = t.x; v[i + 1] = t.y; v[i + 2] = t.z; v[i + 3] = t.w;
            }
        } else if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < W; i += 2) {
                uint2 t = *reinterpret_cast<const uint2 *>(p + 2 * i);
                v[i] = t.x; v[i + 1] = t.y;
            }
        } else {
#pragma unroll
            for (int i = 0; i < W; ++i) v[i] = *reinterpret_cast<const uint32_t *>(p + 2 * i);
        }
    }
    __device__ __forceinline__ float get(int i) const
    {
        uint32_t w = v[i >> 1];
        return __uint_as_float((i & 1) ? (w & 0xFFFF0000u) : (w << 16));
    }
};

// Lane l = (a = l >> 4, c = l & 15): the 16 lanes that share `a` are one DPP row, so a sum over c is four
// cross-lane adds inside the VALU (no trip through the LDS crossbar); every lane of the row gets it.
__device__ __forceinline__ float reduce_over_c(float x)
{
    x += dpp_f32<kDppQuadXor1>(x);
    x += dpp_f32<kDppQuadXor2>(x);
    x += dpp_f32<kDppRowHalfMirror>(x);
    x += dpp_f32<kDppRowMirror>(x);
    return x;
}

// ------------------------------------------------------------------------------------------------
// forward.  Block = DV/16 waves = one (b,h); wave w owns state columns [16w, 16w+16); lane (a = l>>4,
// c = l&15) owns rows [c*RK, (c+1)*RK) x columns 16w + [4a, 4a+4).
// ------------------------------------------------------------------------------------------------
template <typename T, typename TO, int RK, int U>
__global__ __launch_bounds__(RK * 64) void recurrent_fwd_kernel(
    const void *__restrict__ h0, const float *__restrict__ g, const T *__restrict__ v,
    const T *__restrict__ k, const T *__restrict__ q, void *__restrict__ hT, TO *__restrict__ out,
    int T_len, int H, int reverse, int hdt)
{
    constexpr int DK = RK * 16, DV = DK;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = lane >> 4, c = lane & 15;
    const int h = blockIdx.x, b = blockIdx.y;
    const int dk0 = c * RK, dv0 = wave * 16 + a * 4;
    const int64_t bh = (int64_t)b * H + h;

    float S[RK][4];
    {
        const int64_t ho = bh * DK * DV + (int64_t)dk0 * DV + dv0;
#pragma unroll
        for (int i = 0; i < RK; ++i) load_hidden<4>(h0, hdt, ho + (int64_t)i * DV, S[i]);
    }
    const int64_t strideK = (int64_t)H * DK, strideV = (int64_t)H * DV;
    const float *gp = g + ((int64_t)b * T_len * H + h) * DK + dk0;
    const T *kp = k + ((int64_t)b * T_len * H + h) * DK + dk0;
    const T *qp = q + ((int64_t)b * T_len * H + h) * DK + dk0;
    const T *vp = v + ((int64_t)b * T_len * H + h) * DV + dv0;
    TO *op = out + ((int64_t)b * T_len * H + h) * DV + dv0;

    struct Step {
        RawVec<float, RK> g;
        RawVec<T, RK> k, q;
        RawVec<T, 4> v;
    };
    auto load_step = [&](Step &s, int step) {
        int t = reverse ? T_len - 1 - step : step;
        s.g.load(gp + t * strideK);
        s.k.load(kp + t * strideK);
        s.q.load(qp + t * strideK);
        s.v.load(vp + t * strideV);
    };
    auto compute = [&](const Step &s, int step) {
        int t = reverse ? T_len - 1 - step : step;
        float vv[4], o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) vv[j] = s.v.get(j);
#pragma unroll
        for (int i = 0; i < RK; ++i) {
            float f = __expf(s.g.get(i)), ki = s.k.get(i), qi = s.q.get(i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                S[i][j] = f * S[i][j] + ki * vv[j];
                o[j] += qi * S[i][j];
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = reduce_over_c(o[j]);
        if (c == 0) store_vec<TO, 4>(op + t * strideV, o);
    };

    Step cur[U], nxt[U];
    const int nblk = T_len / U;
    if (nblk > 0) {
#pragma unroll
        for (int u = 0; u < U; ++u) load_step(cur[u], u);
    }
    for (int blk = 0; blk < nblk; ++blk) {
        if (blk + 1 < nblk) {
#pragma unroll
            for (int u = 0; u < U; ++u) load_step(nxt[u], (blk + 1) * U + u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) compute(cur[u], blk * U + u);
#pragma unroll
        for (int u = 0; u < U; ++u) cur[u] = nxt[u];
    }
    for (int step = nblk * U; step < T_len; ++step) {
        load_step(cur[0], step);
        compute(cur[0], step);
    }
    {
        const int64_t ho = bh * DK * DV + (int64_t)dk0 * DV + dv0;
#pragma unroll
        for (int i = 0; i < RK; ++i) store_hidden<4>(hT, hdt, ho + (int64_t)i * DV, S[i]);
    }
}

// ------------------------------------------------------------------------------------------------
// backward, sweep 1 (same time direction as the forward): recompute S_t, dq_t = S_t do_t.
// Block = DK/16 waves = one (b,h); wave w owns state rows [16w, 16w+16); lane (a, c) owns rows
// 16w + [4a, 4a+4) x columns [c*RV, (c+1)*RV).  Writes dq and, into the d(log_fgate) buffer, q*dq
// in fp32 for sweep 2.
// ------------------------------------------------------------------------------------------------
template <typename T, typename TO, int RV, int U>
__global__ __launch_bounds__(RV * 64) void recurrent_bwd_dq_kernel(
    const void *__restrict__ h0, const float *__restrict__ g, const T *__restrict__ v,
    const T *__restrict__ k, const T *__restrict__ q, const void *__restrict__ dhT,
    const TO *__restrict__ dout, T *__restrict__ dq, float *__restrict__ qdq, int T_len, int H, int reverse,
    int hdt)
{
    constexpr int DV = RV * 16, DK = DV;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = lane >> 4, c = lane & 15;
    const int h = blockIdx.x, b = blockIdx.y;
    const int dk0 = wave * 16 + a * 4, dv0 = c * RV;
    const int64_t bh = (int64_t)b * H + h;

    float S[4][RV];
    {
        const int64_t ho = bh * DK * DV + (int64_t)dk0 * DV + dv0;
#pragma unroll
        for (int i = 0; i < 4; ++i) load_hidden<RV>(h0, hdt, ho + (int64_t)i * DV, S[i]);
    }
    const int64_t strideK = (int64_t)H * DK, strideV = (int64_t)H * DV;
    const int64_t offK = ((int64_t)b * T_len * H + h) * DK + dk0;
    const int64_t offV = ((int64_t)b * T_len * H + h) * DV + dv0;

    struct Step {
        RawVec<float, 4> g;
        RawVec<T, 4> k, q;
        RawVec<T, RV> v;
        RawVec<TO, RV> d;
    };
    auto load_step = [&](Step &s, int step) {
        int t = reverse ? T_len - 1 - step : step;
        s.g.load(g + offK + t * strideK);
        s.k.load(k + offK + t * strideK);
        s.q.load(q + offK + t * strideK);
        s.v.load(v + offV + t * strideV);
        s.d.load(dout + offV + t * strideV);
    };
    auto compute = [&](const Step &s, int step) {
        int t = reverse ? T_len - 1 - step : step;
        float acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float f = __expf(s.g.get(i)), ki = s.k.get(i);
            acc[i] = 0.f;
#pragma unroll
            for (int j = 0; j < RV; ++j) {
                S[i][j] = f * S[i][j] + ki * s.v.get(j);
                acc[i] += S[i][j] * s.d.get(j);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = reduce_over_c(acc[i]);
        if (c == 0) {
            float w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = acc[i] * s.q.get(i);
            store_vec<T, 4>(dq + offK + t * strideK, acc);
            store_vec<float, 4>(qdq + offK + t * strideK, w);
        }
    };

    Step cur[U], nxt[U];
    const int nblk = T_len / U;
    if (nblk > 0) {
#pragma unroll
        for (int u = 0; u < U; ++u) load_step(cur[u], u);
    }
    for (int blk = 0; blk < nblk; ++blk) {
        if (blk + 1 < nblk) {
#pragma unroll
            for (int u = 0; u < U; ++u) load_step(nxt[u], (blk + 1) * U + u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) compute(cur[u], blk * U + u);
#pragma unroll
        for (int u = 0; u < U; ++u) cur[u] = nxt[u];
    }
    for (int step = nblk * U; step < T_len; ++step) {
        load_step(cur[0], step);
        compute(cur[0], step);
    }
    // The last term of gla.py:263, sum_v dhT * hT per key feature, from the fp32 state this sweep ends with
    // (the stored hidden_final is rounded to the element type).  Every d(log_fgate)_t is a sum over the
    // steps s >= t, so the term is added to q*dq of the LAST step and reaches all of them through sweep 2's
    // running sum.  The lane that adds it is the one that stored that q*dq.
    {
        const int64_t ho = bh * DK * DV + (int64_t)dk0 * DV + dv0;
        float f4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float d[RV], acc = 0.f;
            load_hidden<RV>(dhT, hdt, ho + (int64_t)i * DV, d);
#pragma unroll
            for (int j = 0; j < RV; ++j) acc += d[j] * S[i][j];
            f4[i] = reduce_over_c(acc);
        }
        if (c == 0) {
            float *lp = qdq + offK + (int64_t)(reverse ? 0 : T_len - 1) * strideK;
            float w[4];
            load_vec<float, 4>(lp, w);
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] += f4[i];
            store_vec<float, 4>(lp, w);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// backward, sweep 2 (against the forward's time direction), same tiling as sweep 1:
//   dS = dcarry + q_t do_t^T ; dk_t = dS v_t ; dv_t = dS^T k_t ; dcarry = exp(g_t) * dS
//   dg_t = sum_{s>=t}(q_s*dq_s - k_s*dk_s) + sum_v(dhT * hT)                      (gla.py:263)
// (sweep 1 has added the last term to q*dq of the last step)
// dv_t needs a sum over all DK rows, i.e. over the waves of the block: the per-wave partial sums of
// TB steps are parked in LDS and combined once per TB steps.
// ------------------------------------------------------------------------------------------------
template <typename T, typename TO, int RV, int TB>
__global__ __launch_bounds__(RV * 64) void recurrent_bwd_rev_kernel(
    const float *__restrict__ g, const T *__restrict__ v, const T *__restrict__ k,
    const T *__restrict__ q, const void *__restrict__ dhT,
    const TO *__restrict__ dout, void *__restrict__ dh0, float *__restrict__ dg, T *__restrict__ dv,
    T *__restrict__ dk, int T_len, int H, int reverse, int hdt)
{
    constexpr int DV = RV * 16, DK = DV, NW = RV;
    __shared__ float part[TB * NW * 4 * DV];   // [slot][wave][a][dv]: partial dv of 4 state rows each
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int a = lane >> 4, c = lane & 15;
    const int h = blockIdx.x, b = blockIdx.y;
    const int dk0 = wave * 16 + a * 4, dv0 = c * RV;
    const int64_t bh = (int64_t)b * H + h;

    float D[4][RV], run[4];   // run: sum over the later steps of q*dq - k*dk (sweep 1 put sum_v dhT*hT into the last q*dq)
    {
        const int64_t ho = bh * DK * DV + (int64_t)dk0 * DV + dv0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            load_hidden<RV>(dhT, hdt, ho + (int64_t)i * DV, D[i]);
            run[i] = 0.f;
        }
    }
    const int64_t strideK = (int64_t)H * DK, strideV = (int64_t)H * DV;
    const int64_t offK = ((int64_t)b * T_len * H + h) * DK + dk0;
    const int64_t offV = ((int64_t)b * T_len * H + h) * DV + dv0;
    const int64_t offVrow = ((int64_t)b * T_len * H + h) * DV;

    struct Step {
        RawVec<float, 4> g, w;
        RawVec<T, 4> k, q;
        RawVec<T, RV> v;
        RawVec<TO, RV> d;
    };
    // logical step s counts along the forward's direction; this sweep walks s = T-1 .. 0
    auto phys = [&](int s) { return reverse ? T_len - 1 - s : s; };
    auto load_step = [&](Step &s, int step) {
        int t = phys(step);
        s.g.load(g + offK + t * strideK);
        s.w.load(dg + offK + t * strideK);
        s.k.load(k + offK + t * strideK);
        s.q.load(q + offK + t * strideK);
        s.v.load(v + offV + t * strideV);
        s.d.load(dout + offV + t * strideV);
    };
    auto compute = [&](const Step &s, int step, int slot) {
        int t = phys(step);
        float dkk[4], dvv[RV];
#pragma unroll
        for (int j = 0; j < RV; ++j) dvv[j] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float f = __expf(s.g.get(i)), ki = s.k.get(i), qi = s.q.get(i);
            dkk[i] = 0.f;
#pragma unroll
            for (int j = 0; j < RV; ++j) {
                float d = D[i][j] + qi * s.d.get(j);
                dkk[i] += d * s.v.get(j);
                dvv[j] += ki * d;
                D[i][j] = f * d;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) dkk[i] = reduce_over_c(dkk[i]);
        store_vec<float, RV>(part + (((size_t)slot * NW + wave) * 4 + a) * DV + dv0, dvv);
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            run[i] += s.w.get(i) - dkk[i] * s.k.get(i);
            o[i] = run[i];
        }
        if (c == 0) {
            store_vec<T, 4>(dk + offK + t * strideK, dkk);
            store_vec<float, 4>(dg + offK + t * strideK, o);
        }
    };
    auto flush = [&](int first_step, int count) {
        // steps first_step, first_step-1, ... live in slots 0..count-1
        __syncthreads();
        for (int idx = threadIdx.x; idx < count * DV; idx += blockDim.x) {
            int slot = idx / DV, col = idx % DV;
            float s = 0.f;
            for (int w = 0; w < NW * 4; ++w) s += part[((size_t)slot * NW * 4 + w) * DV + col];
            int t = phys(first_step - slot);
            Elem<T>::store(dv + offVrow + t * strideV + col, s);
        }
        __syncthreads();
    };

    Step cur[TB], nxt[TB];
    const int nblk = T_len / TB;
    const int tail = T_len - nblk * TB;
    // the tail (highest logical steps not filling a block) goes first, one step at a time
    for (int i = 0; i < tail; ++i) {
        int step = T_len - 1 - i;
        load_step(cur[0], step);
        compute(cur[0], step, 0);
        flush(step, 1);
    }
    const int top = nblk * TB - 1;
    if (nblk > 0) {
#pragma unroll
        for (int u = 0; u < TB; ++u) load_step(cur[u], top - u);
    }
    for (int blk = 0; blk < nblk; ++blk) {
        const int first = top - blk * TB;
        if (blk + 1 < nblk) {
#pragma unroll
            for (int u = 0; u < TB; ++u) load_step(nxt[u], first - TB - u);
        }
#pragma unroll
        for (int u = 0; u < TB; ++u) compute(cur[u], first - u, u);
        flush(first, TB);
#pragma unroll
        for (int u = 0; u < TB; ++u) cur[u] = nxt[u];
    }
    {
        const int64_t ho = bh * DK * DV + (int64_t)dk0 * DV + dv0;
#pragma unroll
        for (int i = 0; i < 4; ++i) store_hidden<RV>(dh0, hdt, ho + (int64_t)i * DV, D[i]);
    }
}

// ------------------------------------------------------------------------------------------------
template <typename T, typename TO>
static int launch_fwd(hipStream_t st, int B, int T_len, int H, int DK, int DV, int reverse, int hdt,
                      const void *h0, const float *g, const void *v, const void *k, const void *q,
                      void *hT, void *out)
{
    dim3 grid(H, B), block(DV / 16 * 64);
#define GLA_FWD_CASE(RK_, U_)                                                                        \
    hipLaunchKernelGGL((recurrent_fwd_kernel<T, TO, RK_, U_>), grid, block, 0, st, h0, g,            \
                       (const T *)v, (const T *)k, (const T *)q, hT, (TO *)out, T_len, H,            \
                       reverse, hdt)
    switch (DK / 16) {
    case 1: GLA_FWD_CASE(1, 4); break;
    case 2: GLA_FWD_CASE(2, 4); break;
    case 4: GLA_FWD_CASE(4, 4); break;
    case 8: GLA_FWD_CASE(8, 2); break;
    case 16: GLA_FWD_CASE(16, 1); break;
    default: return GLA_ERR_SHAPE;
    }
#undef GLA_FWD_CASE
    return launch_status();
}

template <typename T, typename TO>
static int launch_bwd(hipStream_t st, int B, int T_len, int H, int DK, int DV, int reverse, int hdt,
                      const void *h0, const float *g, const void *v, const void *k, const void *q,
                      const void * /* hidden_final: recomputed in fp32 by sweep 1 */, const void *dhT,
                      const void *dout, void *dh0, float *dg, void *dv, void *dk, void *dq, int wide)
{
    dim3 grid(H, B), block(DK / 16 * 64);
    // bf16 data at head dimensions 64 and 128 runs both sweeps on the matrix cores, whatever the type of dout
    if (sizeof(T) == 2 && (DK == 64 || DK == 128)) {
        const int dout_f32 = sizeof(TO) == 4;
        int e = launch_recurrent_stream_dq(st, B, T_len, H, DK, reverse, hdt, dout_f32, h0, g, v, k, q, dhT, dout, dq,
                                           dg, wide);
        if (e) return e;
        return launch_recurrent_stream_rev(st, B, T_len, H, DK, reverse, hdt, dout_f32, g, v, k, q, dhT, dout, dh0, dg,
                                           dv, dk, wide);
    }
    if (wide && sizeof(T) != 4) return GLA_ERR_UNSUPPORTED;   // float gradients: the matrix-core kernels or float data
#define GLA_BWD_CASE(RV_, U_, TB_)                                                                      \
    do {                                                                                                \
        hipLaunchKernelGGL((recurrent_bwd_dq_kernel<T, TO, RV_, U_>), grid, block, 0, st,               \
                           h0, g, (const T *)v, (const T *)k, (const T *)q,                             \
                           dhT, (const TO *)dout, (T *)dq, dg, T_len, H, reverse, hdt);                 \
        hipLaunchKernelGGL((recurrent_bwd_rev_kernel<T, TO, RV_, TB_>), grid, block, 0, st, g,          \
                           (const T *)v, (const T *)k, (const T *)q, dhT,                               \
                           (const TO *)dout, dh0, dg, (T *)dv, (T *)dk, T_len, H, reverse, hdt);        \
    } while (0)
    switch (DV / 16) {
    case 1: GLA_BWD_CASE(1, 4, 4); break;
    case 2: GLA_BWD_CASE(2, 4, 4); break;
    case 4: GLA_BWD_CASE(4, 4, 4); break;
    case 8: GLA_BWD_CASE(8, 2, 2); break;
    case 16: GLA_BWD_CASE(16, 1, 1); break;
    default: return GLA_ERR_SHAPE;
    }
#undef GLA_BWD_CASE
    return launch_status();
}

static int check_recurrent(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, int dtype,
                           int hidden_dtype, int out_dtype)
{
    if (hidden_dtype != GLA_F32 && hidden_dtype != GLA_BF16) return GLA_ERR_DTYPE;
    if (B <= 0 || T <= 0 || H <= 0 || DK <= 0 || DV <= 0) return GLA_ERR_SHAPE;
    if (B > 65535 || H > 65535 || T > (1 << 30)) return GLA_ERR_SHAPE;
    // the reference requires DK == DV for this path (gla.py:120, 391)
    if (DK != DV || !(DK == 16 || DK == 32 || DK == 64 || DK == 128 || DK == 256)) return GLA_ERR_SHAPE;
    if (dtype != GLA_F32 && dtype != GLA_BF16) return GLA_ERR_DTYPE;
    if (out_dtype != GLA_F32 && out_dtype != GLA_BF16) return GLA_ERR_DTYPE;
    if (out_dtype == GLA_BF16 && dtype == GLA_F32) return GLA_ERR_DTYPE;
    return GLA_OK;
}

}  // namespace gla

// ---- head dimension 256 as four problems of head dimension 128 (gla_split.hip) ---------------------------------
// Two passes of the 128-feature kernels over 2H heads, their results left in fp32 and added with one rounding.
// rows: one [B,T,H,256] array of floats; hid: one [B,2H,128,128] array of states (sized for fp32 states).
namespace gla {
struct SplitSizes {
    size_t rows_e, rows_f32, hid;
    SplitSizes(int64_t B, int64_t T, int64_t H, int dtype)
        : rows_e(round_up256((size_t)B * T * H * 256 * (dtype == GLA_BF16 ? 2 : 4))),
          rows_f32(round_up256((size_t)B * T * H * 256 * 4)), hid(round_up256((size_t)B * 2 * H * 128 * 128 * 4))
    {
    }
    static size_t round_up256(size_t x) { return (x + 255) & ~(size_t)255; }
    // forward: value rows with their halves exchanged, both passes' out, hidden_init and hidden_final in blocks
    size_t fwd() const { return rows_e + 2 * rows_f32 + 4 * hid; }
    // backward: value and dout rows exchanged, both passes' dq, dk, dv, the second pass's d(log_fgate), hidden_init,
    // dhidden_final and dhidden_init in blocks
    size_t bwd() const { return rows_e + rows_f32 + 7 * rows_f32 + 6 * hid; }
};
}  // namespace gla

static int recurrent_fwd_run(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, gla_dtype dtype,
                             gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse, const void *hidden_init,
                             const float *log_fgate, const void *value, const void *key, const void *query,
                             void *hidden_final, void *out)
{
    int rc = gla::check_recurrent(B, T, H, DK, DV, dtype, hidden_dtype, out_dtype);
    if (rc) return rc;
    if (!hidden_init || !log_fgate || !value || !key || !query || !hidden_final || !out)
        return GLA_ERR_NULL;
    const void *ptrs[] = {hidden_init, log_fgate, value, key, query, hidden_final, out};
    for (const void *p : ptrs)
        if (!gla::aligned16(p)) return GLA_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    // bf16 inputs at head dimension 64 or 128 run on the matrix cores, 64 or 128 steps per iteration; fp32 `out`
    // (the recurrent_gla_naive flavour, gla.py:37) is the same kernel storing its fp32 accumulators unrounded
    if (dtype == GLA_BF16 && (DK == 64 || DK == 128)) {
        if (out_dtype == GLA_F32)
            return gla::launch_recurrent_stream_fwd<float>(st, B, T, H, DK, reverse, hidden_dtype, hidden_init,
                                                           log_fgate, value, key, query, hidden_final, out);
        return gla::launch_recurrent_stream_fwd<__bf16>(st, B, T, H, DK, reverse, hidden_dtype, hidden_init,
                                                        log_fgate, value, key, query, hidden_final, out);
    }
    if (dtype == GLA_BF16 && out_dtype == GLA_BF16)
        return gla::launch_fwd<__bf16, __bf16>(st, B, T, H, DK, DV, reverse, hidden_dtype, hidden_init, log_fgate, value,
                                               key, query, hidden_final, out);
    if (dtype == GLA_BF16)
        return gla::launch_fwd<__bf16, float>(st, B, T, H, DK, DV, reverse, hidden_dtype, hidden_init, log_fgate, value,
                                              key, query, hidden_final, out);
    return gla::launch_fwd<float, float>(st, B, T, H, DK, DV, reverse, hidden_dtype, hidden_init, log_fgate, value, key,
                                         query, hidden_final, out);
}

extern "C" int gla_recurrent_fwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                 gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                                 const void *hidden_init, const float *log_fgate, const void *value,
                                 const void *key, const void *query, void *hidden_final, void *out)
{
    return recurrent_fwd_run(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init, log_fgate,
                             value, key, query, hidden_final, out);
}

// ---- a sequence as S segments side by side (gla_timesplit.hip) -------------------------------------------------
// With few (batch, head) pairs (at most half of the GPU's compute units for bf16 data at 64 features and more, a
// quarter otherwise), a call with a workspace runs every sequence as S segments at once: one pass from zero states for the segments' own contributions, a scan over the
// segments, and the real pass with the states that enter each segment (fp32); the backward does the same for
// the states' cotangents.  The segments are batch entries of the same kernels: [B,T,H,D] is [B*S,T/S,H,D].
namespace gla {
constexpr int64_t kComputeUnits = 256;       // MI355X
constexpr int64_t kMinSegment = 128;         // steps: one or two iterations of the kernels (with 256 the small shapes left
                                             // compute units idle: B1 T2048 H4 D128 0.31 -> 0.20 ms, B1 T1024 H8 D64 0.11 -> 0.08)
constexpr int64_t kMinLeanPiece = 256;       // steps of a piece where the lean passes take a segment in two
// bf16 data at head dimensions 64, 128 (and 256 as two passes of 128): the forward kernel has a form that leaves out
// everything but the state
static inline bool has_lean_pass(int dtype, int64_t DK) { return dtype == GLA_BF16 && DK >= 64; }
struct TimeSplit {
    int64_t S = 1, L = 0;
    int64_t F = 1, Lf = 0;       // the lean passes run every segment as F pieces of Lf steps
    size_t hid = 0, hidf = 0, sums = 0;
    TimeSplit(int64_t B, int64_t T, int64_t H, int64_t DK, int dtype)
    {
        const int64_t seqs = B * H * (DK == 256 ? 2 : 1);    // head dimension 256 runs as 2H heads of 128
        // the most segments that divide T into pieces of kMinSegment steps or more without asking for more
        // workgroups than there are compute units
        for (int64_t s = kComputeUnits / (seqs > 0 ? seqs : 1); s > 1; --s)
            if (T % s == 0 && T / s >= kMinSegment && B * s <= 65535) {
                S = s;
                break;
            }
        // At 128 features an iteration of the kernels is 64 steps, and segments of one iteration still pay while they
        // leave half of the compute units idle or more (B1 T2048 H4 D128 0.20 -> 0.17 ms); beyond that a segment's
        // own state, read and written once per pass, outweighs its 64 rows (B1 T8192 H2 D128 0.27 -> 0.29 ms).
        if (DK >= 128 && S > 1 && seqs * S * 2 <= kComputeUnits / 2 && (T / S) % 2 == 0 && T / S / 2 >= 64 &&
            B * S * 2 <= 65535)
            S *= 2;
        // Two segments mean two passes over half the steps each: that pays where the first pass is the lean one (bf16
        // data at 64 features and more: B16 T2048 H8 1.47 -> 1.08 ms at 128 features, 0.44 -> 0.39 ms at 64); where it
        // is a full kernel, from four segments on.
        const bool heavy = dtype == GLA_BF16 && DK >= 128;
        if (S < (has_lean_pass(dtype, DK) ? 2 : 4)) S = 1;
        L = T / S;
        // The lean kernel of 128 features fits a compute unit twice (256 registers, 52 KB of LDS) where the full
        // kernels fit once: its passes take every segment in two pieces (512 workgroups: 100 -> 70 us at 1024 steps
        // per segment), and the scan puts the pieces together.  Pieces of 128 steps are two iterations of the kernel
        // and lose what the second workgroup gains.
        if (S > 1 && heavy && L % 2 == 0 && L / 2 >= kMinLeanPiece && B * S * 2 <= 65535) F = 2;
        Lf = L / F;
        hid = SplitSizes::round_up256((size_t)B * S * H * DK * DK * 4);
        hidf = SplitSizes::round_up256((size_t)B * S * F * H * DK * DK * 4);
        sums = SplitSizes::round_up256((size_t)B * S * F * H * DK * 4);
    }
    bool on() const { return S > 1; }
    // forward: entering states, the pieces' own contributions, gate sums
    size_t fwd() const { return on() ? hid + hidf + sums : 0; }
    // backward: the same, the cotangents that leave the segments, and a second array of contributions for an fp32
    // dout beside bf16 data (two passes)
    size_t bwd() const { return on() ? 2 * hid + 2 * hidf + sums : 0; }
};
static size_t inner_fwd_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int dtype)
{
    return DK == 256 ? SplitSizes(B, T, H, dtype).fwd() : 0;
}
static size_t inner_bwd_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int dtype)
{
    return DK == 256 ? SplitSizes(B, T, H, dtype).bwd() : 0;
}
}  // namespace gla

extern "C" size_t gla_recurrent_fwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                                    gla_dtype dtype)
{
    if (gla::check_recurrent(B, T, H, DK, DV, dtype, GLA_F32, GLA_F32) || 2 * H > 65535) return 0;
    const gla::TimeSplit ts(B, T, H, DK, dtype);      // the passes run on B*S batch entries of L steps: their state blocks count
    return ts.fwd() + gla::inner_fwd_bytes(B * ts.S * ts.F, ts.Lf, H, DK, dtype);
}

extern "C" size_t gla_recurrent_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                                    gla_dtype dtype)
{
    if (gla::check_recurrent(B, T, H, DK, DV, dtype, GLA_F32, GLA_F32) || 2 * H > 65535) return 0;
    const gla::TimeSplit ts(B, T, H, DK, dtype);
    return ts.bwd() + gla::inner_bwd_bytes(B * ts.S * ts.F, ts.Lf, H, DK, dtype);
}

// One pass over whole sequences; arguments checked by the caller.  Head dimension 256 with a workspace: two passes
// of the 128-feature kernels; everything else: the kernels directly.
static int recurrent_fwd_inner(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, gla_dtype dtype,
                               gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse, const void *hidden_init,
                               const float *log_fgate, const void *value, const void *key, const void *query,
                               void *hidden_final, void *out, void *workspace, bool state_only = false,
                               int g_shift = 0, float *gate_sums = nullptr)
{
    // state_only: the caller wants hidden_final alone and `out` is a buffer it will overwrite.  The matrix-core
    // kernels have a form without the output products (hidden_init may be null there: zeros); the other kernels
    // write the unused `out`.
    // g_shift (lean passes only): the gates are taken one row further on (+1) or back (-1), see the launcher.
    const bool lean = state_only && dtype == GLA_BF16;
    // gate_sums (lean passes only): the pass also leaves the sum of every sequence's gates there, [B][H][DK].
    if ((g_shift || gate_sums) && !(lean && DK >= 64)) return GLA_ERR_UNSUPPORTED;
    if (lean && (DK == 64 || DK == 128))
        return gla::launch_recurrent_stream_state((hipStream_t)stream, B, T, H, DK, reverse, hidden_dtype, hidden_init,
                                                  log_fgate, value, key, query, hidden_final, g_shift, gate_sums);
    if (DK != 256 || !workspace)
        return recurrent_fwd_run(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init,
                                 log_fgate, value, key, query, hidden_final, out);
    const gla::SplitSizes z(B, T, H, dtype);
    hipStream_t st = (hipStream_t)stream;
    unsigned char *ws = (unsigned char *)workspace;
    unsigned char *v_sw = ws, *out1 = v_sw + z.rows_e, *out2 = out1 + z.rows_f32, *h0_same = out2 + z.rows_f32,
                  *h0_cross = h0_same + z.hid, *hT_same = h0_cross + z.hid, *hT_cross = hT_same + z.hid;
    int e = 0;
    if (hidden_init) {      // (a lean pass may start from zeros: no initial state given)
        e = gla::launch_hidden_blocks(st, hidden_dtype, B * H, const_cast<void *>(hidden_init), h0_same, h0_cross, 1);
        if (e) return e;
    }
    e = gla::launch_swap_halves(st, dtype, B * T * H, v_sw, value);
    if (e) return e;
    // key half a with value half a on the arrays as they lie, then key half a with the other value half; `out` of
    // both in fp32 (the recurrent_gla_naive flavour of the 128-feature kernels)
    if (lean) {
        e = gla::launch_recurrent_stream_state(st, B, T, 2 * H, 128, reverse, hidden_dtype, hidden_init ? h0_same : nullptr,
                                               log_fgate, value, key, query, hT_same, g_shift, gate_sums);
        if (e) return e;
        e = gla::launch_recurrent_stream_state(st, B, T, 2 * H, 128, reverse, hidden_dtype,
                                               hidden_init ? h0_cross : nullptr, log_fgate, v_sw, key, query, hT_cross,
                                               g_shift);
        if (e) return e;
        return gla::launch_hidden_blocks(st, hidden_dtype, B * H, hidden_final, hT_same, hT_cross, 0);
    }
    e = recurrent_fwd_run(stream, B, T, 2 * H, 128, 128, dtype, hidden_dtype, GLA_F32, reverse, h0_same, log_fgate,
                          value, key, query, hT_same, out1);
    if (e) return e;
    e = recurrent_fwd_run(stream, B, T, 2 * H, 128, 128, dtype, hidden_dtype, GLA_F32, reverse, h0_cross, log_fgate, v_sw,
                          key, query, hT_cross, out2);
    if (e) return e;
    e = gla::launch_sum_rows(st, out_dtype, B * T * H, out, (const float *)out1, (const float *)out2, 1);
    if (e) return e;
    return gla::launch_hidden_blocks(st, hidden_dtype, B * H, hidden_final, hT_same, hT_cross, 0);
}

extern "C" int gla_recurrent_fwd_ws(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                    gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                                    const void *hidden_init, const float *log_fgate, const void *value,
                                    const void *key, const void *query, void *hidden_final, void *out,
                                    void *workspace, size_t workspace_bytes)
{
    const size_t need = gla_recurrent_fwd_workspace_bytes(B, T, H, DK, DV, dtype);
    if (!need)      // nothing to gain from a workspace at this shape
        return recurrent_fwd_run(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init,
                                 log_fgate, value, key, query, hidden_final, out);
    int rc = gla::check_recurrent(B, T, H, DK, DV, dtype, hidden_dtype, out_dtype);
    if (rc) return rc;
    const void *ptrs[] = {hidden_init, log_fgate, value, key, query, hidden_final, out};
    for (const void *p : ptrs) {
        if (!p) return GLA_ERR_NULL;
        if (!gla::aligned16(p)) return GLA_ERR_ALIGN;
    }
    if (!workspace || workspace_bytes < need) return GLA_ERR_WORKSPACE;
    if (!gla::aligned16(workspace)) return GLA_ERR_ALIGN;
    const gla::TimeSplit ts(B, T, H, DK, dtype);
    if (!ts.on())
        return recurrent_fwd_inner(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init,
                                   log_fgate, value, key, query, hidden_final, out, workspace);
    hipStream_t st = (hipStream_t)stream;
    unsigned char *ws = (unsigned char *)workspace;
    float *entering = (float *)ws, *loc = (float *)(ws + ts.hid), *sums = (float *)(ws + ts.hid + ts.hidf);
    void *inner_ws = DK == 256 ? ws + ts.fwd() : nullptr;
    const bool lean = gla::has_lean_pass(dtype, DK);
    const int64_t pieces = B * ts.S * ts.F;
    int e = 0;
    if (!lean) {            // (F = 1 then) the full kernels want an initial state, zeros, and leave the gate sums to a kernel
        e = gla::launch_segment_gate_sums(st, B, ts.S * ts.F, ts.Lf, H, (int)DK, log_fgate, sums);
        if (e) return e;
        e = gla::launch_zero_fill(st, entering, ts.hid);
        if (e) return e;
    }
    // every piece from a zero state: its own contribution to the state that leaves it, and its gate sums (where this
    // is a full pass, it writes an `out` that the pass below writes again)
    e = recurrent_fwd_inner(stream, pieces, ts.Lf, H, DK, DV, dtype, GLA_F32, out_dtype, reverse, lean ? nullptr : entering,
                            log_fgate, value, key, query, loc, out, inner_ws, true, 0, lean ? sums : nullptr);
    if (e) return e;
    e = gla::launch_segment_scan(st, B, ts.S, ts.F, ts.Lf, H, (int)DK, hidden_dtype, hidden_init, loc, nullptr, sums,
                                 nullptr, 0, reverse, entering, hidden_final);
    if (e) return e;
    return recurrent_fwd_inner(stream, B * ts.S, ts.L, H, DK, DV, dtype, GLA_F32, out_dtype, reverse, entering,
                               log_fgate, value, key, query, loc, out, inner_ws);
}

// wide != 0: dvalue, dkey, dquery are float arrays whatever `dtype` is
static int recurrent_bwd_run(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, gla_dtype dtype,
                             gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse, const void *hidden_init,
                             const float *log_fgate, const void *value, const void *key, const void *query,
                             const void *hidden_final, const void *dhidden_final, const void *dout,
                             void *dhidden_init, float *dlog_fgate, void *dvalue, void *dkey, void *dquery, int wide)
{
    int rc = gla::check_recurrent(B, T, H, DK, DV, dtype, hidden_dtype, out_dtype);
    if (rc) return rc;
    const void *ptrs[] = {hidden_init, log_fgate, value, key, query, hidden_final, dhidden_final,
                          dout, dhidden_init, dlog_fgate, dvalue, dkey, dquery};
    for (const void *p : ptrs) {
        if (!p) return GLA_ERR_NULL;
        if (!gla::aligned16(p)) return GLA_ERR_ALIGN;
    }
    hipStream_t st = (hipStream_t)stream;
    if (dtype == GLA_BF16 && out_dtype == GLA_BF16)
        return gla::launch_bwd<__bf16, __bf16>(st, B, T, H, DK, DV, reverse, hidden_dtype, hidden_init, log_fgate, value,
                                               key, query, hidden_final, dhidden_final, dout, dhidden_init,
                                               dlog_fgate, dvalue, dkey, dquery, wide);
    if (dtype == GLA_BF16)
        return gla::launch_bwd<__bf16, float>(st, B, T, H, DK, DV, reverse, hidden_dtype, hidden_init, log_fgate, value,
                                              key, query, hidden_final, dhidden_final, dout, dhidden_init,
                                              dlog_fgate, dvalue, dkey, dquery, wide);
    return gla::launch_bwd<float, float>(st, B, T, H, DK, DV, reverse, hidden_dtype, hidden_init, log_fgate, value, key,
                                         query, hidden_final, dhidden_final, dout, dhidden_init, dlog_fgate,
                                         dvalue, dkey, dquery, wide);
}

extern "C" int gla_recurrent_bwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                 gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                                 const void *hidden_init, const float *log_fgate, const void *value,
                                 const void *key, const void *query, const void *hidden_final,
                                 const void *dhidden_final, const void *dout, void *dhidden_init,
                                 float *dlog_fgate, void *dvalue, void *dkey, void *dquery)
{
    return recurrent_bwd_run(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init, log_fgate,
                             value, key, query, hidden_final, dhidden_final, dout, dhidden_init, dlog_fgate, dvalue,
                             dkey, dquery, 0);
}

// One backward over whole sequences; arguments checked by the caller (see recurrent_fwd_inner).
static int recurrent_bwd_inner(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, gla_dtype dtype,
                               gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse, const void *hidden_init,
                               const float *log_fgate, const void *value, const void *key, const void *query,
                               const void *hidden_final, const void *dhidden_final, const void *dout,
                               void *dhidden_init, float *dlog_fgate, void *dvalue, void *dkey, void *dquery,
                               void *workspace)
{
    if (DK != 256 || !workspace)
        return recurrent_bwd_run(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init,
                                 log_fgate, value, key, query, hidden_final, dhidden_final, dout, dhidden_init,
                                 dlog_fgate, dvalue, dkey, dquery, 0);
    const gla::SplitSizes z(B, T, H, dtype);
    hipStream_t st = (hipStream_t)stream;
    unsigned char *ws = (unsigned char *)workspace;
    unsigned char *v_sw = ws, *do_sw = v_sw + z.rows_e, *dg2 = do_sw + z.rows_f32, *dq1 = dg2 + z.rows_f32,
                  *dq2 = dq1 + z.rows_f32, *dk1 = dq2 + z.rows_f32, *dk2 = dk1 + z.rows_f32, *dv1 = dk2 + z.rows_f32,
                  *dv2 = dv1 + z.rows_f32, *h0_same = dv2 + z.rows_f32, *h0_cross = h0_same + z.hid,
                  *dhT_same = h0_cross + z.hid, *dhT_cross = dhT_same + z.hid, *dh0_same = dhT_cross + z.hid,
                  *dh0_cross = dh0_same + z.hid;
    const int64_t rows = B * T * H;
    int e = gla::launch_hidden_blocks(st, hidden_dtype, B * H, const_cast<void *>(hidden_init), h0_same, h0_cross, 1);
    if (e) return e;
    e = gla::launch_hidden_blocks(st, hidden_dtype, B * H, const_cast<void *>(dhidden_final), dhT_same, dhT_cross, 1);
    if (e) return e;
    e = gla::launch_swap_halves(st, dtype, rows, v_sw, value);
    if (e) return e;
    e = gla::launch_swap_halves(st, out_dtype, rows, do_sw, dout);
    if (e) return e;
    // hidden_final is not read by the kernels (sweep 1 forms the final state again in fp32); it is handed on as it is
    e = recurrent_bwd_run(stream, B, T, 2 * H, 128, 128, dtype, hidden_dtype, out_dtype, reverse, h0_same, log_fgate,
                          value, key, query, hidden_final, dhT_same, dout, dh0_same, dlog_fgate, dv1, dk1, dq1, 1);
    if (e) return e;
    e = recurrent_bwd_run(stream, B, T, 2 * H, 128, 128, dtype, hidden_dtype, out_dtype, reverse, h0_cross, log_fgate,
                          v_sw, key, query, hidden_final, dhT_cross, do_sw, dh0_cross, (float *)dg2, dv2, dk2, dq2, 1);
    if (e) return e;
    e = gla::launch_sum_rows(st, dtype, rows, dquery, (const float *)dq1, (const float *)dq2, 0);
    if (e) return e;
    e = gla::launch_sum_rows(st, dtype, rows, dkey, (const float *)dk1, (const float *)dk2, 0);
    if (e) return e;
    e = gla::launch_sum_rows(st, dtype, rows, dvalue, (const float *)dv1, (const float *)dv2, 1);
    if (e) return e;
    e = gla::launch_add_rows(st, GLA_F32, rows, dlog_fgate, dg2, 0);
    if (e) return e;
    return gla::launch_hidden_blocks(st, hidden_dtype, B * H, dhidden_init, dh0_same, dh0_cross, 0);
}

extern "C" int gla_recurrent_bwd_ws(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                    gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                                    const void *hidden_init, const float *log_fgate, const void *value,
                                    const void *key, const void *query, const void *hidden_final,
                                    const void *dhidden_final, const void *dout, void *dhidden_init,
                                    float *dlog_fgate, void *dvalue, void *dkey, void *dquery, void *workspace,
                                    size_t workspace_bytes)
{
    const size_t need = gla_recurrent_bwd_workspace_bytes(B, T, H, DK, DV, dtype);
    if (!need)
        return recurrent_bwd_run(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init,
                                 log_fgate, value, key, query, hidden_final, dhidden_final, dout, dhidden_init,
                                 dlog_fgate, dvalue, dkey, dquery, 0);
    int rc = gla::check_recurrent(B, T, H, DK, DV, dtype, hidden_dtype, out_dtype);
    if (rc) return rc;
    const void *ptrs[] = {hidden_init, log_fgate, value, key, query, hidden_final, dhidden_final,
                          dout, dhidden_init, dlog_fgate, dvalue, dkey, dquery};
    for (const void *p : ptrs) {
        if (!p) return GLA_ERR_NULL;
        if (!gla::aligned16(p)) return GLA_ERR_ALIGN;
    }
    if (!workspace || workspace_bytes < need) return GLA_ERR_WORKSPACE;
    if (!gla::aligned16(workspace)) return GLA_ERR_ALIGN;
    const gla::TimeSplit ts(B, T, H, DK, dtype);
    // The pass for the states' cotangents reads dout where the forward kernels read value, so dout must come in
    // value's type.  An fp32 dout beside bf16 data (the recurrent_gla_naive flavour) is cut into two bf16 arrays, head
    // and remainder, whose passes' states add (the pass is linear in it); that needs the lean kernels, which write no
    // `out`: where there are none (D = 16, 32) such a call runs the sequences whole.
    const bool split_dout = out_dtype != dtype;
    if (!ts.on() || (split_dout && DK < 64))
        return recurrent_bwd_inner(stream, B, T, H, DK, DV, dtype, hidden_dtype, out_dtype, reverse, hidden_init,
                                   log_fgate, value, key, query, hidden_final, dhidden_final, dout, dhidden_init,
                                   dlog_fgate, dvalue, dkey, dquery, DK == 256 ? (unsigned char *)workspace + ts.bwd() : nullptr);
    hipStream_t st = (hipStream_t)stream;
    unsigned char *ws = (unsigned char *)workspace;
    float *entering = (float *)ws, *dleaving = (float *)(ws + ts.hid), *loc = (float *)(ws + 2 * ts.hid),
          *loc_rem = (float *)(ws + 2 * ts.hid + ts.hidf), *sums = (float *)(ws + 2 * ts.hid + 2 * ts.hidf);
    void *inner_ws = DK == 256 ? ws + ts.bwd() : nullptr;      // sized for the backward, which needs more
    const int64_t BS = B * ts.S, pieces = BS * ts.F;
    const bool lean = gla::has_lean_pass(dtype, DK);
    // 1. the states that enter the segments, as the forward formed them (where the pass is a full one, its `out` lands
    //    in dquery, which the backward proper overwrites)
    int e = 0;
    if (!lean) {
        e = gla::launch_segment_gate_sums(st, B, ts.S * ts.F, ts.Lf, H, (int)DK, log_fgate, sums);
        if (e) return e;
        e = gla::launch_zero_fill(st, entering, ts.hid);
        if (e) return e;
        e = gla::launch_zero_fill(st, dleaving, ts.hid);
        if (e) return e;
    }
    e = recurrent_fwd_inner(stream, pieces, ts.Lf, H, DK, DV, dtype, GLA_F32, out_dtype, reverse, lean ? nullptr : entering,
                            log_fgate, value, key, query, loc, dquery, inner_ws, true, 0, lean ? sums : nullptr);
    if (e) return e;
    e = gla::launch_segment_scan(st, B, ts.S, ts.F, ts.Lf, H, (int)DK, hidden_dtype, hidden_init, loc, nullptr, sums,
                                 nullptr, 0, reverse, entering, nullptr);
    if (e) return e;
    // 2. the cotangents of the states that leave the segments.  d(state) obeys the state's recurrence against time
    //    with query for key and dout for value, the decay between two steps being the later step's gate: the same
    //    forward kernels in the other direction with the gates taken one row further on.  The lean kernels read
    //    them there; for the others a copy moved by one row is kept in dlog_fgate until the backward proper writes
    //    there (and the pass's `out` lands in dkey).
    const int shift = reverse ? -1 : 1;
    const float *gates = log_fgate;
    if (!lean) {
        e = gla::launch_shift_rows(st, B, T, H * DK, log_fgate, dlog_fgate, shift);
        if (e) return e;
        gates = dlog_fgate;
    }
    const int gs = lean ? shift : 0;
    const float *loc2 = nullptr;
    if (split_dout) {
        // dkey and dvalue hold the two halves of dout until the backward proper writes its results there
        e = gla::launch_head_remainder(st, B * T * H * DV, (const float *)dout, dkey, dvalue);
        if (e) return e;
        e = recurrent_fwd_inner(stream, pieces, ts.Lf, H, DK, DV, dtype, GLA_F32, dtype, !reverse, nullptr, gates, dkey,
                                query, key, loc, nullptr, inner_ws, true, gs);
        if (e) return e;
        e = recurrent_fwd_inner(stream, pieces, ts.Lf, H, DK, DV, dtype, GLA_F32, dtype, !reverse, nullptr, gates, dvalue,
                                query, key, loc_rem, nullptr, inner_ws, true, gs);
        if (e) return e;
        loc2 = loc_rem;
    } else {
        e = recurrent_fwd_inner(stream, pieces, ts.Lf, H, DK, DV, dtype, GLA_F32, out_dtype, !reverse,
                                lean ? nullptr : dleaving, gates, dout, query, key, loc, dkey, inner_ws, true, gs);
        if (e) return e;
    }
    // what enters segment p from the steps behind it: per piece, the gate of its first step (in the order of the
    // recurrence) times its own contribution, plus its whole decay times what entered from further behind; after
    // the last piece that is dhidden_init
    e = gla::launch_segment_scan(st, B, ts.S, ts.F, ts.Lf, H, (int)DK, hidden_dtype, dhidden_final, loc, loc2, sums,
                                 log_fgate, reverse ? (int)ts.Lf - 1 : 0, !reverse, dleaving, dhidden_init);
    if (e) return e;
    // 3. the backward proper, every segment with its entering state and its leaving cotangent: the gate gradient's
    //    running sum starts from sum_v d(state) * state at the segment's end, which is what the steps behind it add
    return recurrent_bwd_inner(stream, BS, ts.L, H, DK, DV, dtype, GLA_F32, out_dtype, reverse, entering, log_fgate,
                               value, key, query, hidden_final, dleaving, dout, loc, dlog_fgate, dvalue, dkey, dquery,
                               inner_ws);
}
