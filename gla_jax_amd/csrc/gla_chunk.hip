// C-ABI entry points of chunk_gla: argument checks, workspace layout, kernel sequence.
//
// forward  (gla.py:483-550):  outer(kv_n, decay_n)  ->  scan(chunk-start states, hidden_final)  ->  out
// backward (gla.py:552-625):  outer(dstate_n)       ->  reverse scan(d chunk-end states, dhidden_init)
//                             ->  grad (dq, dk, dv, dlog_fgate)
#include "gla_chunk_kernels.hpp"

#include <atomic>

namespace gla {

struct ChunkPlan {
    int C = 0;       // tokens per workgroup actually used (a divisor of chunk_size)
    int D = 0;       // head dimension the kernels work on: DK, or 32 for DK = 16 (rows padded by zeros on the way in)
    size_t prod = 0, decay = 0, states = 0;   // byte sizes, each rounded up to 256
    size_t scale_off = 0;                     // where the products' exponents start inside the decay region
    int bwd_states = 2;                       // arrays of d(chunk-end state): one (tiled) for 16-bit data, both orientations for fp32
    size_t resid = 0;                         // the forward residual: N + 1 states per (b,h), the last one final
    // Head dimension 256 runs as two passes of the 128-feature kernels over 2H heads (gla_split.hip); the
    // sizes above are then those of one such pass, and:
    bool split = false;
    size_t rows = 0;                          // one [B,T,H,256] array of the element type
    size_t rows_f32 = 0;                      // ... of floats
    size_t hid = 0;                           // one [B,2H,128,128] array of states (sized for fp32 states)
    bool wide = false;                        // bf16 data: both passes leave their results in fp32, summed and rounded once
    // forward: value rows with their halves exchanged, the second pass's out (fp32 data) or both passes' (bf16 data),
    // hidden_init and hidden_final in blocks; backward: value and dout rows exchanged, the second pass's dq, dk, dv
    // (or both passes'), its d(log_fgate), the states' cotangents in blocks
    size_t fwd_bytes() const { return prod + decay + states + (split ? rows + (wide ? 2 : 1) * rows_f32 + 4 * hid : 0); }
    size_t bwd_bytes() const
    {
        return prod + decay + bwd_states * states + (split ? 2 * rows + (wide ? 7 : 4) * rows_f32 + 4 * hid : 0);
    }
    size_t resid_bytes() const { return split ? 2 * resid : resid; }
};

static size_t round256(size_t x) { return (x + 255) & ~(size_t)255; }

// The result does not depend on the chunk length (only its rounding does): chunk_size is checked as the
// reference checks it, and the kernels then run with the largest compiled tile that divides T, whatever
// size was asked for (at the headline shape a 64-token tile takes 1.5x, a 32-token tile 2.5x the time of
// the 128-token one: twice or four times the chunk states).  Sizes below 32 tokens are refused: the leaf
// of the reference needs 32 rows as well (gla.py:975-977).
static int plan_chunk(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, int64_t chunk, int dtype,
                      ChunkPlan *plan, int hidden_dtype = GLA_BF16)
{
    if (hidden_dtype != GLA_F32 && hidden_dtype != GLA_BF16) return GLA_ERR_DTYPE;
    if (B <= 0 || T <= 0 || H <= 0 || DK <= 0 || DV <= 0) return GLA_ERR_SHAPE;
    if (B > 65535 || H > 65535 || T > (1 << 30) || B * H > 0x7fffffffLL) return GLA_ERR_SHAPE;   // grid limits
    if (dtype != GLA_F32 && dtype != GLA_BF16) return GLA_ERR_DTYPE;
    if (DK != DV) return GLA_ERR_SHAPE;                      // gla.py:499
    if (!is_pow2(chunk) || T % chunk != 0) return GLA_ERR_CHUNK;   // gla.py:500, 674
    if (chunk < 32) return GLA_ERR_UNSUPPORTED;
    if (DK == 256) {
        int rc = plan_chunk(B, T, 2 * H, 128, 128, chunk, dtype, plan, hidden_dtype);
        if (rc) return rc;
        plan->split = true;
        plan->wide = dtype == GLA_BF16;
        plan->rows = round256((size_t)B * T * H * 256 * (dtype == GLA_BF16 ? 2 : 4));
        plan->rows_f32 = round256((size_t)B * T * H * 256 * sizeof(float));
        plan->hid = round256((size_t)B * 2 * H * 128 * 128 * sizeof(float));
        return GLA_OK;
    }
    // largest tile built: 128 tokens for bf16, for fp32 (tiles twice as wide) 64 at D<=64 and 32 at D=128
    int64_t C = dtype == GLA_BF16 ? 128 : (DK > 64 ? 32 : 64);
    while (T % C != 0) C /= 2;                               // chunk >= 32 divides T, so this stops at 32 or above
    int Dk = 0;
#define GLA_PLAN_CASE(T_, C_, D_, DM_) \
    if (((dtype == GLA_BF16) == (sizeof(T_) == 2)) && C == C_ && DK == DM_) Dk = D_;
    GLA_FOR_EACH_CHUNK_CONFIG(GLA_PLAN_CASE)
#undef GLA_PLAN_CASE
    if (!Dk) return GLA_ERR_UNSUPPORTED;
    plan->D = Dk;
    DK = DV = Dk;                                            // the library's own buffers are sized for the kernels' D
    const size_t N = (size_t)(T / C);
    if ((int64_t)N * H > 0x7fffffffLL) return GLA_ERR_SHAPE;   // chunks x heads is the grid's x extent
    const size_t esz = dtype == GLA_BF16 ? 2 : 4;
    plan->C = (int)C;
    // per-chunk products: float for float data, 16-bit mantissas for bf16 data; their exponents (one byte per 16
    // values) sit behind the decays
    plan->prod = round256((size_t)B * H * N * DK * DV * esz);
    plan->scale_off = (size_t)B * H * N * DK * sizeof(float);
    plan->decay = round256(plan->scale_off + (size_t)B * H * N * (DK * DV / 16));
    plan->states = round256((size_t)B * H * N * DK * DV * esz);
    plan->bwd_states = dtype == GLA_BF16 ? 1 : 2;
    plan->resid = round256((size_t)B * H * (N + 1) * DK * DV * esz);
    return GLA_OK;
}

template <typename F> static int dispatch(int dtype, int C, int DM, F &&f)
{
#define GLA_DISPATCH_CASE(T_, C_, D_, DM_)                                      \
    if (((dtype == GLA_BF16) == (sizeof(T_) == 2)) && C == C_ && DM == DM_)     \
        return f(T_{}, std::integral_constant<int, C_>{}, std::integral_constant<int, D_>{},            \
                 std::integral_constant<int, DM_>{});
    GLA_FOR_EACH_CHUNK_CONFIG(GLA_DISPATCH_CASE)
#undef GLA_DISPATCH_CASE
    return GLA_ERR_UNSUPPORTED;
}

// ---- the statically allocated workspace of gla_chunk_fwd_static ---------------------------------------------
// Device memory that belongs to the library's code object: every GPU the library runs on holds its own copy,
// at its own address, from the moment the code object is loaded there until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress; the address that kernels and copies may use is
// looked up once per device (with that device current) and kept in g_scratch_ptr.
constexpr size_t kStaticScratchBytes = GLA_CHUNK_FWD_STATIC_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices];

static int static_scratch(void **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return GLA_ERR_UNSUPPORTED;
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return GLA_ERR_WORKSPACE;
        g_scratch_ptr[dev].store(p, std::memory_order_release);   // two racing first calls store the same address
    }
    *out = p;
    return GLA_OK;
}

}  // namespace gla

using namespace gla;

extern "C" size_t gla_chunk_states_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                         int64_t chunk_size, gla_dtype dtype)
{
    ChunkPlan p;
    return plan_chunk(B, T, H, DK, DV, chunk_size, dtype, &p) == GLA_OK ? p.resid_bytes() : 0;
}

extern "C" size_t gla_chunk_fwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                                int64_t chunk_size, gla_dtype dtype)
{
    ChunkPlan p;
    // per-chunk products, decays, and the chunk-start states in [dv][dk] orientation for the output kernel
    return plan_chunk(B, T, H, DK, DV, chunk_size, dtype, &p) == GLA_OK ? p.fwd_bytes() : 0;
}

extern "C" size_t gla_chunk_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                                int64_t chunk_size, gla_dtype dtype)
{
    ChunkPlan p;
    // per-chunk products, decays, and d(chunk-end state) in both orientations
    return plan_chunk(B, T, H, DK, DV, chunk_size, dtype, &p) == GLA_OK ? p.bwd_bytes() : 0;
}

// wide != 0 (bf16 data at head dimension 128 only): `out` is a float array
static int chunk_fwd_run(void *stream, int stages, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype, const void *hidden_init,
                         const float *log_fgate, const void *value, const void *key, const void *query,
                         void *hidden_final, void *out, void *states, void *workspace, size_t workspace_bytes,
                         int wide)
{
    ChunkPlan p;
    int rc = plan_chunk(B, T, H, DK, DV, chunk_size, dtype, &p, hidden_dtype);
    if (rc) return rc;
    const void *req[] = {hidden_init, log_fgate, value, key, query, hidden_final, out};
    for (const void *ptr : req) {
        if (!ptr) return GLA_ERR_NULL;
        if (!aligned16(ptr)) return GLA_ERR_ALIGN;
    }
    if (!workspace || workspace_bytes < p.fwd_bytes()) return GLA_ERR_WORKSPACE;
    if (!aligned16(workspace) || (states && !aligned16(states))) return GLA_ERR_ALIGN;
    unsigned char *ws = (unsigned char *)workspace;
    if (p.split) {
        // Two passes of the 128-feature kernels over 2H heads: key half a with value half a on the arrays as they
        // lie, then key half a with the other value half (value rows with their halves exchanged); the second
        // pass's outputs belong to the other half of each row and are added there.
        if (stages != 7) return GLA_ERR_UNSUPPORTED;
        hipStream_t st = (hipStream_t)stream;
        const size_t sub = p.prod + p.decay + p.states;
        if (wide) return GLA_ERR_UNSUPPORTED;
        unsigned char *v_sw = ws + sub, *out2 = v_sw + p.rows, *out1 = out2 + p.rows_f32,
                      *h0_same = out2 + (p.wide ? 2 : 1) * p.rows_f32, *h0_cross = h0_same + p.hid,
                      *hT_same = h0_cross + p.hid, *hT_cross = hT_same + p.hid;
        int e = launch_hidden_blocks(st, hidden_dtype, B * H, const_cast<void *>(hidden_init), h0_same, h0_cross, 1);
        if (e) return e;
        e = launch_swap_halves(st, dtype, B * T * H, v_sw, value);
        if (e) return e;
        e = chunk_fwd_run(stream, 7, B, T, 2 * H, 128, 128, chunk_size, dtype, hidden_dtype, h0_same, log_fgate, value,
                          key, query, hT_same, p.wide ? (void *)out1 : out, states, ws, sub, p.wide);
        if (e) return e;
        e = chunk_fwd_run(stream, 7, B, T, 2 * H, 128, 128, chunk_size, dtype, hidden_dtype, h0_cross, log_fgate, v_sw,
                          key, query, hT_cross, out2, states ? (unsigned char *)states + p.resid : nullptr, ws, sub,
                          p.wide);
        if (e) return e;
        e = p.wide ? launch_sum_rows(st, dtype, B * T * H, out, (const float *)out1, (const float *)out2, 1)
                   : launch_add_rows(st, dtype, B * T * H, out, out2, 1);
        if (e) return e;
        return launch_hidden_blocks(st, hidden_dtype, B * H, hidden_final, hT_same, hT_cross, 0);
    }
    void *prodT = (void *)ws;
    float *decay = (float *)(ws + p.prod);
    unsigned char *pexp = ws + p.prod + p.scale_off;
    void *ws_states = (void *)(ws + p.prod + p.decay);
    hipStream_t st = (hipStream_t)stream;
    const int N = (int)(T / p.C);
    // 16-bit data: ONE array of chunk-start states, tiled, read by the output kernel and (as the residual) by the
    // gradient kernel; without a residual to write it goes to the workspace.  fp32 data: the [dv][dk] copy for the
    // output kernel in the workspace beside the residual.
    const bool tiled = dtype == GLA_BF16;
    void *statesT = tiled ? nullptr : ws_states;
    void *statesN = tiled && !states ? ws_states : states;
    const int tail = statesN == states ? 1 : 0;            // the residual has a slot for the final state
    const void *out_states = tiled ? statesN : statesT;
    const int slots = tiled ? N + tail : N;
    return dispatch(dtype, p.C, (int)DK, [&](auto t, auto c, auto d, auto dm) -> int {
        typedef decltype(t) E;
        constexpr int C_ = decltype(c)::value, D_ = decltype(d)::value, DM_ = decltype(dm)::value;
        int e = 0;
        if (stages & 1)
            e = launch_chunk_outer<E, C_, D_, DM_>(st, 0, (int)B, (int)T, (int)H, log_fgate, value, key, prodT, decay,
                                                   pexp);
        if (e) return e;
        if (stages & 2)
            e = launch_chunk_scan<E, D_, DM_>(st, (int)(B * H), N, 0, hidden_dtype, hidden_init, prodT, decay, pexp,
                                              statesT, statesN, hidden_final, tail, tiled);
        if (e) return e;
        if ((stages & 4) && !wide)
            e = launch_chunk_out<E, C_, D_, DM_>(st, (int)B, (int)T, (int)H, log_fgate, value, key, query, out_states,
                                                 slots, out);
        if ((stages & 4) && wide) {
            if constexpr (sizeof(E) == 2 && D_ == 128 && DM_ == 128)
                e = launch_chunk_out<E, C_, D_, DM_, true>(st, (int)B, (int)T, (int)H, log_fgate, value, key, query,
                                                           out_states, slots, out);
            else
                e = GLA_ERR_UNSUPPORTED;
        }
        return e;
    });
}

extern "C" int gla_chunk_fwd_stages(void *stream, int stages, int64_t B, int64_t T, int64_t H, int64_t DK,
                                    int64_t DV, int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                                    const void *hidden_init,
                                    const float *log_fgate, const void *value, const void *key,
                                    const void *query, void *hidden_final, void *out, void *states,
                                    void *workspace, size_t workspace_bytes)
{
    return chunk_fwd_run(stream, stages, B, T, H, DK, DV, chunk_size, dtype, hidden_dtype, hidden_init, log_fgate,
                         value, key, query, hidden_final, out, states, workspace, workspace_bytes, 0);
}

extern "C" int gla_chunk_fwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                             int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype, const void *hidden_init,
                             const float *log_fgate, const void *value, const void *key, const void *query,
                             void *hidden_final, void *out, void *states, void *workspace,
                             size_t workspace_bytes)
{
    return gla_chunk_fwd_stages(stream, 7, B, T, H, DK, DV, chunk_size, dtype, hidden_dtype, hidden_init, log_fgate,
                                value, key, query, hidden_final, out, states, workspace, workspace_bytes);
}

extern "C" int gla_chunk_fwd_static(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                    int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                                    const void *hidden_init,
                                    const float *log_fgate, const void *value, const void *key,
                                    const void *query, void *hidden_final, void *out, void *states)
{
    ChunkPlan p;
    int rc = plan_chunk(B, T, H, DK, DV, chunk_size, dtype, &p, hidden_dtype);
    if (rc) return rc;
    if (p.fwd_bytes() > kStaticScratchBytes) return GLA_ERR_WORKSPACE;   // beyond the static array
    void *ws = nullptr;
    rc = static_scratch(&ws);
    if (rc) return rc;
    // the workspace needs no clearing: the per-chunk products and decays are written by the first kernel
    // before the scan reads them, the chunk-start states by the scan before the output kernel reads them
    return gla_chunk_fwd_stages(stream, 7, B, T, H, DK, DV, chunk_size, dtype, hidden_dtype, hidden_init, log_fgate,
                                value, key, query, hidden_final, out, states, ws, kStaticScratchBytes);
}

// wide != 0 (bf16 data at head dimension 128 only): `dvalue`, `dkey`, `dquery` are float arrays
static int chunk_bwd_run(void *stream, int stages, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype, const float *log_fgate,
                         const void *value, const void *key, const void *query, const void *states,
                         const void *dhidden_final, const void *dout, void *dhidden_init, float *dlog_fgate,
                         void *dvalue, void *dkey, void *dquery, void *workspace, size_t workspace_bytes, int wide)
{
    ChunkPlan p;
    int rc = plan_chunk(B, T, H, DK, DV, chunk_size, dtype, &p, hidden_dtype);
    if (rc) return rc;
    const void *req[] = {log_fgate, value, key, query, states, dhidden_final, dout,
                         dhidden_init, dlog_fgate, dvalue, dkey, dquery};
    for (const void *ptr : req) {
        if (!ptr) return GLA_ERR_NULL;
        if (!aligned16(ptr)) return GLA_ERR_ALIGN;
    }
    if (!workspace || workspace_bytes < p.bwd_bytes()) return GLA_ERR_WORKSPACE;
    if (!aligned16(workspace)) return GLA_ERR_ALIGN;
    unsigned char *ws = (unsigned char *)workspace;
    if (p.split) {
        // The two passes of the forward again: the first writes its gradients into the caller's arrays, the second
        // into the workspace, from where they are added (those of the value side to the other half of each row).
        if (stages != 7) return GLA_ERR_UNSUPPORTED;
        hipStream_t st = (hipStream_t)stream;
        const size_t sub = p.prod + p.decay + p.bwd_states * p.states;
        if (wide) return GLA_ERR_UNSUPPORTED;
        unsigned char *v_sw = ws + sub, *do_sw = v_sw + p.rows, *dg2 = do_sw + p.rows, *dq2 = dg2 + p.rows_f32,
                      *dk2 = dq2 + p.rows_f32, *dv2 = dk2 + p.rows_f32, *dq1 = dv2 + p.rows_f32,
                      *dk1 = dq1 + p.rows_f32, *dv1 = dk1 + p.rows_f32,
                      *dhT_same = dv2 + (p.wide ? 4 : 1) * p.rows_f32, *dhT_cross = dhT_same + p.hid,
                      *dh0_same = dhT_cross + p.hid, *dh0_cross = dh0_same + p.hid;
        const int64_t rows = B * T * H;
        int e = launch_hidden_blocks(st, hidden_dtype, B * H, const_cast<void *>(dhidden_final), dhT_same, dhT_cross, 1);
        if (e) return e;
        e = launch_swap_halves(st, dtype, rows, v_sw, value);
        if (e) return e;
        e = launch_swap_halves(st, dtype, rows, do_sw, dout);
        if (e) return e;
        e = chunk_bwd_run(stream, 7, B, T, 2 * H, 128, 128, chunk_size, dtype, hidden_dtype, log_fgate, value, key,
                          query, states, dhT_same, dout, dh0_same, dlog_fgate, p.wide ? (void *)dv1 : dvalue,
                          p.wide ? (void *)dk1 : dkey, p.wide ? (void *)dq1 : dquery, ws, sub, p.wide);
        if (e) return e;
        e = chunk_bwd_run(stream, 7, B, T, 2 * H, 128, 128, chunk_size, dtype, hidden_dtype, log_fgate, v_sw, key, query,
                          (const unsigned char *)states + p.resid, dhT_cross, do_sw, dh0_cross, (float *)dg2, dv2, dk2,
                          dq2, ws, sub, p.wide);
        if (e) return e;
        if (p.wide) {
            e = launch_sum_rows(st, dtype, rows, dquery, (const float *)dq1, (const float *)dq2, 0);
            if (e) return e;
            e = launch_sum_rows(st, dtype, rows, dkey, (const float *)dk1, (const float *)dk2, 0);
            if (e) return e;
            e = launch_sum_rows(st, dtype, rows, dvalue, (const float *)dv1, (const float *)dv2, 1);
            if (e) return e;
        } else {
            e = launch_add_rows(st, dtype, rows, dquery, dq2, 0);
            if (e) return e;
            e = launch_add_rows(st, dtype, rows, dkey, dk2, 0);
            if (e) return e;
            e = launch_add_rows(st, dtype, rows, dvalue, dv2, 1);
            if (e) return e;
        }
        e = launch_add_rows(st, GLA_F32, rows, dlog_fgate, dg2, 0);
        if (e) return e;
        return launch_hidden_blocks(st, hidden_dtype, B * H, dhidden_init, dh0_same, dh0_cross, 0);
    }
    void *prodT = (void *)ws;
    float *decay = (float *)(ws + p.prod);
    unsigned char *pexp = ws + p.prod + p.scale_off;
    // d(chunk-end state): for 16-bit data ONE tiled array, for fp32 data [dv][dk] and [dk][dv]
    void *dstatesT = dtype == GLA_BF16 ? nullptr : (void *)(ws + p.prod + p.decay);
    void *dstatesN = (void *)(ws + p.prod + p.decay + (dtype == GLA_BF16 ? 0 : p.states));
    hipStream_t st = (hipStream_t)stream;
    const int N = (int)(T / p.C);
    return dispatch(dtype, p.C, (int)DK, [&](auto t, auto c, auto d, auto dm) -> int {
        typedef decltype(t) E;
        constexpr int C_ = decltype(c)::value, D_ = decltype(d)::value, DM_ = decltype(dm)::value;
        int e = 0;
        if (stages & 1)
            e = launch_chunk_outer<E, C_, D_, DM_>(st, 1, (int)B, (int)T, (int)H, log_fgate, dout, query, prodT, decay,
                                                   pexp);
        if (e) return e;
        if (stages & 2)
            e = launch_chunk_scan<E, D_, DM_>(st, (int)(B * H), N, 1, hidden_dtype, dhidden_final, prodT, decay, pexp,
                                              dstatesT, dstatesN, dhidden_init, 0, dtype == GLA_BF16);
        if (e) return e;
        if ((stages & 4) && !wide)
            e = launch_chunk_grad<E, C_, D_, DM_>(st, (int)B, (int)T, (int)H, log_fgate, value, key, query, dout,
                                                  states, dstatesT, dstatesN, dlog_fgate, dvalue, dkey, dquery);
        if ((stages & 4) && wide) {
            if constexpr (sizeof(E) == 2 && D_ == 128 && DM_ == 128)
                e = launch_chunk_grad<E, C_, D_, DM_, true>(st, (int)B, (int)T, (int)H, log_fgate, value, key, query,
                                                            dout, states, dstatesT, dstatesN, dlog_fgate, dvalue, dkey,
                                                            dquery);
            else
                e = GLA_ERR_UNSUPPORTED;
        }
        return e;
    });
}

extern "C" int gla_chunk_bwd_stages(void *stream, int stages, int64_t B, int64_t T, int64_t H, int64_t DK,
                                    int64_t DV, int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                                    const float *log_fgate,
                                    const void *value, const void *key, const void *query, const void *states,
                                    const void *dhidden_final, const void *dout, void *dhidden_init,
                                    float *dlog_fgate, void *dvalue, void *dkey, void *dquery,
                                    void *workspace, size_t workspace_bytes)
{
    return chunk_bwd_run(stream, stages, B, T, H, DK, DV, chunk_size, dtype, hidden_dtype, log_fgate, value, key, query,
                         states, dhidden_final, dout, dhidden_init, dlog_fgate, dvalue, dkey, dquery, workspace,
                         workspace_bytes, 0);
}

extern "C" int gla_chunk_bwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                             int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype, const float *log_fgate,
                             const void *value,
                             const void *key, const void *query, const void *states,
                             const void *dhidden_final, const void *dout, void *dhidden_init,
                             float *dlog_fgate, void *dvalue, void *dkey, void *dquery, void *workspace,
                             size_t workspace_bytes)
{
    return gla_chunk_bwd_stages(stream, 7, B, T, H, DK, DV, chunk_size, dtype, hidden_dtype, log_fgate, value, key,
                                query, states, dhidden_final, dout, dhidden_init, dlog_fgate, dvalue, dkey, dquery,
                                workspace, workspace_bytes);
}
