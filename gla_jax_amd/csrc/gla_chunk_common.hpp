// Building blocks of the chunk_gla kernels (gfx950).
//
// Data model.  A workgroup handles one chunk of C tokens of one (batch, head) pair with C/16 waves;
// wave w owns the 16-token sub-block w.  Inside a wave, lane l = (r, c) with r = l % 16 (token row
// of the sub-block) and c = l / 16; the lane holds, for its row, the D/4 feature values
//       d = 32*ks + 8*c + e,   ks = 0..D/32-1, e = 0..7                       ("row layout")
// which is at the same time the A/B operand layout of the K=32 MFMA when the contraction runs over
// d (lane (row, c) supplies k-slots 8c..8c+7 of k-step ks).  Products whose output is indexed by
// (feature, token) are issued as (M = feature, N = token) so that the 4 accumulator rows of a lane
// are again features of ITS token: with the feature permutation
//       pi(t, m) = 32*(t/2) + 8*(m/4) + 4*(t%2) + m%4        (t = 16x16 output tile, m = tile row)
// accumulator element (t, e) of lane (r, c) is feature 32*(t/2) + 8c + 4*(t%2) + e, i.e. element
// 4t+e of the row layout.  Contractions over tokens read their A operand from natural
// [token][feature] LDS tiles with the transposing LDS read of gfx950.
#pragma once

#include "gla_common.hpp"

namespace gla {

struct f32x8 {
    float v[8];
};

template <typename T> struct FragTypes;
template <> struct FragTypes<__bf16> {
    typedef bf16x8 d8;  // 8 features of one token (one k-step of a feature contraction)
    typedef bf16x4 t4;  // 4 tokens of one feature (one k-step of a token contraction)
};
template <> struct FragTypes<float> {
    typedef f32x8 d8;
    typedef f32x4 t4;
};

// ---- MFMA wrappers ----------------------------------------------------------------------------
// mma_d: 16x16 += A(16 x 32) B(32 x 16), contraction over 32 features.
__device__ __forceinline__ f32x4 mma_d(bf16x8 a, bf16x8 b, f32x4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma_d(const f32x8 &a, const f32x8 &b, f32x4 c)
{
#pragma unroll
    for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[e], b.v[e], c, 0, 0, 0);
    return c;
}
// mma_t: 16x16 += A(16 x 16) B(16 x 16), contraction over 16 tokens.
__device__ __forceinline__ f32x4 mma_t(bf16x4 a, bf16x4 b, f32x4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4v, a),
                                                     __builtin_bit_cast(short4v, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma_t(f32x4 a, f32x4 b, f32x4 c)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], c, 0, 0, 0);
    return c;
}

// ---- packing ----------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ typename FragTypes<T>::d8 pack8(const float *x);
template <> __device__ __forceinline__ bf16x8 pack8<__bf16>(const float *x)
{
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (__bf16)x[e];
    return r;
}
template <> __device__ __forceinline__ f32x8 pack8<float>(const float *x)
{
    f32x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r.v[e] = x[e];
    return r;
}
template <typename T> __device__ __forceinline__ typename FragTypes<T>::t4 pack4(f32x4 x);
template <> __device__ __forceinline__ bf16x4 pack4<__bf16>(f32x4 x)
{
    bf16x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = (__bf16)x[e];
    return r;
}
template <> __device__ __forceinline__ f32x4 pack4<float>(f32x4 x) { return x; }

__device__ __forceinline__ void unpack8(bf16x8 f, float *x)
{
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)f[e];
}
__device__ __forceinline__ void unpack8(const f32x8 &f, float *x)
{
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = f.v[e];
}

// ---- memory access ----------------------------------------------------------------------------
// 8 consecutive features from global or LDS memory (16-byte aligned).
__device__ __forceinline__ bf16x8 ld8(const __bf16 *p) { return *reinterpret_cast<const bf16x8 *>(p); }
__device__ __forceinline__ f32x8 ld8(const float *p)
{
    f32x4 a = reinterpret_cast<const f32x4 *>(p)[0], b = reinterpret_cast<const f32x4 *>(p)[1];
    f32x8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r.v[e] = a[e]; r.v[4 + e] = b[e]; }
    return r;
}
__device__ __forceinline__ void st8(__bf16 *p, bf16x8 v) { *reinterpret_cast<bf16x8 *>(p) = v; }
__device__ __forceinline__ void st8(float *p, const f32x8 &v)
{
    f32x4 a = {v.v[0], v.v[1], v.v[2], v.v[3]}, b = {v.v[4], v.v[5], v.v[6], v.v[7]};
    reinterpret_cast<f32x4 *>(p)[0] = a;
    reinterpret_cast<f32x4 *>(p)[1] = b;
}

// The same for global data that is touched exactly once (streamed state rows, outputs): non-temporal
// accesses, which leave the L2 lines of the inputs that are read again alone.
__device__ __forceinline__ bf16x8 ld8_once(const __bf16 *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const bf16x8 *>(p));
}
__device__ __forceinline__ f32x8 ld8_once(const float *p)
{
    f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p)),
          b = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p) + 1);
    f32x8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r.v[e] = a[e]; r.v[4 + e] = b[e]; }
    return r;
}
__device__ __forceinline__ void st8_once(__bf16 *p, bf16x8 v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<bf16x8 *>(p));
}
__device__ __forceinline__ void st8_once(float *p, const f32x8 &v)
{
    f32x4 a = {v.v[0], v.v[1], v.v[2], v.v[3]}, b = {v.v[4], v.v[5], v.v[6], v.v[7]};
    __builtin_nontemporal_store(a, reinterpret_cast<f32x4 *>(p));
    __builtin_nontemporal_store(b, reinterpret_cast<f32x4 *>(p) + 1);
}

// Head dimension 16 runs on the kernels for 32 features.  A row of the caller's arrays then has DM = 16 features
// where the kernel works on D = 32: the lanes that would hold features 16..31 (c >= 2) read the first features
// of their row instead (an address inside the array) and replace what they read by zeros, which is what the
// padded features are (a zero log-gate, key, query and value leave every result of the real features alone);
// their results are not stored.  The chunk states, the per-chunk products and the decays are the library's own
// buffers and are kept at D x D.
template <int D, int DM> struct RowMap {
    static_assert(DM == D || (D == 32 && DM == 16), "padding is built for head dimension 16 only");
    static constexpr bool kPadded = DM < D;
    static __device__ __forceinline__ bool live(int c) { return !kPadded || 8 * c < DM; }
    static __device__ __forceinline__ int col(int c) { return live(c) ? 8 * c : 0; }
};
// 8 features of a row: `row_ks` points at feature 32*ks of the lane's row, c is the lane's feature group.
template <int D, int DM, typename P> __device__ __forceinline__ auto ld8_row(const P *row_ks, int c)
{
    auto x = ld8(row_ks + RowMap<D, DM>::col(c));
    if constexpr (DM < D) {
        if (!RowMap<D, DM>::live(c)) x = decltype(x){};
    }
    return x;
}
template <int D, int DM, typename P> __device__ __forceinline__ auto ld8_row_once(const P *row_ks, int c)
{
    auto x = ld8_once(row_ks + RowMap<D, DM>::col(c));
    if constexpr (DM < D) {
        if (!RowMap<D, DM>::live(c)) x = decltype(x){};
    }
    return x;
}
template <int D, int DM, typename P, typename V> __device__ __forceinline__ void st8_row_once(P *row_ks, int c, const V &v)
{
    if (RowMap<D, DM>::live(c)) st8_once(row_ks + 8 * c, v);
}

// The chunk states of 16-bit data lie in memory as 32 x 32 tiles, [dk/32][dv/32][32][32] (2 KB each), so that both a
// slab of 32 key features (all value features) and a slab of 32 value features (all key features) are made of
// whole tiles: the scan writes ONE array per direction and every consumer reads 2 KB pieces whichever way it
// contracts.  fp32 states stay row-major (and are written in both orientations).
template <typename T, int D> __device__ __forceinline__ int state_offset(int dk, int dv)
{
    if constexpr (sizeof(T) == 2) return (((dk >> 5) * (D / 32) + (dv >> 5)) << 10) + ((dk & 31) << 5) + (dv & 31);
    else return dk * D + dv;
}

// LDS tiles are row-major [rows][D] with a 16-byte pad per row.
template <typename T, int D> struct TileGeom {
    static constexpr int kStride = D + 16 / (int)sizeof(T);
};

// Transposing LDS read.  For a natural [row][col] tile and a 4-row band starting at row k0, lane
// i = lane % 16 of every 16-lane group receives tile[k0 + 0..3][colbase(i / 4) + i % 4].  On bf16 this is
// one ds_read_b64_tr_b16: lane j of the group fetches 4 consecutive columns (8 bytes) of row
// k0 + j/4 starting at ITS colbase(j % 4), and the hardware hands lane i column i%4 of the lanes i/4,
// i/4+4, i/4+8, i/4+12.  With the feature permutation pi, colbase(m) = 32*(t/2) + 8*m + 4*(t%2).
//
// All addresses are split into a per-lane part, computed once per kernel (TrLane), and a compile-time
// part that folds into the instruction's immediate offset, so a kernel keeps a handful of address
// registers instead of one per (tile, sub-block, feature tile).
template <typename T> struct TrLane {
    int nat;   // natural reads:   row r,            features 8c..8c+7          -> r*S + 8c
    int k4;    // transposed read: rows 4c + ...,    feature block (r>>2 | r&3)
    int k8;    // transposed read: rows 8c + ...  (contractions over 32 rows, two reads 4 rows apart)
    int own;   // natural read of the row pi(., m = r): (8*(r>>2) + (r&3))*S + 8c
};
template <typename T> __device__ __forceinline__ TrLane<T> make_tr_lane(int stride)
{
    const int lane = threadIdx.x & 63, r = lane & 15, c = lane >> 4;
    TrLane<T> t;
    t.nat = r * stride + 8 * c;
    t.own = (8 * (r >> 2) + (r & 3)) * stride + 8 * c;
    if constexpr (sizeof(T) == 2) {
        t.k4 = (4 * c + (r >> 2)) * stride + 8 * (r & 3);
        t.k8 = (8 * c + (r >> 2)) * stride + 8 * (r & 3);
    } else {
        t.k4 = 4 * c * stride + 8 * (r >> 2) + (r & 3);
        t.k8 = 8 * c * stride + 8 * (r >> 2) + (r & 3);
    }
    return t;
}
__device__ __forceinline__ bf16x4 lds_tr4(const __bf16 *p, int stride)
{
    (void)stride;
    typedef __attribute__((ext_vector_type(4))) short v4s;
    v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)p);
    return __builtin_bit_cast(bf16x4, v);
}
__device__ __forceinline__ f32x4 lds_tr4(const float *p, int stride)
{
    f32x4 r = {p[0], p[stride], p[2 * stride], p[3 * stride]};
    return r;
}

// Plain mapping: tile t covers features 16t .. 16t+15, lane i gets feature 16t + i.
template <typename T> __device__ __forceinline__ int plain_tr_lane(int stride)
{
    const int lane = threadIdx.x & 63, r = lane & 15, c = lane >> 4;
    if constexpr (sizeof(T) == 2) return (4 * c + (r >> 2)) * stride + 4 * (r & 3);
    else return 4 * c * stride + r;
}

// ---- gate prefix/suffix hierarchy inside a 16-token sub-block -------------------------------------
// After `levels` steps (h = 1, 2, 4, ...) p holds the inclusive prefix sum of the gate over the lane's
// aligned group of size 2h and s the exclusive suffix sum over it; lanes r of a DPP row are the 16
// tokens.  One step: every lane learns the total of the sibling group and adds it to p (if it sits in
// the upper sibling) or to s (lower sibling).
template <int H> __device__ __forceinline__ float sibling_total(float tot)
{
    if constexpr (H == 1) return dpp_f32<kDppQuadXor1>(tot);
    else if constexpr (H == 2) return dpp_f32<kDppQuadXor2>(tot);
    else if constexpr (H == 4) return dpp_f32<kDppRowHalfMirror>(tot);
    else return dpp_f32<kDppRowMirror>(tot);
}

template <int H, int NV> __device__ __forceinline__ void hier_step(float (&p)[NV], float (&s)[NV], bool upper)
{
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        float other = sibling_total<H>(p[i] + s[i]);
        p[i] += upper ? other : 0.f;
        s[i] += upper ? 0.f : other;
    }
}

// Inclusive prefix / suffix sum over the 16 token rows of the wave (lanes of one DPP row): lane r
// receives the sum over rows <= r (>= r).  Lanes shifted in from outside the row read 0.
__device__ __forceinline__ float prefix_sum_rows(float x)
{
    x += dpp_f32<0x111>(x);   // row_shr:1
    x += dpp_f32<0x112>(x);
    x += dpp_f32<0x114>(x);
    x += dpp_f32<0x118>(x);
    return x;
}
__device__ __forceinline__ float suffix_sum_rows(float x)
{
    x += dpp_f32<0x101>(x);   // row_shl:1
    x += dpp_f32<0x102>(x);
    x += dpp_f32<0x104>(x);
    x += dpp_f32<0x108>(x);
    return x;
}

// A sub-block whose gate sums stay below this many powers of two (in either direction, for every
// feature and every row) is handled with ONE anchor instead of the dyadic recursion: its rescaled
// operands are at most 2^48 and their products cannot overflow.  log_sigmoid gates reach this only
// when they average below -2 nats per token over 16 tokens; harder gates (up to outright resets) take
// the recursion, whose factors never exceed 1.
constexpr float kOneAnchorSpan = 48.f;

// Wave-uniform: true if x < limit on every lane (a NaN counts as not below).
__device__ __forceinline__ bool wave_all_below(float x, float limit)
{
    return __ballot(!(x < limit)) == 0ull;
}

// Hides a pointer's provenance from the optimiser: loads through the result are not merged with
// earlier loads of (or forwarded from earlier stores to) the same address, so a value can be dropped
// from registers and fetched again (an L2 hit) where it is needed next.
template <typename P> __device__ __forceinline__ P *refetch(P *ptr)
{
    asm volatile("" : "+v"(ptr));
    return ptr;
}

// Sum over the 4 lanes (c = 0..3) that hold the same token row.
__device__ __forceinline__ float reduce_over_cgroups(float x)
{
    x += shfl_xor_f32(x, 16);
    x += shfl_xor_f32(x, 32);
    return x;
}

}  // namespace gla
