// chunk_gla and recurrent_gla at head dimension 256 as four problems of head dimension 128.
//
// The recurrence is a sum over key features and independent over value features: with the key features split
// into halves a and the value features into halves b,
//     out[:, b] = sum_a GLA(q_a, k_a, g_a, v_b),      hidden[a, b] = the state of GLA(q_a, k_a, g_a, v_b),
// and every gradient is a sum of the same four problems' gradients (dq_a, dk_a, dg_a over b; dv_b over a).
// A [B,T,H,256] array read as [B,T,2H,128] has the halves of head h as heads 2h and 2h+1, so the two problems
// with a == b are ONE run of the 128-feature kernels on the arrays as they lie, and the two with a != b are a
// second run on q, k, g as they lie and the value-side arrays with the halves of every row exchanged.  This file
// holds the small kernels around those runs: exchanging halves, adding the two runs' results (for bf16 data both runs
// leave out, dq, dk and dv in fp32 and the sum is rounded once, as one kernel over all 256 features would round it),
// and cutting the [256,256] states into their four [128,128] blocks and back.
#include "gla_split.hpp"

namespace gla {

namespace {

constexpr int kRow = 256;        // elements of a row (one head of one token)
constexpr int kHalf = kRow / 2;

template <typename T> __device__ __forceinline__ void load8(const T *p, float (&x)[8]) { load_vec<T, 8>(p, x); }
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&x)[8]) { store_vec<T, 8>(p, x); }

// dst[row][j] = src[row][j ^ 128]: eight elements per thread
template <typename T>
__global__ __launch_bounds__(256) void swap_halves_kernel(T *__restrict__ dst, const T *__restrict__ src, int64_t n8)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const int64_t e = i * 8;
    float x[8];
    load8<T>(src + (e ^ kHalf), x);
    store8<T>(dst + e, x);
}

// dst[row][j] += src[row][j] (swapped == 0) or src[row][j ^ 128]; the sum is formed in fp32 and rounded once
template <typename T>
__global__ __launch_bounds__(256) void add_rows_kernel(T *__restrict__ dst, const T *__restrict__ src, int64_t n8,
                                                       int swapped)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const int64_t e = i * 8;
    float x[8], y[8];
    load8<T>(dst + e, x);
    load8<T>(src + (swapped ? e ^ kHalf : e), y);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] += y[j];
    store8<T>(dst + e, x);
}

// dst[row][j] = a[row][j] + b[row][j] (swapped == 0) or b[row][j ^ 128], rounded to dst's type once
template <typename T>
__global__ __launch_bounds__(256) void sum_rows_kernel(T *__restrict__ dst, const float *__restrict__ a,
                                                       const float *__restrict__ b, int64_t n8, int swapped)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const int64_t e = i * 8;
    float x[8], y[8];
    load8<float>(a + e, x);
    load8<float>(b + (swapped ? e ^ kHalf : e), y);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] += y[j];
    store8<T>(dst + e, x);
}

// The four [128,128] blocks of every [256,256] state.  full: [BH][256][256]; same: [BH][2][128][128], block a =
// rows and columns of half a; cross: [BH][2][128][128], block a = rows of half a, columns of the other half.
// gather != 0 copies full -> blocks, else blocks -> full.
template <typename T>
__global__ __launch_bounds__(256) void hidden_blocks_kernel(T *__restrict__ full, T *__restrict__ same,
                                                            T *__restrict__ cross, int64_t n8, int gather)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const int64_t e = i * 8;                           // element of `full`
    const int64_t bh = e / (kRow * kRow);
    const int row = (int)(e / kRow % kRow), col = (int)(e % kRow);
    const int a = row / kHalf, b = col / kHalf;
    T *blk = (a == b ? same : cross) + ((bh * 2 + a) * kHalf + row % kHalf) * kHalf + col % kHalf;
    float x[8];
    if (gather) {
        load8<T>(full + e, x);
        store8<T>(blk, x);
    } else {
        load8<T>(blk, x);
        store8<T>(full + e, x);
    }
}

inline dim3 grid_for(int64_t n8) { return dim3((unsigned)((n8 + 255) / 256)); }

}  // namespace

int launch_swap_halves(hipStream_t st, int dtype, int64_t rows, void *dst, const void *src)
{
    const int64_t n8 = rows * kRow / 8;
    if (n8 > 0x7fffffffLL * 256) return GLA_ERR_SHAPE;
    if (dtype == GLA_BF16)
        hipLaunchKernelGGL(swap_halves_kernel<__bf16>, grid_for(n8), dim3(256), 0, st, (__bf16 *)dst,
                           (const __bf16 *)src, n8);
    else
        hipLaunchKernelGGL(swap_halves_kernel<float>, grid_for(n8), dim3(256), 0, st, (float *)dst, (const float *)src,
                           n8);
    return launch_status();
}

int launch_add_rows(hipStream_t st, int dtype, int64_t rows, void *dst, const void *src, int swapped)
{
    const int64_t n8 = rows * kRow / 8;
    if (n8 > 0x7fffffffLL * 256) return GLA_ERR_SHAPE;
    if (dtype == GLA_BF16)
        hipLaunchKernelGGL(add_rows_kernel<__bf16>, grid_for(n8), dim3(256), 0, st, (__bf16 *)dst, (const __bf16 *)src,
                           n8, swapped);
    else
        hipLaunchKernelGGL(add_rows_kernel<float>, grid_for(n8), dim3(256), 0, st, (float *)dst, (const float *)src, n8,
                           swapped);
    return launch_status();
}

int launch_sum_rows(hipStream_t st, int dtype, int64_t rows, void *dst, const float *a, const float *b, int swapped)
{
    const int64_t n8 = rows * kRow / 8;
    if (n8 > 0x7fffffffLL * 256) return GLA_ERR_SHAPE;
    if (dtype == GLA_BF16)
        hipLaunchKernelGGL(sum_rows_kernel<__bf16>, grid_for(n8), dim3(256), 0, st, (__bf16 *)dst, a, b, n8, swapped);
    else
        hipLaunchKernelGGL(sum_rows_kernel<float>, grid_for(n8), dim3(256), 0, st, (float *)dst, a, b, n8, swapped);
    return launch_status();
}

int launch_hidden_blocks(hipStream_t st, int hdt, int64_t BH, void *full, void *same, void *cross, int gather)
{
    const int64_t n8 = BH * kRow * kRow / 8;
    if (hdt == GLA_BF16)
        hipLaunchKernelGGL(hidden_blocks_kernel<__bf16>, grid_for(n8), dim3(256), 0, st, (__bf16 *)full, (__bf16 *)same,
                           (__bf16 *)cross, n8, gather);
    else
        hipLaunchKernelGGL(hidden_blocks_kernel<float>, grid_for(n8), dim3(256), 0, st, (float *)full, (float *)same,
                           (float *)cross, n8, gather);
    return launch_status();
}

}  // namespace gla
