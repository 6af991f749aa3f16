// Shared device/host helpers for the gfx950 GLA kernels: element types, MFMA and DPP wrappers,
// status codes.  Everything here is written for CDNA4 (64-wide wavefronts) only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <type_traits>

#include "../../include/gla_hip.h"

namespace gla {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short short4v;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr float kLog2e = 1.4426950408889634f;

// ---- element traits ---------------------------------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Elem<__bf16> {
    static __device__ __forceinline__ float load(const __bf16 *p) { return (float)*p; }
    static __device__ __forceinline__ void store(__bf16 *p, float v) { *p = (__bf16)v; }
};

// Loads N consecutive elements (N*sizeof(T) a multiple of 4 and the address aligned to it, up to
// 16 bytes per access) and widens them to float.
template <typename T, int N>
__device__ __forceinline__ void load_vec(const T *p, float (&dst)[N])
{
    if constexpr (sizeof(T) == 4) {
        if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) {
                f32x4 t = *reinterpret_cast<const f32x4 *>(p + i);
                dst[i] = t[0]; dst[i + 1] = t[1]; dst[i + 2] = t[2]; dst[i + 3] = t[3];
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 2) {
                f32x2 t = *reinterpret_cast<const f32x2 *>(p + i);
                dst[i] = t[0]; dst[i + 1] = t[1];
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) dst[i] = p[i];
        }
    } else {
        if constexpr (N % 8 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 8) {
                bf16x8 t = *reinterpret_cast<const bf16x8 *>(p + i);
#pragma unroll
                for (int j = 0; j < 8; ++j) dst[i + j] = (float)t[j];
            }
        } else if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) {
                bf16x4 t = *reinterpret_cast<const bf16x4 *>(p + i);
#pragma unroll
                for (int j = 0; j < 4; ++j) dst[i + j] = (float)t[j];
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 2) {
                bf16x2 t = *reinterpret_cast<const bf16x2 *>(p + i);
                dst[i] = (float)t[0]; dst[i + 1] = (float)t[1];
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) dst[i] = (float)p[i];
        }
    }
}

template <typename T, int N>
__device__ __forceinline__ void store_vec(T *p, const float (&src)[N])
{
    if constexpr (sizeof(T) == 4) {
        if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) {
                f32x4 t = {src[i], src[i + 1], src[i + 2], src[i + 3]};
                *reinterpret_cast<f32x4 *>(p + i) = t;
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 2) {
                f32x2 t = {src[i], src[i + 1]};
                *reinterpret_cast<f32x2 *>(p + i) = t;
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) p[i] = src[i];
        }
    } else {
        if constexpr (N % 8 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 8) {
                bf16x8 t;
#pragma unroll
                for (int j = 0; j < 8; ++j) t[j] = (__bf16)src[i + j];
                *reinterpret_cast<bf16x8 *>(p + i) = t;
            }
        } else if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) {
                bf16x4 t;
#pragma unroll
                for (int j = 0; j < 4; ++j) t[j] = (__bf16)src[i + j];
                *reinterpret_cast<bf16x4 *>(p + i) = t;
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 2) {
                bf16x2 t;
                t[0] = (__bf16)src[i]; t[1] = (__bf16)src[i + 1];
                *reinterpret_cast<bf16x2 *>(p + i) = t;
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) p[i] = (__bf16)src[i];
        }
    }
}

// The state arrays (hidden_init, hidden_final and their cotangents) carry an element type of their own, `hdt`
// (a gla_dtype, uniform over the launch): the reference loads the initial state in its own dtype into an fp32
// state and stores the final one back in it, whatever the type of value/key/query (gla.py:44-46, 89-97).
template <int N>
__device__ __forceinline__ void load_hidden(const void *base, int hdt, int64_t idx, float (&dst)[N])
{
    if (hdt == GLA_F32) load_vec<float, N>(static_cast<const float *>(base) + idx, dst);
    else load_vec<__bf16, N>(static_cast<const __bf16 *>(base) + idx, dst);
}
template <int N>
__device__ __forceinline__ void store_hidden(void *base, int hdt, int64_t idx, const float (&src)[N])
{
    if (hdt == GLA_F32) store_vec<float, N>(static_cast<float *>(base) + idx, src);
    else store_vec<__bf16, N>(static_cast<__bf16 *>(base) + idx, src);
}

__device__ __forceinline__ float load_hidden1(const void *base, int hdt, int64_t idx)
{
    return hdt == GLA_F32 ? static_cast<const float *>(base)[idx] : (float)static_cast<const __bf16 *>(base)[idx];
}
__device__ __forceinline__ void store_hidden1(void *base, int hdt, int64_t idx, float x)
{
    if (hdt == GLA_F32) static_cast<float *>(base)[idx] = x;
    else static_cast<__bf16 *>(base)[idx] = (__bf16)x;
}

// ---- cross-lane ---------------------------------------------------------------------------------
// DPP controls (GFX9/CDNA encoding).
constexpr int kDppQuadXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppRowMirror = 0x140;      // lane r -> 15-r inside a 16-lane row
constexpr int kDppRowHalfMirror = 0x141;  // lane r -> 7-r inside an 8-lane half row

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float shfl_xor_f32(float v, int mask)
{
    return __shfl_xor(v, mask, 64);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Workgroup barrier for data exchanged through LDS only: waits for the wave's LDS operations, not for its
// global loads and stores (`__syncthreads()` waits for those too, i.e. for prefetches that are not needed yet
// and for streamed stores nobody in the workgroup reads).
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- host side ------------------------------------------------------------------------------
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }

// Dynamic LDS above 64 KB has to be granted per kernel before the launch (gfx950 has 160 KB per CU).  The grant
// sticks to the kernel on the device it was made on, so it is made once per (kernel, device): every launcher
// keeps one LdsGrant per kernel it launches, a bit per device index.  This and the per-device address of the
// static scratch array are the only state the library keeps between calls.
struct LdsGrant {
    std::atomic<uint64_t> done{0};
};
inline int allow_lds(LdsGrant &grant, const void *kernel, size_t bytes)
{
    if (bytes <= 65536) return 0;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const uint64_t bit = dev < 64 ? (1ull << dev) : 0;
    if (bit && (grant.done.load(std::memory_order_acquire) & bit)) return 0;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return (int)e;
    grant.done.fetch_or(bit, std::memory_order_release);
    return 0;
}

inline int launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace gla
