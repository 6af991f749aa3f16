// Launchers of the chunk_gla kernels, one explicit instantiation per (element type, chunk, head dim).
#pragma once

#include "gla_common.hpp"
#include "gla_split.hpp"

namespace gla {

// (T, C, D) combinations that are compiled.  C = tokens per chunk handled by one workgroup
// (C/16 waves), D = head dimension (DK == DV, gla.py:499).  Head dimension 256 has no kernels of its own: it runs
// as four problems of head dimension 128 (gla_split.hip).  D = 32 is the
// smallest head dimension whose feature contractions fill one k-step of the 16x16x32 matrix instruction; head
// dimension 16 (the smallest the reference's score kernel takes, gla.py:975) runs on those kernels with its
// rows padded by zeros on the way in.
// DM is the head dimension of the caller's arrays: D, or 16 on the kernels built for D = 32 (see RowMap).
#define GLA_FOR_EACH_CHUNK_CONFIG(M) \
    M(__bf16, 128, 128, 128)         \
    M(__bf16, 64, 128, 128)          \
    M(__bf16, 32, 128, 128)          \
    M(__bf16, 128, 64, 64)           \
    M(__bf16, 64, 64, 64)            \
    M(__bf16, 32, 64, 64)            \
    M(__bf16, 128, 32, 32)           \
    M(__bf16, 64, 32, 32)            \
    M(__bf16, 32, 32, 32)            \
    M(__bf16, 128, 32, 16)           \
    M(__bf16, 64, 32, 16)            \
    M(__bf16, 32, 32, 16)            \
    M(float, 64, 64, 64)             \
    M(float, 32, 64, 64)             \
    M(float, 64, 32, 32)             \
    M(float, 32, 32, 32)             \
    M(float, 64, 32, 16)             \
    M(float, 32, 32, 16)             \
    M(float, 32, 128, 128)

template <typename T, int C, int D, int DM>
// prodT: the per-chunk products in the library's own layout and type (gla_chunk_state.hip), pexp: their exponents
int launch_chunk_outer(hipStream_t st, int mode, int B, int T_len, int H, const float *g, const void *x,
                       const void *y, void *prodT, float *decay, unsigned char *pexp);

template <typename T, int D, int DM>
// hdt = gla_dtype of hin / hout (hidden_init and hidden_final, or their cotangents)
int launch_chunk_scan(hipStream_t st, int BH, int N, int reverse, int hdt, const void *hin, const void *prodT,
                      const float *decay, const unsigned char *pexp, void *statesT, void *statesN, void *hout,
                      int tail, int tiled);

// WIDE (built for bf16 at D = 128 only): `out`, or `dv`, `dk`, `dq`, are float arrays, for the two passes that make
// up head dimension 256
template <typename T, int C, int D, int DM, bool WIDE = false>
// states: the chunk-start states the kernel contracts over dk: for 16-bit data the tiled [dk][dv] array with `slots`
// states per (b,h) (the residual, or its stand-in in the workspace), for fp32 data the [dv][dk] array of the workspace
int launch_chunk_out(hipStream_t st, int B, int T_len, int H, const float *g, const void *v, const void *k,
                     const void *q, const void *states, int slots, void *out);

template <typename T, int C, int D, int DM, bool WIDE = false>
int launch_chunk_grad(hipStream_t st, int B, int T_len, int H, const float *g, const void *v, const void *k,
                      const void *q, const void *dout, const void *statesN, const void *dstatesT,
                      const void *dstatesN, float *dg, void *dv, void *dk, void *dq);

}  // namespace gla
