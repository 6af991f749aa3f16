// Launchers of the matrix-core recurrent_gla kernels (bf16 inputs, head dimension 64 or 128).  `hdt` is the
// gla_dtype of the state arrays (h0, hT, dhT, dh0).
#pragma once

#include "gla_common.hpp"

namespace gla {

// TO = element type of `out` (__bf16, or float for the recurrent_gla_naive flavour).
template <typename TO>
int launch_recurrent_stream_fwd(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt,
                                const void *h0, const float *g, const void *v, const void *k, const void *q,
                                void *hT, void *out);

// The forward without its outputs: hidden_final alone (what a segment contributes to the state that leaves it).
// h0 may be null: the state starts from zeros.  g_shift = +1 or -1: every step takes the gate of the next (previous)
// row of the array instead of its own (the recurrence of the state's cotangent, where the decay between two steps
// belongs to the later one); the first step of a sequence, whose gate scales the initial state, may get any row's.
// gate_sums (may be null; not with g_shift): [B][H][D] floats, the sum of every sequence's gates.
int launch_recurrent_stream_state(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, const void *h0,
                                 const float *g, const void *v, const void *k, const void *q, void *hT,
                                 int g_shift = 0, float *gate_sums = nullptr);

// Sweep 1 of the backward: dq, and q*dq in fp32 into `qdq` (the last step's carries sum_v dhT * (final state)
// on top).  dout_f32 != 0: `dout` is float (the recurrent_gla_naive flavour), else bf16.  wide != 0 (head dimension
// 128 only): `dq` is a float array, for the two passes that make up head dimension 256.
int launch_recurrent_stream_dq(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                               const void *h0, const float *g, const void *v, const void *k, const void *q,
                               const void *dhT, const void *dout, void *dq, float *qdq, int wide = 0);

// The same sweep with two waves per sub-block (head dimension 64).
int launch_recurrent_stream_dq2(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                                const void *h0, const float *g, const void *v, const void *k, const void *q,
                                const void *dhT, const void *dout, void *dq, float *qdq);

// Sweep 2: dk, dv, dh0 and dlog_fgate (`dg` holds sweep 1's q*dq on entry).  wide != 0 (head dimension 128 only):
// `dv` and `dk` are float arrays.
int launch_recurrent_stream_rev(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                                const float *g, const void *v, const void *k, const void *q, const void *dhT,
                                const void *dout, void *dh0, float *dg, void *dv, void *dk, int wide = 0);

// The same sweep with two waves per sub-block (head dimension 64).
int launch_recurrent_stream_rev2(hipStream_t st, int B, int T_len, int H, int D, int reverse, int hdt, int dout_f32,
                                 const float *g, const void *v, const void *k, const void *q, const void *dhT,
                                 const void *dout, void *dh0, float *dg, void *dv, void *dk);

}  // namespace gla
