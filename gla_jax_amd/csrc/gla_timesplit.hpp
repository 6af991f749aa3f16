// recurrent_gla on few sequences: the small kernels that let a sequence run as S segments side by side
// (gla_timesplit.hip; the entry points that use them are in gla_recurrent.hip).
#pragma once

#include "gla_common.hpp"

namespace gla {

// sums[b][p][h][d] = sum of g[b][p*L + t][h][d] over the L rows of segment p.  g: [B][S*L][H][D] floats.
int launch_segment_gate_sums(hipStream_t st, int64_t B, int64_t S, int64_t L, int64_t H, int D, const float *g,
                             float *sums);
// dst[b][t] = src[b][t + dir] (dir = +1 or -1) for rows that exist, zeros for the one row per batch entry that has no
// such neighbour.  Rows are [H*D] floats, T rows per batch entry.
int launch_shift_rows(hipStream_t st, int64_t B, int64_t T, int64_t row_len, const float *src, float *dst, int dir);
// The recurrence over segments, elementwise over a [D][D] state per (b, h).  Every segment may come as F consecutive
// pieces of Lf steps (loc, loc2, sums indexed [b][piece], S*F pieces per batch entry):
//     x <- exp(sums[b][piece][h][dk]) * x + exp(edge) * (loc + loc2)[b][piece][h][dk][dv],
// pieces ascending, or descending from the last, with entering[b][p] = x before segment p's first piece (fp32) and
// `final` = x after the last piece (type hdt; may be null).  x starts as init[b][h] (type hdt).
// edge = g[b][piece*Lf + edge_row][h][dk] when g is given, else 0.  loc2 may be null.
int launch_segment_scan(hipStream_t st, int64_t B, int64_t S, int64_t F, int64_t Lf, int64_t H, int D, int hdt,
                        const void *init, const float *loc, const float *loc2, const float *sums, const float *g,
                        int edge_row, int descending, float *entering, void *final);
// hi[i] = bf16(x[i]), lo[i] = bf16(x[i] - hi[i]) for n floats (n a multiple of 8): a float array as two bf16 arrays
// whose sum keeps 16 bits of mantissa
int launch_head_remainder(hipStream_t st, int64_t n, const float *x, void *hi, void *lo);
// n bytes of zeros (a multiple of 16, the address aligned to 16)
int launch_zero_fill(hipStream_t st, void *dst, size_t n);

}  // namespace gla
