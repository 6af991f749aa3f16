// Head dimension 256 as four problems of head dimension 128: the small kernels around the two passes (gla_split.hip).
#pragma once

#include "gla_common.hpp"

namespace gla {

// rows = number of 256-element rows; dtype / hdt = gla_dtype of the elements
// dst[row][j] = src[row][j ^ 128]
int launch_swap_halves(hipStream_t st, int dtype, int64_t rows, void *dst, const void *src);
// dst[row][j] += src[row][j], or src[row][j ^ 128] when swapped != 0 (summed in fp32, rounded once)
int launch_add_rows(hipStream_t st, int dtype, int64_t rows, void *dst, const void *src, int swapped);
// dst[row][j] = a[row][j] + b[row][j], or b[row][j ^ 128] when swapped != 0, rounded to dst's type (dtype) once
int launch_sum_rows(hipStream_t st, int dtype, int64_t rows, void *dst, const float *a, const float *b, int swapped);
// full [BH][256][256] <-> same [BH][2][128][128] (block a = rows and columns of half a) and cross (block a = rows
// of half a, columns of the other half); gather != 0: full -> blocks, else blocks -> full
int launch_hidden_blocks(hipStream_t st, int hdt, int64_t BH, void *full, void *same, void *cross, int gather);

}  // namespace gla
