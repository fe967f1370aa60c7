// Internal interface of the bf16 matrix products of the lm_head training step (lmhead_gemm.hip).
#pragma once

#include "mrl_internal.h"

namespace mrl {

// out[n][m] (+)= sum_k a[m][k] * b[n][k]: a is [m, k] with leading dimension lda, b is [n, k] with
// ldb, both bf16 with k contiguous, k % 64 == 0, m % 4 == 0; out is [n, m] with leading dimension
// ldo, bf16 (overwritten) or, with accumulate_f32, fp32 (added to).  `fn` names the caller in errors.
int gemm_nt_bf16(const char* fn, const void* a, int64_t lda, int64_t m, const void* b, int64_t ldb, int64_t n, int64_t k,
                 void* out, int64_t ldo, bool accumulate_f32, hipStream_t stream);

// dst[c][r] = src[r][c] (16-bit elements) for r < rows, c < cols; dst is [dst_rows, ld_dst] and is
// written completely, zeros outside the transposed block.
int transpose_bf16(const char* fn, const void* src, int64_t ld_src, int64_t rows, int64_t cols, void* dst, int64_t ld_dst,
                   int64_t dst_rows, hipStream_t stream);

}  // namespace mrl
