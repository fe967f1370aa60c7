// Internal interface of the bf16 matrix products of the lm_head training step (lmhead_gemm.hip).
#pragma once

#include "mrl_internal.h"

namespace mrl {

// out[n][m] (+)= sum_k a[m][k] * b[n][k], bf16 operands, fp32 accumulation.  An operand is either
// k-contiguous ([m, k] / [n, k] with leading dimension lda / ldb, read up to the next multiple of 64
// in k) or k-major ([k, m] / [k, n], rows of k beyond `k` count as zero, m / n a multiple of 8).
// out is [n, m] with leading dimension ldo: bf16 (overwritten) or, with accumulate_f32, fp32 (added
// to).  Built combinations: (a, b) k-contiguous -> bf16; a k-major, b k-contiguous -> bf16; both
// k-major -> fp32 accumulate.  `fn` names the caller in errors.
int gemm_bf16(const char* fn, const void* a, int64_t lda, int64_t m, bool a_kmajor, const void* b, int64_t ldb, int64_t n,
              bool b_kmajor, int64_t k, void* out, int64_t ldo, bool accumulate_f32, hipStream_t stream);

}  // namespace mrl
