// Internal interface of the row-in-registers sweeps (row_sweep.hip): argument bundles and the
// per-row operand layout shared with the loss-side prepare / reduce kernels.
#pragma once

#include "mrl_internal.h"

// row_ops[r*8 + ...]: the loss operands of logits row r
#define MRL_ROW_OPS 8
#define MRL_OP_OLD 0     // old_log_prob of the token
#define MRL_OP_REF 1     // ref_log_prob of the token
#define MRL_OP_ADV 2     // advantage of the token
#define MRL_OP_MASK 3    // mask weight; 0 for rows that are not response tokens
#define MRL_OP_WPG 4     // weight of the surrogate term: 1/(N+1e-8) or 1/(B * M_i)
#define MRL_OP_INVTOK 5  // 1/(N+1e-8)

namespace mrl {

struct FusedArgs {
    const void* logits; int dtype; int64_t n_rows, vocab, row_stride;
    const void* labels; int labels_dtype; float inv_t;
    const float* row_ops; int has_old;
    float clip_lo, clip_hi; int kl_penalty; float kl_coef, entropy_coeff, grad_scale;
    const float* grad_scale_dev;    // nullable device scalar that multiplies grad_scale
    void* workspace;                // nullable for narrow rows: row counter (+ half-row records)
    bool workspace_cleared;         // the caller has zeroed it on this stream
    bool wide;                      // rows cut in two halves held by two workgroups
    int64_t half_elems;             // entries of the first half
    void* dlogits; int64_t d_stride;
    float* logp; float* entropy; float* row_terms;
    bool with_entropy;
    hipStream_t stream;
};

struct BwdArgs {
    const void* logits; int dtype; int64_t n_rows, vocab, row_stride;
    const void* labels; int labels_dtype; float inv_t;
    const float* lse; const float* entropy; const float* g_logp; const float* g_entropy;
    void* dlogits; int64_t d_stride;
    hipStream_t stream;
};

// Backward of log-prob / entropy for given per-row upstream gradients, dlogits in the dtype of the
// logits, as a stream of 16-byte vectors.  Call only if bwd_chunks_supported().
int launch_bwd_chunks(const BwdArgs& a);
bool bwd_chunks_supported(int dtype, int64_t vocab, const void* in, int64_t in_stride, const void* out,
                          int64_t out_stride, int64_t n_rows);

// True if rows of this dtype / vocab / alignment fit the row-in-registers kernels.
bool row_sweep_supported(int dtype, int64_t vocab, const void* in, int64_t in_stride, const void* out,
                         int64_t out_stride, int64_t n_rows);

}  // namespace mrl
