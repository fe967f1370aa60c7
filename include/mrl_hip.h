/*
 * mrl_hip.h - C ABI of libmrl_hip.so: MI355X (gfx950) kernels for the actor log-probability
 * and GRPO/DAPO policy-loss path of MindSpeed-RL.
 *
 * The reference has no native code and no FFI for this path: every function below replaces a
 * chain of torch ops in the reference's Python (cited per entry point, paths relative to the
 * reference tree).  Host code binds these symbols with ctypes (mindspeed_rl_amd/_lib.py holds
 * the argument types of every entry point).
 *
 * Conventions, all entry points:
 *   - plain C: raw DEVICE pointers, explicit int64 sizes, dtype enums, the HIP stream as void*
 *     (NULL = the null stream); no ownership is taken, nothing is allocated or freed;
 *   - kernels are enqueued asynchronously on `stream`, no hidden synchronisation;
 *   - return 0 on success, a negative mrl_status otherwise (nothing is launched then);
 *     mrl_last_error() gives the message of the calling thread's last failure;
 *   - tensors are dense row-major; "nullable" pointers may be NULL.
 */
#ifndef MRL_HIP_H_
#define MRL_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MRL_VERSION 300

enum mrl_status {
    MRL_OK = 0,
    MRL_ERR_INVALID_ARG = -1,  /* NULL where a pointer is required, negative size, bad enum */
    MRL_ERR_UNSUPPORTED = -2,  /* dtype / size combination the kernels do not cover        */
    MRL_ERR_MISALIGNED = -3,   /* pointer not aligned to its element size                  */
    MRL_ERR_LAUNCH = -4        /* the HIP runtime rejected the launch                      */
};

enum mrl_dtype {
    MRL_F32 = 0,
    MRL_BF16 = 1,
    MRL_F16 = 2,
    MRL_I32 = 3,
    MRL_I64 = 4,
    MRL_U8 = 5, /* also torch.bool */
    MRL_F64 = 6
};

enum mrl_kl_penalty {
    MRL_KL_NONE = 0,      /* DAPO: kl_loss == 0 (dapo_actor_loss_func.py:150) */
    MRL_KL_KL = 1,        /* logp - ref                                        */
    MRL_KL_ABS = 2,       /* |logp - ref|                                      */
    MRL_KL_MSE = 3,       /* 0.5 (logp - ref)^2                                */
    MRL_KL_LOW_VAR = 4    /* k3 with clamps +-20 / +-10 (utils/compute.py:120-126) */
};

/* Library version (MRL_VERSION of the build). */
int mrl_version(void);

/* Message of the calling thread's last failed call ("" if none). */
const char* mrl_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Vocabulary sweep, forward.  Replaces compute_log_probs (mindspeed_rl/utils/compute.py:29-51,
 * i.e. Megatron's vocab_parallel_cross_entropy at tp=1), _VocabParallelEntropy.forward
 * (utils/compute.py:56-73) and the caller's `output.div_(temperature)`
 * (models/base/base_training_engine.py:237) in ONE read of the logits.
 *
 *   z' = logits * inv_temperature
 *   lse[t]     = logsumexp_j z'[t,j]
 *   logp[t]    = z'[t, label_t] - lse[t]      (label outside [0,vocab): max_j z'[t,j] - lse[t],
 *                                               which is what Megatron's target mask yields)
 *   entropy[t] = lse[t] - sum_j softmax(z')_j z'[t,j]
 *
 * logits: [n_rows, vocab] of logits_dtype (F32, BF16, F16), row t at logits + t*row_stride
 * elements; it is only read.  labels: [n_rows] I32 or I64.  row_active (nullable): [n_rows]
 * bytes, rows with 0 are skipped and get logp = entropy = lse = 0.  entropy and lse are
 * nullable; logp is required.  Accumulation is fp32.
 */
int mrl_vocab_logprob_fwd(const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                          int64_t row_stride, const void* labels, int labels_dtype,
                          const uint8_t* row_active, float inv_temperature, float* logp,
                          float* entropy, float* lse, void* stream);

/* ------------------------------------------------------------------------------------------
 * Vocabulary sweep, backward.  Replaces Megatron's cross-entropy backward,
 * _VocabParallelEntropy.backward (utils/compute.py:76-85) and autograd of the temperature
 * division with one read of the logits and one write of dlogits:
 *
 *   p = exp(z' - lse)
 *   dlogits[t,j] = inv_temperature * ( g_logp[t] * (onehot(label_t)_j - p_j)
 *                                      - g_entropy[t] * p_j * (z'_j - (lse[t] - entropy[t])) )
 *
 * lse (and entropy, if g_entropy is given) are the forward's outputs.  g_logp and g_entropy are
 * [n_rows] fp32, each nullable (NULL = zero).  Rows whose incoming gradients are both zero are
 * written as zeros without reading the logits.  dlogits has dlogits_dtype (F32, BF16, F16) and
 * its own row stride; it may alias logits exactly (same pointer, dtype and stride) for an
 * in-place backward.
 */
int mrl_vocab_logprob_bwd(const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                          int64_t row_stride, const void* labels, int labels_dtype,
                          float inv_temperature, const float* lse, const float* entropy,
                          const float* g_logp, const float* g_entropy, void* dlogits,
                          int dlogits_dtype, int64_t dlogits_row_stride, void* stream);

/* ------------------------------------------------------------------------------------------
 * Remove-padding index maps.  Replace the per-sequence Python loops of preprocess_packed_seqs
 * (mindspeed_rl/utils/remove_padding.py:38-87).  All integer results are bit-exact.
 *
 * mrl_pack_index_build: seqlens[i] = int32 sum of attention_mask[i,:] (mask dtype I64, I32, U8
 * or F32; if attention_mask is NULL, seqlens is an input), pad_i = (align - len_i % align) %
 * align, cu_seqlens_padded[0] = 0, cu_seqlens_padded[i+1] = int32 running sum of len_i + pad_i.
 * total (nullable) receives cu_seqlens_padded[batch] as int64.  One workgroup; batch <= 2^20.
 */
int mrl_pack_index_build(const void* attention_mask, int mask_dtype, int64_t batch, int64_t width,
                         int64_t align, int32_t* seqlens, int32_t* cu_seqlens_padded,
                         int64_t* total, void* stream);

/* mrl_pack_rows: dst[t] = src[i, t - cu[i]] for cu[i] <= t < cu[i] + seqlens[i], else 0;
 * position_ids[t] = t - cu[i] (runs through the alignment padding, remove_padding.py:66-72).
 * src/dst (and the optional second pair src2/dst2, e.g. ids and labels in one launch) hold
 * elem_bytes = 4 or 8 byte integers; src is [batch, width], dst is [total].  position_ids
 * (nullable) is int32 [total].  Positions t >= cu[batch] are written as 0. */
int mrl_pack_rows(const void* src, void* dst, const void* src2, void* dst2, int elem_bytes,
                  int64_t batch, int64_t width, const int32_t* seqlens,
                  const int32_t* cu_seqlens_padded, int64_t total, int32_t* position_ids,
                  void* stream);

/* mrl_unpad_gather: postprocess_packed_seqs (remove_padding.py:116-136).  packed is
 * [total, inner] of elem_bytes (2, 4 or 8) bytes, out is [batch, seq_len, inner], fully
 * written (zeros where nothing is copied).  Per sequence: start = cu[i], n = seqlens[i]; if
 * prompt_length is given (I32 or I64, [batch]) and P_i - 1 < n then n -= P_i, start += P_i - 1;
 * out[i, :n] = packed[start : start + n].  Where the reference raises on n > seq_len this
 * kernel copies the first seq_len entries. */
int mrl_unpad_gather(const void* packed, int elem_bytes, int64_t total, int64_t inner,
                     const int32_t* seqlens, const int32_t* cu_seqlens_padded,
                     const void* prompt_length, int prompt_dtype, int64_t batch, int64_t seq_len,
                     void* out, void* stream);

/* mrl_pad_scatter: adjoint of mrl_unpad_gather for fp32 gradients with inner == 1:
 * g_packed[t] = g_out[i, t - start_i] if t lies in sequence i's copied window, else 0.
 * Written as a gather over t (binary search in cu), so it is deterministic. */
int mrl_pad_scatter(const float* g_out, int64_t batch, int64_t seq_len, const int32_t* seqlens,
                    const int32_t* cu_seqlens_padded, const void* prompt_length, int prompt_dtype,
                    int64_t total, float* g_packed, void* stream);

/* mrl_window_gather: truncate_prompt_and_pad / truncate_middle_and_pad
 * (mindspeed_rl/utils/pad_process.py:74-141).  src is [batch, width, inner] of elem_bytes, window
 * is [batch, 2] (I32 or I64) = (start, end), clamped to [0, width]; out is [batch, out_len,
 * inner], filled with pad_bits (the element's bit pattern, low elem_bytes bytes) and then
 * out[i, :end-start] = src[i, start:end].  Copies at most out_len entries per row. */
int mrl_window_gather(const void* src, int elem_bytes, int64_t batch, int64_t width, int64_t inner,
                      const void* window, int window_dtype, int64_t out_len, uint64_t pad_bits,
                      void* out, void* stream);

/* mrl_window_scatter: adjoint of mrl_window_gather for fp32, inner == 1: g_src is [batch, width],
 * g_src[i, start+j] = g_out[i, j] for j < min(end-start, out_len), zero elsewhere. */
int mrl_window_scatter(const float* g_out, int64_t batch, int64_t width, const void* window,
                       int window_dtype, int64_t out_len, float* g_src, void* stream);

/* mrl_generate_mask: generate_mask (mindspeed_rl/utils/utils.py:57-67): out[i, j] =
 * (j < lengths[i]) as int64, [batch, width]; lengths is I32 or I64.  Negative lengths give an
 * all-zero row, lengths above width an all-one row. */
int mrl_generate_mask(const void* lengths, int lengths_dtype, int64_t batch, int64_t width,
                      int64_t* out, void* stream);

/* ------------------------------------------------------------------------------------------
 * Ragged <-> padded experience columns: the wire format either side of the path.  Replace the
 * per-row Python loops of unpack_pad_experience (mindspeed_rl/trainer/utils/transfer_dock.py:
 * 1092-1198) and truncate_rows (mindspeed_rl/utils/pad_process.py:144-166).  Bit-exact copies.
 *
 * mrl_ragged_layout: cu[0] = 0, cu[i+1] = cu[i] + len_i (int32 [batch+1]); info[0] = cu[batch],
 * info[1] = max_i len_i rounded up to `multiple` (int64 [2]).  len_i = lengths[i] (I32 / I64), < 0
 * counts as 0.  With width > 0, len_i follows truncate_rows for rows of that width: clamped to
 * width; with left_pad a zero length keeps the whole row (python's x[-0:]); and if `rows`
 * ([batch, width] integers, elem_bytes 4 or 8) is given, 0 where lengths[i] == 0 and
 * rows[i, 0] == -1.  eff_len (nullable int32 [batch]) receives the len_i.  One workgroup;
 * batch <= 2^20. */
int mrl_ragged_layout(const void* lengths, int lengths_dtype, int64_t batch, int64_t multiple,
                      const void* rows, int elem_bytes, int64_t width, int left_pad, int32_t* eff_len,
                      int32_t* cu, int64_t* info, void* stream);

/* mrl_first_match: the search inside remove_padding_and_split_to_list
 * (mindspeed_rl/utils/pad_process.py:44-62): first[i] = index of the first entry of integer row i
 * (elem_bytes 4 or 8) that equals `value`, plus `extra` (0 or 1), clamped to width; width if the
 * row has no such entry.  int32 [batch]. */
int mrl_first_match(const void* rows, int elem_bytes, int64_t batch, int64_t width, int64_t value, int extra,
                    int32_t* first, void* stream);

/* out[i, d, j] = flat[d * flat_stride + cu[i] + j] for j < cu[i+1] - cu[i], else pad_bits; out is
 * [batch, first_dim, width] (first_dim = 1 for ordinary columns, 3 for mrope position ids). */
int mrl_ragged_to_padded(const void* flat, int elem_bytes, int64_t first_dim, int64_t flat_stride,
                         const int32_t* cu, int64_t batch, int64_t width, uint64_t pad_bits, void* out,
                         void* stream);

/* flat[cu[i] + j] = padded[i, j] (left_pad = 0) or padded[i, width - len_i + j] (left_pad = 1). */
int mrl_padded_to_ragged(const void* padded, int elem_bytes, int64_t batch, int64_t width,
                         const int32_t* cu, int left_pad, int64_t total, void* flat, void* stream);

/* ------------------------------------------------------------------------------------------
 * Group-relative advantages.  Replaces compute_group_norm_advantage_return
 * (mindspeed_rl/trainer/utils/compute_utils.py:152-191): rows i*group .. (i+1)*group-1 form one
 * group; in fp64, score = (r - mean) / (unbiased_std + 1e-6); cast to fp32; advantages[i, j] =
 * score_i * mask[i, j].  rewards: [batch] F32 or F64; mask: [batch, width] F32, I64, I32 or U8;
 * advantages / returns: [batch, width] fp32 (returns nullable, a second copy as in the
 * reference).  batch must be a multiple of group.  group == 1 yields NaN, as torch.std does. */
int mrl_group_advantage(const void* rewards, int rewards_dtype, int64_t batch, int64_t group,
                        const void* mask, int mask_dtype, int64_t width, float* advantages,
                        float* returns, void* stream);

/* mrl_group_standardize: get_last_reward (mindspeed_rl/trainer/utils/compute_utils.py:277-291):
 * out[i] = (r_i - mean_g) / (unbiased_std_g + eps) over the group of `group` consecutive rewards
 * that holds i; fp64 internally, fp32 result.  n must be a multiple of group. */
int mrl_group_standardize(const void* rewards, int rewards_dtype, int64_t n, int64_t group, double eps,
                          float* out, void* stream);

/* DAPO dynamic-sampling predicate (mindspeed_rl/workers/dynamic_sampling.py:81-86): keep[r] = 1
 * for every row of a group iff numpy.std(group) > 0 or the group has one member, else 0.  The
 * arithmetic follows numpy's (pairwise summation, mean, squared deviations, in the metric's own
 * dtype F32 or F64) so that the comparison with 0 is bit-exact.  n need not be a multiple of
 * group: the last group is short, as python slicing makes it. */
int mrl_group_keep_mask(const void* metric, int metric_dtype, int64_t n, int64_t group,
                        uint8_t* keep, void* stream);

/* ------------------------------------------------------------------------------------------
 * Policy loss, forward.  Replaces _compute_grpo_policy_loss
 * (mindspeed_rl/models/loss/grpo_actor_loss_func.py:127-144), _compute_dapo_policy_loss
 * (dapo_actor_loss_func.py:129-152), compute_kl_penalty (utils/compute.py:100-133), the
 * masked_mean calls (utils/torch_functional.py:38-59) and the dynamic-batch rescale
 * (grpo_actor_loss_func.py:74-79) with one launch plus a tiny finalize launch.
 *
 * All per-token tensors are [batch, width] fp32, dense.  old_log_prob NULL means ratio == 1;
 * ref_log_prob is required unless kl_penalty == MRL_KL_NONE; entropy NULL means zeros.  The mask
 * is either `mask` ([batch, width] of mask_dtype F32, I64, I32, U8) or, if mask is NULL,
 * j < response_length[i] (I32 or I64).  ratio is clamped to [clip_lo, clip_hi] (pass
 * float(1 - eps_low), float(1 + eps_high)).  seq_mean = 0: token mean with the reference's 1e-8
 * in the denominator; seq_mean = 1: DAPO's mean over sequences of per-sequence token means
 * (no epsilon: an all-masked row gives NaN, and the clip fraction is 0, as in the reference).
 *
 * out[8] (fp32): [0] loss_scale * pg_loss (the tensor the caller back-propagates),
 *   [1] pg_loss, [2] pg_clipfrac, [3] ppo_kl, [4] kl_loss, [5] entropy mean, [6] sum(mask),
 *   [7] number of rows.
 * row_sums: workspace of batch*8 floats, kept for the backward.
 */
int mrl_policy_loss_fwd(const float* log_prob, const float* old_log_prob,
                        const float* ref_log_prob, const float* advantages, const float* entropy,
                        const void* mask, int mask_dtype, const void* response_length,
                        int length_dtype, int64_t batch, int64_t width, float clip_lo,
                        float clip_hi, int kl_penalty, float kl_coef, float entropy_coeff,
                        int seq_mean, float loss_scale, float* row_sums, float* out,
                        void* stream);

/* Policy loss, backward: what autograd derives from the torch expression of the reference,
 * including torch.max's half/half split on ties and clamp's closed-interval pass-through.
 * upstream (nullable) is a DEVICE scalar multiplying everything (Megatron's loss scaling).
 * g_log_prob [batch, width] is required; g_entropy is nullable (needed if entropy_coeff != 0). */
int mrl_policy_loss_bwd(const float* log_prob, const float* old_log_prob,
                        const float* ref_log_prob, const float* advantages, const void* mask,
                        int mask_dtype, const void* response_length, int length_dtype,
                        int64_t batch, int64_t width, float clip_lo, float clip_hi,
                        int kl_penalty, float kl_coef, float entropy_coeff, int seq_mean,
                        float loss_scale, const float* row_sums, const float* out,
                        const float* upstream, float* g_log_prob, float* g_entropy, void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused forward + backward ("eager gradient").  The loss gradient of a token depends only on
 * that token's own log-prob, its old/ref log-probs, advantage and mask, and on denominators
 * that are known from the mask before the sweep - so dlogits can be produced in the SAME pass
 * that computes the log-prob: one read of the logits and one write of dlogits for the whole
 * path (2 bytes-moved units instead of 3), with each row held in registers by one workgroup.
 * Replaces, in one chain: compute_log_probs + vocab_parallel_entropy (utils/compute.py:29-97),
 * postprocess_packed_seqs / truncate_prompt_and_pad (the response window), the policy loss
 * (grpo_actor_loss_func.py:127-144, dapo_actor_loss_func.py:129-152) and all their backwards.
 *
 * Call order: mrl_fused_loss_prepare -> mrl_fused_logprob_loss -> mrl_fused_loss_reduce, and
 * mrl_scale_rows_note when autograd later delivers an upstream gradient: four launches for the
 * forward and backward of the whole path when the mask is given by the response lengths.
 */

/* Largest vocabulary the row-in-registers kernels hold for a logits dtype (0 = bad dtype): one
 * workgroup keeps up to 19 456 16-byte vectors of a row in registers, and rows of up to twice that
 * (311 296 bf16 / fp16 or 155 648 fp32 logits) are cut in two halves held by two workgroups at the
 * same time, which exchange the statistics of their halves through the workspace. */
int64_t mrl_fused_max_vocab(int logits_dtype);

/* Bytes of workspace mrl_fused_logprob_loss wants for this shape (16-byte aligned device memory):
 * 16 for rows that one workgroup holds (the row counter of the persistent workgroups), 16 + 32 *
 * n_rows for wider rows (plus one 16-byte record per half row); 0 if the fused sweep does not take
 * the shape at all. */
int64_t mrl_fused_workspace_bytes(int logits_dtype, int64_t n_rows, int64_t vocab);

/* Step 1.  Maps the [batch, width] loss operands onto logits rows.
 *   layout 0, packed [n_rows, V] logits: sequence i owns the rows postprocess_packed_seqs copies
 *     (start = cu[i], n = seqlens[i]; with prompt_length and P_i - 1 < n: n -= P_i, start += P_i - 1);
 *   layout 1, padded [batch, padded_seq_len, V] logits: rows [P_i - 1, P_i + R_i - 1) clamped to
 *     [0, padded_seq_len] of block i (base_loss_func.py:47-53, pad_process.py:120-123).
 * Row start_i + j holds token (i, j), j < min(n, width).  The mask is `mask` ([batch, width] F32,
 * I64, I32, U8) or j < response_length[i].  old_log_prob / ref_log_prob may be NULL.
 * Outputs: row_start int64 [batch], row_count int32 [batch], seq_mask_sum float [batch] (sum of
 * each mask row), row_ops float [n_rows * 8] = {old, ref, adv, mask, w_pg, 1/(N+1e-8), 0, 0} per
 * logits row, mask = 0 for rows outside every window; N = sum of the whole mask; w_pg is
 * 1/(N+1e-8) (seq_mean 0) or 1/(batch * seq_mask_sum[i]) (seq_mean 1).  prompt_length >= 1.
 * The same launch prepares the sweep that follows on `stream`: sweep_workspace (nullable, a multiple
 * of 8 bytes) is zeroed, which is what mrl_fused_logprob_loss asks of a workspace handed to it as
 * `workspace_cleared`, and scale_out (nullable, two floats, 8-byte aligned) receives
 * {scale_host * *scale_in, 0}: the scale the sweep is to write into its gradients (scale_in, a
 * nullable DEVICE scalar, NULL = 1: what mrl_scale_rows_note learned at the previous backward) next
 * to the zeroed counter that mrl_scale_rows_note keeps there.  With the mask given by the response
 * lengths (mask NULL) and at most 2048 sequences all of this is ONE launch. */
int mrl_fused_loss_prepare(int layout, int64_t batch, int64_t width, int64_t n_rows,
                           const int32_t* seqlens, const int32_t* cu_seqlens_padded,
                           int64_t padded_seq_len, const void* prompt_length, int prompt_dtype,
                           const void* response_length, int response_dtype,
                           const float* old_log_prob, const float* ref_log_prob,
                           const float* advantages, const void* mask, int mask_dtype, int seq_mean,
                           int64_t* row_start, int32_t* row_count, float* seq_mask_sum,
                           float* row_ops, void* sweep_workspace, int64_t sweep_workspace_bytes,
                           const float* scale_in, float scale_host, float* scale_out, void* stream);

/* Step 2.  The sweep.  Per row with a non-zero mask: logp, entropy (if `entropy` is given) as in
 * mrl_vocab_logprob_fwd; the token's loss terms as in mrl_policy_loss_fwd; then
 *   dlogits = grad_scale * (*grad_scale_dev) * d(loss)/d(logits)
 * written in the logits dtype.  grad_scale carries what the host knows (loss_scale, and the upstream
 * gradient if the caller was told it); grad_scale_dev (nullable, NULL = 1) is a DEVICE scalar read by
 * the kernel, typically the upstream gradient that mrl_grad_scale_note recorded at the previous
 * backward - Megatron's 1/num_microbatches and loss scale reach the loss function only through
 * autograd (models/base/base_training_engine.py:238-270), so the host never knows them in time.  Rows with mask 0 get zero dlogits and are not read.  dlogits may
 * alias logits exactly (in-place).  row_terms float [n_rows * 8] receives {pg, clipped, old-lp,
 * kl, entropy, 1} * mask per row for step 3.  logp / entropy: nullable [n_rows] outputs.
 * has_old = 0 means old_log_prob = log_prob.detach() (ratio 1).  workspace:
 * mrl_fused_workspace_bytes(dtype, n_rows, vocab) bytes of device memory owned by the caller: the
 * counter from which the persistent workgroups take their next row and, for rows wider than one
 * workgroup holds, the records through which the two halves of a row exchange their statistics.
 * Both must be zero when the sweep starts: with workspace_cleared != 0 the caller vouches for that
 * (mrl_fused_loss_prepare clears it in passing), else this call clears it on `stream` first.  A
 * workspace must not be shared by sweeps that can be in flight at the same time, and a captured
 * graph keeps using the address it was captured with.  NULL is allowed for rows that one workgroup
 * holds: every row then gets a workgroup of its own, which costs large batches about a quarter more
 * time.  Needs 16-byte aligned rows, vocab % (16/elem) == 0 and
 * vocab <= mrl_fused_max_vocab(dtype); else MRL_ERR_UNSUPPORTED (use the split fwd/bwd entry points
 * then).  The wait of a workgroup for the other half of its row is bounded
 * (mrl_set_wide_spin_limit): past the bound it computes that half's statistics itself from memory,
 * with the same result to the last bit; in place that is safe because a workgroup overwrites its
 * half only after its record has reached memory, and a reader that finds the record after all
 * discards what it read. */
int mrl_fused_logprob_loss(const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                           int64_t row_stride, const void* labels, int labels_dtype,
                           float inv_temperature, const float* row_ops, int has_old,
                           float clip_lo, float clip_hi, int kl_penalty, float kl_coef,
                           float entropy_coeff, float grad_scale, const float* grad_scale_dev,
                           void* dlogits, int64_t dlogits_row_stride, float* logp, float* entropy,
                           float* row_terms, void* workspace, int64_t workspace_bytes,
                           int workspace_cleared, void* stream);

/* Polls a workgroup spends waiting for the record of the other half of a wide row before it reads
 * that half itself (default 2^18; 0 = never wait, which exercises the fallback; negative restores
 * the default).  Process-wide, read at every launch; returns the previous value.  No counterpart
 * in the reference. */
int64_t mrl_set_wide_spin_limit(int64_t polls);

/* Step 3.  Sums row_terms per sequence (tokens with a non-zero mask but no logits row enter with
 * log_prob = entropy = 0, as in the split path) and finalizes out[8] / row_sums exactly like
 * mrl_policy_loss_fwd.  done_counter (nullable): four zeroed bytes of device memory (word 1 of a
 * cleared sweep workspace serves); with it the whole step is one launch - the workgroup that
 * finishes last combines the sequences - and the counter is zero again afterwards.  loss_out
 * (nullable): receives out[0] once more, for a caller that wants the loss in storage of its own. */
int mrl_fused_loss_reduce(const float* row_terms, const int64_t* row_start,
                          const int32_t* row_count, int64_t batch, int64_t width,
                          const float* old_log_prob, const float* ref_log_prob,
                          const float* advantages, const void* mask, int mask_dtype,
                          const void* response_length, int response_dtype, float clip_lo,
                          float clip_hi, int kl_penalty, float kl_coef, float entropy_coeff,
                          int seq_mean, float loss_scale, float* row_sums, float* out,
                          uint32_t* done_counter, float* loss_out, void* stream);

/* x[r, :] *= (*upstream / *applied) in place, unless that ratio is exactly 1 (then the kernel
 * exits without touching memory).  upstream and applied are DEVICE scalars: the gradient autograd
 * delivers and the scale x already carries.  Lets the eager gradient honour whatever scalar arrives
 * (Megatron's 1/num_microbatches and loss scale) without a host synchronisation.  Neither scalar is
 * written; follow the last mrl_scale_rows of a backward with mrl_grad_scale_note. */
int mrl_scale_rows(void* x, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                   const float* upstream, const float* applied, void* stream);

/* Book-keeping after the mrl_scale_rows calls of one backward (no counterpart in the reference,
 * where autograd multiplies by the upstream gradient as part of every backward op): *applied =
 * *upstream, so a second backward over the same buffers rescales by the ratio of the two upstream
 * values only; *learned (nullable) = *upstream if that is finite and non-zero - the scalar the next
 * mrl_fused_logprob_loss reads through grad_scale_dev; *rescales (nullable) is incremented when
 * upstream differed from applied, i.e. when the rescale moved memory.  All DEVICE pointers. */
int mrl_grad_scale_note(const float* upstream, float* applied, float* learned, uint32_t* rescales,
                        void* stream);

/* mrl_scale_rows followed by mrl_grad_scale_note for ONE buffer in ONE launch.  applied: two
 * floats, 8-byte aligned: {the scale x carries, a counter that is zero between calls} - the pair
 * mrl_fused_loss_prepare writes to scale_out.  An upstream gradient of 0, Inf or NaN is applied like
 * any other (autograd's product) and recorded as the scale x now carries; it cannot be undone, so a
 * later backward over the same buffer yields NaN rather than a wrong finite value. */
int mrl_scale_rows_note(void* x, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                        const float* upstream, float* applied, float* learned, uint32_t* rescales,
                        void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused lm_head + log-prob, forward (no counterpart in the reference, which always materialises
 * the [T, V] logits in GPTModel.output_layer and then runs compute_log_probs on them,
 * utils/compute.py:29-51): logits[t, v] = sum_k hidden[t, k] * weight[v, k] are produced tile by
 * tile on the bf16 matrix cores with fp32 accumulation and consumed by an online log-sum-exp,
 * so they never reach memory.  The statistics use the fp32 logits (the reference rounds the
 * materialised logits to bf16 first).
 *
 * hidden: [n_tokens, hidden_dim] bf16, weight: [vocab, hidden_dim] bf16 (the layout of a
 * torch.nn.Linear weight), both dense and 16-byte aligned; hidden_dim % 64 == 0.  labels
 * [n_tokens] I32 / I64.  Outputs as mrl_vocab_logprob_fwd (entropy, lse nullable).  workspace:
 * mrl_lmhead_workspace_bytes(n_tokens, vocab) bytes of device memory, 16-byte aligned, holding
 * the per-vocabulary-group partial statistics (MRL_LMHEAD_GROUPS x n_tokens x 16 bytes).
 */
#define MRL_LMHEAD_GROUPS 8
int64_t mrl_lmhead_workspace_bytes(int64_t n_tokens, int64_t vocab);
int mrl_lmhead_logprob_fwd(const void* hidden, const void* weight, int64_t n_tokens, int64_t vocab,
                           int64_t hidden_dim, const void* labels, int labels_dtype,
                           float inv_temperature, float* logp, float* entropy, float* lse,
                           void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Training step from the hidden states (configs "fused lm_head"): the three matrix products around
 * the fused sweep, hand-written for the bf16 matrix cores (same tile loop as the forward above).
 * The reference has no counterpart: its model materialises all [T, V] logits
 * (models/base/base_training_engine.py:221-258) and autograd runs the two backward products of the
 * output layer.  Here the caller walks the tokens in chunks and only a chunk of logits exists:
 *
 *   mrl_lmhead_logits            logits[t, v] = sum_h hidden[t, h] * weight[v, h]      (bf16 out)
 *   mrl_fused_logprob_loss       turns the chunk into dlogits in place (see above)
 *   mrl_lmhead_logprob_bwd       dHidden[t, h] = sum_v dlogits[t, v] * weight[v, h]     (bf16 out)
 *                                dWeight[v, h] += sum_t dlogits[t, v] * hidden[t, h]    (fp32, added)
 *
 * hidden [n_tokens, hidden_dim] and weight [vocab, hidden_dim] are dense bf16, hidden_dim % 64 == 0,
 * vocab % 8 == 0; logits / dlogits rows are logits_row_stride / dlogits_row_stride apart.  The
 * backward reads hidden, weight and dlogits as they lie (no transposed copies, no workspace); it
 * wants dlogits_row_stride a multiple of 64 (and at least vocab) with zeros in the padding columns,
 * since it reads whole steps of 64 columns; n_tokens is arbitrary.  dWeight is accumulated chunk
 * after chunk in stream order, without atomics, so the result does not depend on timing.  Nothing
 * here allocates. */
int mrl_lmhead_logits(const void* hidden, const void* weight, int64_t n_tokens, int64_t vocab,
                      int64_t hidden_dim, void* logits, int64_t logits_row_stride, void* stream);
int mrl_lmhead_logprob_bwd(const void* hidden, const void* weight, const void* dlogits,
                           int64_t dlogits_row_stride, int64_t n_tokens, int64_t vocab,
                           int64_t hidden_dim, void* d_hidden, float* d_weight, void* stream);

/* mrl_lmhead_logprob_fwd for callers that cannot allocate device memory or pass a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in
 * the reference.  Same arguments, kernels and results as mrl_lmhead_logprob_fwd, but the partial
 * statistics live in a static device array of the library (8 MiB per GPU that runs it, looked up
 * once per device with hipGetSymbolAddress and held until the process ends), so at most
 * mrl_lmhead_static_max_tokens() = 65536 tokens per call: more is rejected with
 * MRL_ERR_UNSUPPORTED (slice the tokens).  Calls nothing that allocates or frees.  Every call on a
 * GPU shares that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
 * race and give wrong results - serialise them.  The array needs no clearing between calls: every
 * entry a call reads was written by that call. */
int64_t mrl_lmhead_static_max_tokens(void);
int mrl_lmhead_logprob_fwd_static(const void* hidden, const void* weight, int64_t n_tokens,
                                  int64_t vocab, int64_t hidden_dim, const void* labels,
                                  int labels_dtype, float inv_temperature, float* logp,
                                  float* entropy, float* lse, void* stream);

/* ------------------------------------------------------------------------------------------
 * PPO's value side (the "next" row after the actor path): rewards with the KL penalty, GAE,
 * whitening and the critic's clipped value loss.  All tensors [batch, width] fp32, contiguous.
 *
 * mrl_kl_token_rewards: the arithmetic inside apply_kl_penalty
 * (mindspeed_rl/trainer/utils/compute_utils.py:80-97): mask = (j < response_length[i]);
 * kld = compute_kl_penalty(old_log_prob, ref_log_prob, kl_penalty) * mask; rewards[i, j] =
 * (j == response_length[i] - 1 ? scores[i] : 0) - beta * kld (a zero length puts the score on the
 * last column, like python's index -1); row_kl[i] = sum_j kld / (sum_j mask + 1e-8).  The caller
 * averages row_kl for kl_ctrl.update(). */
int mrl_kl_token_rewards(const float* old_log_prob, const float* ref_log_prob,
                         const void* response_length, int length_dtype, const float* scores,
                         int64_t batch, int64_t width, int kl_penalty, float beta, float* rewards,
                         float* row_kl, void* stream);

/* mrl_gae_scan: the reverse scan of compute_gae_advantage_return (compute_utils.py:134-145), before
 * its whitening: delta_t = rewards[t] + gamma * values[t+1] - values[t] (values[width] = 0),
 * lastgaelam = delta_t + gamma_lam * lastgaelam, advantages[t] = lastgaelam, returns =
 * advantages + values.  gamma_lam is the product gamma * lam formed in DOUBLE and rounded to fp32
 * once (python evaluates `gamma * lam` first, torch then rounds the scalar); gamma is rounded on its
 * own.  fp32 with the reference's operation order and roundings: bit-identical to the torch loop.
 * Outputs must not alias the inputs. */
int mrl_gae_scan(const float* rewards, const float* values, int64_t batch, int64_t width, float gamma,
                 float gamma_lam, float* advantages, float* returns, void* stream);

/* mrl_masked_whiten: masked_whiten / masked_var / masked_mean (mindspeed_rl/utils/
 * torch_functional.py:46-106) over n entries: mean = sum(x*mask)/(sum(mask)+1e-8), var the same of
 * (x-mean)^2 times sum(mask)/(sum(mask)-1) unless sum(mask) == 1, out = (x-mean)*rsqrt(var+1e-8)
 * (+ mean unless shift_mean).  mask: F32, I64, I32 or U8.  info (3 doubles on the device) receives
 * sum(mask), mean, var; the caller raises the reference's ValueError when sum(mask) == 0.
 * out may alias x. */
int mrl_masked_whiten(const float* x, const void* mask, int mask_dtype, int64_t n, int shift_mean,
                      float* out, double* info, void* stream);

/* mrl_value_loss_fwd / _bwd: CriticLossFunc._compute_value_loss
 * (mindspeed_rl/models/loss/critic_loss_func.py:82-111) and its backward with respect to vpreds:
 * vf_loss = 0.5 * masked_mean(max((vp-ret)^2, (clamp(vp, v-c, v+c)-ret)^2)), vf_clipfrac =
 * masked_mean(second > first).  The mask is `mask` or, if NULL, (j < response_length[i]).
 * out (4 floats): loss_scale * vf_loss, vf_loss, vf_clipfrac, sum(mask).  The backward follows
 * torch: the larger operand of max gets the gradient (halved on ties), clamp passes it inside the
 * closed interval; g_vpreds = upstream[0] * d(out[0])/d(vpreds). */
int mrl_value_loss_fwd(const float* vpreds, const float* returns, const float* values, const void* mask,
                       int mask_dtype, const void* response_length, int length_dtype, int64_t batch,
                       int64_t width, float cliprange_value, float loss_scale, float* out, void* stream);
int mrl_value_loss_bwd(const float* vpreds, const float* returns, const float* values, const void* mask,
                       int mask_dtype, const void* response_length, int length_dtype, int64_t batch,
                       int64_t width, float cliprange_value, float loss_scale, const float* out,
                       const float* upstream, float* g_vpreds, void* stream);

/* ------------------------------------------------------------------------------------------
 * Plain device-to-device copy kernel of n_bytes (multiple of 16, 16-byte aligned pointers);
 * used to calibrate the rocprofv3 FETCH_SIZE / WRITE_SIZE counters and as the measured
 * bandwidth ceiling next to the 8 TB/s vendor peak.  No counterpart in the reference. */
int mrl_copy_bytes(const void* src, void* dst, int64_t n_bytes, void* stream);

/* Bandwidth probes with the sweeps' access pattern (one 1024-thread workgroup per row of row_bytes
 * bytes, a multiple of 16, at most 311 296): mode 0 reads n_rows rows from src (dst: 4 writable
 * bytes, never written in practice), mode 1 writes n_rows rows to dst, mode 2 copies src to dst with
 * the whole row in registers (all loads of a workgroup before its stores).  Modes 3, 4, 5 are the
 * same read / write / copy of n_rows * row_bytes bytes as one vector per thread in small
 * workgroups that retire at once: the requests in flight cover one compact stretch of memory,
 * which is the pattern the HBM system serves best.  They measure the practical ceilings that the
 * roofline fractions are also quoted against.  No counterpart in the reference. */
int mrl_bandwidth_probe(int mode, const void* src, void* dst, int64_t n_rows, int64_t row_bytes,
                        void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MRL_HIP_H_ */
