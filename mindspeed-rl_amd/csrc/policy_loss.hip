// GRPO / DAPO clipped-ratio policy loss for gfx950: forward (loss + the five statistics) and
// backward (dL/dlog_prob, dL/dentropy).
//
// Forward: one workgroup per sequence row reduces six masked sums over the row (fp32 per
// thread, fp64 across threads), a single-workgroup finalize kernel combines the rows in a fixed
// order - deterministic, no float atomics - and writes the eight output scalars.  Backward is
// one element-wise launch that re-derives each token's local gradient from the inputs and the
// saved denominators.
#include "mrl_internal.h"
#include "policy_terms.h"
#include "row_sweep.h"

namespace {

using namespace mrl_loss;

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;

__device__ __forceinline__ double block_sum(double v, double* lds) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();                      // lds may still be read from the previous call
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    double r = 0.0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) r += lds[w];
    return r;
}

__device__ __forceinline__ int64_t load_i64(const void* p, int dtype, int64_t i) {
    return dtype == MRL_I32 ? (int64_t) reinterpret_cast<const int32_t*>(p)[i] : reinterpret_cast<const int64_t*>(p)[i];
}

__global__ __launch_bounds__(kBlock) void policy_loss_rows_kernel(
    const float* __restrict__ lp, const float* __restrict__ old, const float* __restrict__ ref,
    const float* __restrict__ adv, const float* __restrict__ ent, const void* __restrict__ mask, int mdtype,
    const void* __restrict__ lens, int ldtype, int64_t width, Params p, float* __restrict__ row_sums) {
    __shared__ double lds[kWaves];
    const int64_t i = blockIdx.x;
    float acc[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int64_t j = threadIdx.x; j < width; j += kBlock) {
        const float m = mask_at(mask, mdtype, lens, ldtype, i, j, width);
        if (m == 0.f) continue;           // values outside the mask never enter (NaN-safe)
        const int64_t e = i * width + j;
        const float lpe = lp[e];
        const Token t = token_terms<false>(lpe, old ? old[e] : 0.f, old != nullptr, ref ? ref[e] : 0.f, adv[e], p);
        acc[S_PG] += t.pg * m;
        acc[S_CLIP] += t.clipped * m;
        acc[S_PPOKL] += t.neg_logr * m;
        acc[S_KL] += t.kl * m;
        acc[S_ENT] += (ent ? ent[e] : 0.f) * m;
        acc[S_MASK] += m;
    }
#pragma unroll
    for (int q = 0; q < 6; ++q) {
        const double s = block_sum((double)acc[q], lds);
        if (threadIdx.x == 0) row_sums[i * S_N + q] = (float)s;
    }
    if (threadIdx.x == 0) {
        row_sums[i * S_N + 6] = 0.f;
        row_sums[i * S_N + 7] = 0.f;
    }
}

// Combines the per-sequence sums in a fixed order and writes the eight output scalars (and the loss
// once more to loss_out, if given: a 0-dim tensor of its own for autograd).  kCoherent: the sums were
// written by other workgroups of the SAME launch with device-scope stores and are read likewise.
template <bool kCoherent>
__device__ __forceinline__ void finalize_sums(const float* row_sums, int64_t batch, const Params& p,
                                              float* __restrict__ out, float* __restrict__ loss_out, double* lds) {
    auto at = [&](int64_t e) {
        return kCoherent ? __hip_atomic_load(row_sums + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : row_sums[e];
    };
    double acc[6] = {0, 0, 0, 0, 0, 0};
    double seq_acc = 0.0;
    for (int64_t i = threadIdx.x; i < batch; i += kBlock) {
        float v[6];
#pragma unroll
        for (int q = 0; q < 6; ++q) {
            v[q] = at(i * S_N + q);
            acc[q] += (double)v[q];
        }
        // per-sequence token mean, no epsilon: 0/0 = NaN for an all-masked row (as the reference)
        seq_acc += (double)(v[S_PG] / v[S_MASK]);
    }
    double tot[6];
#pragma unroll
    for (int q = 0; q < 6; ++q) tot[q] = block_sum(acc[q], lds);
    const double seq_tot = block_sum(seq_acc, lds);
    if (threadIdx.x == 0) {
        const double denom = tot[S_MASK] + 1e-8;
        const float clipfrac = p.seq_mean ? 0.f : (float)(tot[S_CLIP] / denom);
        const float pg_mean = p.seq_mean ? (float)(seq_tot / (double)batch) : (float)(tot[S_PG] / denom);
        const float ppo_kl = (float)(tot[S_PPOKL] / denom);
        const float kl_mean = p.kl_penalty == MRL_KL_NONE ? 0.f : (float)(tot[S_KL] / denom);
        const float ent_mean = (float)(tot[S_ENT] / denom);
        const float pg_loss = pg_mean + kl_mean * p.kl_coef - p.entropy_coeff * ent_mean;
        out[0] = pg_loss * p.loss_scale;
        out[1] = pg_loss;
        out[2] = clipfrac;
        out[3] = ppo_kl;
        out[4] = kl_mean;
        out[5] = ent_mean;
        out[6] = (float)tot[S_MASK];
        out[7] = (float)batch;
        if (loss_out) *loss_out = pg_loss * p.loss_scale;
    }
}

__global__ __launch_bounds__(kBlock) void policy_loss_finalize_kernel(const float* __restrict__ row_sums,
                                                                      int64_t batch, Params p,
                                                                      float* __restrict__ out,
                                                                      float* __restrict__ loss_out) {
    __shared__ double lds[kWaves];
    finalize_sums<false>(row_sums, batch, p, out, loss_out, lds);
}

__global__ __launch_bounds__(kBlock) void policy_loss_bwd_kernel(
    const float* __restrict__ lp, const float* __restrict__ old, const float* __restrict__ ref,
    const float* __restrict__ adv, const void* __restrict__ mask, int mdtype, const void* __restrict__ lens,
    int ldtype, int64_t batch, int64_t width, Params p, const float* __restrict__ row_sums,
    const float* __restrict__ out, const float* __restrict__ upstream, float* __restrict__ g_lp,
    float* __restrict__ g_ent) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= batch * width) return;
    const int64_t i = e / width;
    const int64_t j = e - i * width;
    const float m = mask_at(mask, mdtype, lens, ldtype, i, j, width);
    float glp = 0.f, gent = 0.f;
    const float up = (upstream ? *upstream : 1.f) * p.loss_scale;
    const float inv_tok = 1.f / (out[6] + 1e-8f);
    if (m != 0.f) {
        const Token t = token_terms<true>(lp[e], old ? old[e] : 0.f, old != nullptr, ref ? ref[e] : 0.f, adv[e], p);
        const float w_pg = p.seq_mean ? 1.f / ((float)batch * row_sums[i * S_N + S_MASK]) : inv_tok;
        glp = up * m * (w_pg * t.d_pg + p.kl_coef * inv_tok * t.d_kl);
        gent = up * m * (-p.entropy_coeff * inv_tok);
    } else if (p.seq_mean) {
        // a row whose mask sums to zero makes the reference's sequence mean 0/0: its gradient is NaN too
        const float msum = row_sums[i * S_N + S_MASK];
        if (msum == 0.f) glp = up * (0.f / msum);
    }
    g_lp[e] = glp;
    if (g_ent) g_ent[e] = gent;
}

// ----------------------------------------------------------------------------- fused-path helpers
// Window of logits rows that belongs to sequence i:
//   layout 0 (packed [T, V] logits): the window postprocess_packed_seqs copies
//   layout 1 (padded [B, S, V] logits): [P-1, P+R-1) clamped to [0, S], inside row block i
struct SeqArgs {
    int layout;
    int64_t width, padded_s;
    const int32_t* seqlens;
    const int32_t* cu;
    const void* prompt;
    int pdtype;
    const void* resp;
    int rdtype;
};

__device__ __forceinline__ void seq_window(const SeqArgs& a, int64_t i, int64_t& start, int64_t& n) {
    if (a.layout == 0) {
        start = (int64_t)a.cu[i];
        n = (int64_t)a.seqlens[i];
        if (a.prompt != nullptr) {
            const int64_t skip = load_i64(a.prompt, a.pdtype, i) - 1;
            if (skip < n) {
                n -= skip + 1;
                start += skip;
            }
        }
    } else {
        const int64_t p = load_i64(a.prompt, a.pdtype, i), r = load_i64(a.resp, a.rdtype, i);
        int64_t lo = p - 1, hi = p + r - 1;
        lo = lo < 0 ? 0 : (lo > a.padded_s ? a.padded_s : lo);
        hi = hi < 0 ? 0 : (hi > a.padded_s ? a.padded_s : hi);
        start = i * a.padded_s + lo;
        n = hi - lo;
    }
    if (n < 0) n = 0;
    if (n > a.width) n = a.width;
}

// One workgroup per sequence: its window and the sum of its mask row (the general form, for an
// explicit mask tensor or very many sequences).
__global__ __launch_bounds__(kBlock) void fused_seq_kernel(SeqArgs a, const void* __restrict__ mask, int mdtype,
                                                           int64_t* __restrict__ row_start,
                                                           int32_t* __restrict__ row_count,
                                                           float* __restrict__ seq_msum) {
    __shared__ double lds[kWaves];
    const int64_t i = blockIdx.x;
    float acc = 0.f;
    for (int64_t j = threadIdx.x; j < a.width; j += kBlock) acc += mask_at(mask, mdtype, a.resp, a.rdtype, i, j, a.width);
    const double msum = block_sum((double)acc, lds);
    if (threadIdx.x == 0) {
        int64_t start, n;
        seq_window(a, i, start, n);
        row_start[i] = start;
        row_count[i] = (int32_t)n;
        seq_msum[i] = (float)msum;
    }
}

// Sequences whose tables a workgroup of fused_row_ops_kernel<true> derives by itself, in LDS.
constexpr int kInlineSeqs = 2048;

// What the prepare step does besides the loss operands, folded into the same launch: the workspace
// of the sweep that follows is cleared (its row counter and half-row records start at zero), and the
// scale that the sweep will write into its gradients is fixed: scale_out[0] = scale_host * *scale_in,
// scale_out[1] = 0 (the counter mrl_scale_rows_note keeps next to the scale).
struct PrepareExtras {
    unsigned long long* clear;
    int64_t clear_words;
    const float* scale_in;
    float scale_host;
    float* scale_out;
};

// Loss operands of every logits row: one thread per row finds its (sequence, token) by a binary
// search over the window starts.  Every workgroup first re-derives N = sum of all mask sums in a
// fixed order (batch is small), so no extra launch or atomic is needed.  kInline: the mask is
// j < response_length[i] and the sequences are few, so every workgroup also derives the windows and
// mask sums itself (into LDS; workgroup 0 stores them for the reduce step) - no launch before this one.
template <bool kInline>
__global__ __launch_bounds__(kBlock) void fused_row_ops_kernel(
    SeqArgs sa, int64_t batch, int64_t n_rows, int64_t* row_start_g, int32_t* row_count_g, float* seq_msum_g,
    const float* __restrict__ old, const float* __restrict__ ref, const float* __restrict__ adv,
    const void* __restrict__ mask, int mdtype, int seq_mean, float* __restrict__ row_ops, PrepareExtras ex) {
    __shared__ double lds[kWaves];
    __shared__ int64_t s_start[kInline ? kInlineSeqs : 1];
    __shared__ int32_t s_count[kInline ? kInlineSeqs : 1];
    __shared__ float s_msum[kInline ? kInlineSeqs : 1];
    const int64_t width = sa.width;
    const int64_t gid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    for (int64_t w = gid; w < ex.clear_words; w += (int64_t)gridDim.x * kBlock) ex.clear[w] = 0ull;
    if (gid == 0 && ex.scale_out) {
        ex.scale_out[0] = ex.scale_host * (ex.scale_in ? *ex.scale_in : 1.f);
        ex.scale_out[1] = 0.f;
    }
    double part = 0.0;
    if (kInline) {
        for (int64_t i = threadIdx.x; i < batch; i += kBlock) {
            int64_t start, n;
            seq_window(sa, i, start, n);
            int64_t r = load_i64(sa.resp, sa.rdtype, i);
            r = r < 0 ? 0 : (r > width ? width : r);         // sum over j < width of (j < response_length)
            s_start[i] = start;
            s_count[i] = (int32_t)n;
            s_msum[i] = (float)r;
            part += (double)(float)r;
            if (blockIdx.x == 0) {
                row_start_g[i] = start;
                row_count_g[i] = (int32_t)n;
                seq_msum_g[i] = (float)r;
            }
        }
    } else {
        for (int64_t i = threadIdx.x; i < batch; i += kBlock) part += (double)seq_msum_g[i];
    }
    const double total = block_sum(part, lds);             // its barriers also publish the LDS tables
    const int64_t* row_start = kInline ? s_start : row_start_g;
    const int32_t* row_count = kInline ? s_count : row_count_g;
    const float* seq_msum = kInline ? s_msum : seq_msum_g;
    const float inv_tok = (float)(1.0 / (total + 1e-8));
    const int64_t t = gid;
    if (t >= n_rows) return;
    float o = 0.f, rf = 0.f, a = 0.f, m = 0.f, wpg = 0.f;
    if (batch > 0 && t >= row_start[0]) {
        int64_t lo = 0, hi = batch;                     // largest i with row_start[i] <= t
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if (row_start[mid] <= t) lo = mid; else hi = mid;
        }
        const int64_t i = lo, j = t - row_start[i];
        if (j < (int64_t)row_count[i]) {
            m = mask_at(mask, mdtype, sa.resp, sa.rdtype, i, j, width);
            if (m != 0.f) {
                const int64_t e = i * width + j;
                o = old ? old[e] : 0.f;
                rf = ref ? ref[e] : 0.f;
                a = adv[e];
                wpg = seq_mean ? 1.f / ((float)batch * seq_msum[i]) : inv_tok;
            }
        }
    }
    float* ops = row_ops + t * MRL_ROW_OPS;
    ops[MRL_OP_OLD] = o;
    ops[MRL_OP_REF] = rf;
    ops[MRL_OP_ADV] = a;
    ops[MRL_OP_MASK] = m;
    ops[MRL_OP_WPG] = wpg;
    ops[MRL_OP_INVTOK] = inv_tok;
    ops[6] = 0.f;
    ops[7] = 0.f;
}

// Per-sequence sums of the per-row loss terms written by the fused sweep.  Tokens that carry a
// non-zero mask but have no logits row (j >= row_count) enter with log_prob = entropy = 0, which
// is what they hold in the unpacked [B, L] tensor of the split path.
// done (nullable): a zeroed counter; the workgroup that finishes last then also combines the
// sequences' sums into the outputs (what policy_loss_finalize_kernel does in a launch of its own)
// and leaves the counter at zero again.  The sums then travel with device-scope stores and loads,
// which pass the caches that workgroups of one launch do not share.
__global__ __launch_bounds__(kBlock) void fused_seq_reduce_kernel(
    const float* __restrict__ row_terms, const int64_t* __restrict__ row_start, const int32_t* __restrict__ row_count,
    int64_t width, const float* __restrict__ old, const float* __restrict__ ref, const float* __restrict__ adv,
    const void* __restrict__ mask, int mdtype, const void* __restrict__ resp, int rdtype, Params p,
    float* row_sums, uint32_t* done, float* __restrict__ out, float* __restrict__ loss_out) {
    __shared__ double lds[kWaves];
    __shared__ uint32_t last;
    const int64_t i = blockIdx.x;
    const int64_t start = row_start[i];
    const int64_t count = row_count[i];
    float acc[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int64_t j = threadIdx.x; j < width; j += kBlock) {
        if (j < count) {
            const float* t = row_terms + (start + j) * S_N;
#pragma unroll
            for (int q = 0; q < 6; ++q) acc[q] += t[q];
        } else {
            const float m = mask_at(mask, mdtype, resp, rdtype, i, j, width);
            if (m == 0.f) continue;
            const int64_t e = i * width + j;
            const Token t = token_terms<false>(0.f, old ? old[e] : 0.f, old != nullptr, ref ? ref[e] : 0.f, adv[e], p);
            acc[S_PG] += t.pg * m;
            acc[S_CLIP] += t.clipped * m;
            acc[S_PPOKL] += t.neg_logr * m;
            acc[S_KL] += t.kl * m;
            acc[S_MASK] += m;
        }
    }
    float sums[S_N] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 6; ++q) sums[q] = (float)block_sum((double)acc[q], lds);
    if (threadIdx.x == 0) {
        if (done == nullptr) {
#pragma unroll
            for (int q = 0; q < S_N; ++q) row_sums[i * S_N + q] = sums[q];
        } else {
#pragma unroll
            for (int q = 0; q < S_N; ++q)
                __hip_atomic_store(row_sums + i * S_N + q, sums[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the sums are in memory before this one is counted
            last = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1 ? 1u : 0u;
        }
    }
    if (done == nullptr) return;
    __syncthreads();
    if (last == 0u) return;                                    // uniform
    finalize_sums<true>(row_sums, (int64_t)gridDim.x, p, out, loss_out, lds);
    if (threadIdx.x == 0) __hip_atomic_store(done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

int check_args(const char* fn, const float* lp, const float* ref, const float* adv, const void* mask, int mask_dtype,
               const void* lens, int length_dtype, int64_t batch, int64_t width, int kl_penalty, int seq_mean) {
    MRL_REQUIRE(batch >= 0 && width >= 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn, (long long)batch,
                (long long)width);
    MRL_REQUIRE(batch <= 0x7fffffffLL && (batch * width + kBlock - 1) / kBlock <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED,
                "%s: size exceeds the grid limit", fn);
    MRL_REQUIRE(kl_penalty >= MRL_KL_NONE && kl_penalty <= MRL_KL_LOW_VAR, MRL_ERR_INVALID_ARG, "%s: kl_penalty=%d", fn,
                kl_penalty);
    MRL_REQUIRE(seq_mean == 0 || seq_mean == 1, MRL_ERR_INVALID_ARG, "%s: seq_mean=%d", fn, seq_mean);
    MRL_REQUIRE(mask != nullptr || lens != nullptr || batch == 0, MRL_ERR_INVALID_ARG,
                "%s: need a mask or response lengths", fn);
    MRL_REQUIRE(mask == nullptr || mrl::mask_dtype_bytes(mask_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: mask dtype %d", fn,
                mask_dtype);
    MRL_REQUIRE(mask != nullptr || lens == nullptr || mrl::int_dtype_bytes(length_dtype) != 0, MRL_ERR_UNSUPPORTED,
                "%s: response_length dtype %d (want I32 or I64)", fn, length_dtype);
    if (batch * width == 0) return MRL_OK;
    MRL_REQUIRE(lp && adv, MRL_ERR_INVALID_ARG, "%s: log_prob and advantages are required", fn);
    MRL_REQUIRE(kl_penalty == MRL_KL_NONE || ref != nullptr, MRL_ERR_INVALID_ARG,
                "%s: ref_log_prob is required for kl_penalty %d", fn, kl_penalty);
    return MRL_OK;
}

}  // namespace

extern "C" int mrl_policy_loss_fwd(const float* log_prob, const float* old_log_prob, const float* ref_log_prob,
                                   const float* advantages, const float* entropy, const void* mask, int mask_dtype,
                                   const void* response_length, int length_dtype, int64_t batch, int64_t width,
                                   float clip_lo, float clip_hi, int kl_penalty, float kl_coef, float entropy_coeff,
                                   int seq_mean, float loss_scale, float* row_sums, float* out, void* stream) {
    const char* fn = "mrl_policy_loss_fwd";
    int rc = check_args(fn, log_prob, ref_log_prob, advantages, mask, mask_dtype, response_length, length_dtype, batch,
                        width, kl_penalty, seq_mean);
    if (rc != MRL_OK) return rc;
    MRL_REQUIRE(out != nullptr && (row_sums != nullptr || batch == 0), MRL_ERR_INVALID_ARG, "%s: NULL out or row_sums",
                fn);
    const Params p = {clip_lo, clip_hi, kl_coef, entropy_coeff, loss_scale, kl_penalty, seq_mean};
    hipStream_t s = mrl::as_stream(stream);
    if (batch > 0) {
        hipLaunchKernelGGL(policy_loss_rows_kernel, dim3((unsigned)batch), dim3(kBlock), 0, s, log_prob, old_log_prob,
                           ref_log_prob, advantages, entropy, mask, mask_dtype, response_length, length_dtype, width,
                           p, row_sums);
        rc = mrl::check_launch(fn);
        if (rc != MRL_OK) return rc;
    }
    hipLaunchKernelGGL(policy_loss_finalize_kernel, dim3(1), dim3(kBlock), 0, s, (const float*)row_sums, batch, p,
                       out, (float*)nullptr);
    return mrl::check_launch(fn);
}

extern "C" int mrl_policy_loss_bwd(const float* log_prob, const float* old_log_prob, const float* ref_log_prob,
                                   const float* advantages, const void* mask, int mask_dtype,
                                   const void* response_length, int length_dtype, int64_t batch, int64_t width,
                                   float clip_lo, float clip_hi, int kl_penalty, float kl_coef, float entropy_coeff,
                                   int seq_mean, float loss_scale, const float* row_sums, const float* out,
                                   const float* upstream, float* g_log_prob, float* g_entropy, void* stream) {
    const char* fn = "mrl_policy_loss_bwd";
    int rc = check_args(fn, log_prob, ref_log_prob, advantages, mask, mask_dtype, response_length, length_dtype, batch,
                        width, kl_penalty, seq_mean);
    if (rc != MRL_OK) return rc;
    if (batch * width == 0) return MRL_OK;
    MRL_REQUIRE(row_sums && out && g_log_prob, MRL_ERR_INVALID_ARG, "%s: NULL row_sums, out or g_log_prob", fn);
    const Params p = {clip_lo, clip_hi, kl_coef, entropy_coeff, loss_scale, kl_penalty, seq_mean};
    const unsigned blocks = (unsigned)((batch * width + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(policy_loss_bwd_kernel, dim3(blocks), dim3(kBlock), 0, mrl::as_stream(stream), log_prob,
                       old_log_prob, ref_log_prob, advantages, mask, mask_dtype, response_length, length_dtype, batch,
                       width, p, row_sums, out, upstream, g_log_prob, g_entropy);
    return mrl::check_launch(fn);
}

extern "C" int mrl_fused_loss_prepare(int layout, int64_t batch, int64_t width, int64_t n_rows, const int32_t* seqlens,
                                      const int32_t* cu_seqlens_padded, int64_t padded_seq_len,
                                      const void* prompt_length, int prompt_dtype, const void* response_length,
                                      int response_dtype, const float* old_log_prob, const float* ref_log_prob,
                                      const float* advantages, const void* mask, int mask_dtype, int seq_mean,
                                      int64_t* row_start, int32_t* row_count, float* seq_mask_sum, float* row_ops,
                                      void* sweep_workspace, int64_t sweep_workspace_bytes, const float* scale_in,
                                      float scale_host, float* scale_out, void* stream) {
    const char* fn = "mrl_fused_loss_prepare";
    MRL_REQUIRE(layout == 0 || layout == 1, MRL_ERR_INVALID_ARG, "%s: layout=%d (0 packed, 1 padded)", fn, layout);
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20) && width >= 0 && n_rows >= 0, MRL_ERR_INVALID_ARG,
                "%s: batch=%lld width=%lld n_rows=%lld", fn, (long long)batch, (long long)width, (long long)n_rows);
    MRL_REQUIRE((n_rows + kBlock - 1) / kBlock <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: n_rows exceeds the grid limit",
                fn);
    MRL_REQUIRE(seq_mean == 0 || seq_mean == 1, MRL_ERR_INVALID_ARG, "%s: seq_mean=%d", fn, seq_mean);
    MRL_REQUIRE(mask == nullptr || mrl::mask_dtype_bytes(mask_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: mask dtype %d", fn,
                mask_dtype);
    MRL_REQUIRE(prompt_length == nullptr || mrl::int_dtype_bytes(prompt_dtype) != 0, MRL_ERR_UNSUPPORTED,
                "%s: prompt_length dtype %d (want I32 or I64)", fn, prompt_dtype);
    MRL_REQUIRE(response_length == nullptr || mrl::int_dtype_bytes(response_dtype) != 0, MRL_ERR_UNSUPPORTED,
                "%s: response_length dtype %d (want I32 or I64)", fn, response_dtype);
    MRL_REQUIRE(n_rows == 0 || row_ops != nullptr, MRL_ERR_INVALID_ARG, "%s: row_ops is NULL", fn);
    MRL_REQUIRE(sweep_workspace_bytes >= 0 && sweep_workspace_bytes % 8 == 0 && mrl::aligned(sweep_workspace, 8) &&
                    (sweep_workspace != nullptr || sweep_workspace_bytes == 0),
                MRL_ERR_INVALID_ARG, "%s: the sweep workspace must be 8-byte aligned and a multiple of 8 bytes", fn);
    MRL_REQUIRE(mrl::aligned(scale_in, 4) && mrl::aligned(scale_out, 8), MRL_ERR_MISALIGNED,
                "%s: scale_in must be 4-byte and scale_out 8-byte aligned", fn);
    MRL_REQUIRE(n_rows > 0 || (sweep_workspace_bytes == 0 && scale_out == nullptr), MRL_ERR_INVALID_ARG,
                "%s: nothing clears a workspace or fixes a scale for an empty sweep", fn);
    if (batch > 0) {
        MRL_REQUIRE(row_start && row_count && seq_mask_sum && advantages, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
        MRL_REQUIRE(mask != nullptr || response_length != nullptr, MRL_ERR_INVALID_ARG,
                    "%s: need a mask or response lengths", fn);
        if (layout == 0) {
            MRL_REQUIRE(seqlens && cu_seqlens_padded, MRL_ERR_INVALID_ARG, "%s: packed layout needs seqlens and cu", fn);
        } else {
            MRL_REQUIRE(prompt_length && response_length && padded_seq_len >= 0, MRL_ERR_INVALID_ARG,
                        "%s: padded layout needs prompt_length, response_length and the padded length", fn);
        }
    }
    hipStream_t s = mrl::as_stream(stream);
    const SeqArgs sa = {layout, width, padded_seq_len, seqlens, cu_seqlens_padded, prompt_length, prompt_dtype,
                        response_length, response_dtype};
    const PrepareExtras ex = {reinterpret_cast<unsigned long long*>(sweep_workspace), sweep_workspace_bytes / 8, scale_in,
                              scale_host, scale_out};
    // the mask is implied by the response lengths and the sequences are few: one launch does it all
    const bool inline_tables = mask == nullptr && batch <= kInlineSeqs && n_rows > 0;
    if (batch > 0 && !inline_tables) {
        hipLaunchKernelGGL(fused_seq_kernel, dim3((unsigned)batch), dim3(kBlock), 0, s, sa, mask, mask_dtype, row_start,
                           row_count, seq_mask_sum);
        int rc = mrl::check_launch(fn);
        if (rc != MRL_OK) return rc;
    }
    if (n_rows > 0) {
        const dim3 grid((unsigned)((n_rows + kBlock - 1) / kBlock));
        if (inline_tables)
            hipLaunchKernelGGL(fused_row_ops_kernel<true>, grid, dim3(kBlock), 0, s, sa, batch, n_rows, row_start,
                               row_count, seq_mask_sum, old_log_prob, ref_log_prob, advantages, mask, mask_dtype, seq_mean,
                               row_ops, ex);
        else
            hipLaunchKernelGGL(fused_row_ops_kernel<false>, grid, dim3(kBlock), 0, s, sa, batch, n_rows, row_start,
                               row_count, seq_mask_sum, old_log_prob, ref_log_prob, advantages, mask, mask_dtype, seq_mean,
                               row_ops, ex);
        return mrl::check_launch(fn);
    }
    return MRL_OK;
}

extern "C" int mrl_fused_loss_reduce(const float* row_terms, const int64_t* row_start, const int32_t* row_count,
                                     int64_t batch, int64_t width, const float* old_log_prob,
                                     const float* ref_log_prob, const float* advantages, const void* mask,
                                     int mask_dtype, const void* response_length, int response_dtype, float clip_lo,
                                     float clip_hi, int kl_penalty, float kl_coef, float entropy_coeff, int seq_mean,
                                     float loss_scale, float* row_sums, float* out, uint32_t* done_counter,
                                     float* loss_out, void* stream) {
    const char* fn = "mrl_fused_loss_reduce";
    int rc = check_args(fn, (const float*)row_terms, ref_log_prob, advantages, mask, mask_dtype, response_length,
                        response_dtype, batch, width, kl_penalty, seq_mean);
    if (rc != MRL_OK) return rc;
    MRL_REQUIRE(out != nullptr && (batch == 0 || (row_sums && row_start && row_count)), MRL_ERR_INVALID_ARG,
                "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(done_counter, 4) && mrl::aligned(loss_out, 4), MRL_ERR_MISALIGNED,
                "%s: done_counter and loss_out must be 4-byte aligned", fn);
    const Params p = {clip_lo, clip_hi, kl_coef, entropy_coeff, loss_scale, kl_penalty, seq_mean};
    hipStream_t s = mrl::as_stream(stream);
    if (batch > 0) {
        hipLaunchKernelGGL(fused_seq_reduce_kernel, dim3((unsigned)batch), dim3(kBlock), 0, s, row_terms, row_start,
                           row_count, width, old_log_prob, ref_log_prob, advantages, mask, mask_dtype, response_length,
                           response_dtype, p, row_sums, done_counter, out, loss_out);
        rc = mrl::check_launch(fn);
        if (rc != MRL_OK || done_counter != nullptr) return rc;
    }
    hipLaunchKernelGGL(policy_loss_finalize_kernel, dim3(1), dim3(kBlock), 0, s, (const float*)row_sums, batch, p, out,
                       loss_out);
    return mrl::check_launch(fn);
}
