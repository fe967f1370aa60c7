// GRPO / DAPO clipped-ratio policy loss for gfx950: forward (loss + the five statistics) and
// backward (dL/dlog_prob, dL/dentropy).
//
// Forward: one workgroup per sequence row reduces six masked sums over the row (fp32 per
// thread, fp64 across threads), a single-workgroup finalize kernel combines the rows in a fixed
// order - deterministic, no float atomics - and writes the eight output scalars.  Backward is
// one element-wise launch that re-derives each token's local gradient from the inputs and the
// saved denominators.
#include "mrl_internal.h"

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;

// slots of row_sums[i*8 + ...]
enum { S_PG = 0, S_CLIP = 1, S_PPOKL = 2, S_KL = 3, S_ENT = 4, S_MASK = 5, S_N = 8 };

struct Params {
    float clip_lo, clip_hi, kl_coef, entropy_coeff, loss_scale;
    int kl_penalty, seq_mean;
};

__device__ __forceinline__ float mask_at(const void* __restrict__ mask, int mdtype, const void* __restrict__ lens,
                                         int ldtype, int64_t i, int64_t j, int64_t width) {
    if (mask != nullptr) {
        const int64_t e = i * width + j;
        switch (mdtype) {
            case MRL_I64: return (float) reinterpret_cast<const int64_t*>(mask)[e];
            case MRL_I32: return (float) reinterpret_cast<const int32_t*>(mask)[e];
            case MRL_U8: return (float) reinterpret_cast<const uint8_t*>(mask)[e];
            default: return reinterpret_cast<const float*>(mask)[e];
        }
    }
    const int64_t n = ldtype == MRL_I32 ? (int64_t) reinterpret_cast<const int32_t*>(lens)[i]
                                        : reinterpret_cast<const int64_t*>(lens)[i];
    return j < n ? 1.f : 0.f;
}

// torch.maximum: NaN wins
__device__ __forceinline__ float torch_max(float a, float b) {
    if (a != a) return a;
    if (b != b) return b;
    return a > b ? a : b;
}

__device__ __forceinline__ float clampf(float x, float lo, float hi) {
    // torch.clamp(x, lo, hi) = min(max(x, lo), hi), NaN propagates
    if (x != x) return x;
    return fminf(fmaxf(x, lo), hi);
}

struct Token {
    float pg;        // max(surr1, surr2)
    float clipped;   // surr2 > surr1
    float neg_logr;  // old - lp
    float kl;        // KL penalty term
    float d_pg;      // d pg / d lp
    float d_kl;      // d kl / d lp
};

template <bool kGrad>
__device__ __forceinline__ Token token_terms(float lp, float old, bool has_old, float ref, float adv,
                                             const Params& p) {
    Token t;
    const float logr = has_old ? lp - old : 0.f;   // old == lp.detach() when absent
    const float ratio = expf(logr);
    t.neg_logr = -logr;
    const float na = -adv;
    const float clipped_ratio = clampf(ratio, p.clip_lo, p.clip_hi);
    const float s1 = na * ratio;
    const float s2 = na * clipped_ratio;
    t.pg = torch_max(s1, s2);
    t.clipped = s2 > s1 ? 1.f : 0.f;
    t.d_pg = 0.f;
    t.d_kl = 0.f;
    if (kGrad) {
        // d s1/d lp = na*ratio; d s2/d lp = na*ratio inside the closed clip interval, else 0;
        // torch.maximum sends the gradient to the larger operand and halves it on ties
        const float g1 = na * ratio;
        const float g2 = (ratio >= p.clip_lo && ratio <= p.clip_hi) ? g1 : 0.f;
        if (s1 > s2) t.d_pg = g1;
        else if (s2 > s1) t.d_pg = g2;
        else if (s1 == s2) t.d_pg = 0.5f * g1 + 0.5f * g2;
        else t.d_pg = s1 + s2;   // NaN operands: propagate NaN
    }
    switch (p.kl_penalty) {
        case MRL_KL_KL:
            t.kl = lp - ref;
            if (kGrad) t.d_kl = 1.f;
            break;
        case MRL_KL_ABS: {
            const float d = lp - ref;
            t.kl = fabsf(d);
            if (kGrad) t.d_kl = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
            break;
        }
        case MRL_KL_MSE: {
            const float d = lp - ref;
            t.kl = 0.5f * (d * d);
            if (kGrad) t.d_kl = d;
            break;
        }
        case MRL_KL_LOW_VAR: {
            const float raw = ref - lp;
            const float c = clampf(raw, -20.f, 20.f);
            const float e = expf(c);
            const float k3 = e - c - 1.f;
            t.kl = clampf(k3, -10.f, 10.f);
            if (kGrad) {
                const bool inner = raw >= -20.f && raw <= 20.f;
                const bool outer = k3 >= -10.f && k3 <= 10.f;
                t.d_kl = (inner && outer) ? -(e - 1.f) : 0.f;
            }
            break;
        }
        default:
            t.kl = 0.f;
            break;
    }
    return t;
}

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

__global__ __launch_bounds__(kBlock) void policy_loss_finalize_kernel(const float* __restrict__ row_sums,
                                                                      int64_t batch, Params p,
                                                                      float* __restrict__ out) {
    __shared__ double lds[kWaves];
    double acc[6] = {0, 0, 0, 0, 0, 0};
    double seq_acc = 0.0;
    for (int64_t i = threadIdx.x; i < batch; i += kBlock) {
#pragma unroll
        for (int q = 0; q < 6; ++q) acc[q] += (double)row_sums[i * S_N + q];
        // per-sequence token mean, no epsilon: 0/0 = NaN for an all-masked row (as the reference)
        seq_acc += (double)(row_sums[i * S_N + S_PG] / row_sums[i * S_N + S_MASK]);
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
    }
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
                       out);
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
