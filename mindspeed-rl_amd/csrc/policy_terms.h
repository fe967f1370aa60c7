// Per-token arithmetic of the GRPO / DAPO clipped-ratio loss, shared by the stand-alone policy
// loss kernels and the fused vocabulary sweep: torch-exact max / clamp semantics, the four KL
// penalties and their derivatives with respect to log_prob.
#pragma once

#include "mrl_internal.h"

namespace mrl_loss {

// slots of the per-sequence sums row_sums[i*8 + ...] and of the per-row terms
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

}  // namespace mrl_loss
