// PPO's value side of the path: token-level rewards with the KL penalty, the GAE reverse scan, masked
// whitening, and the clipped value loss of the critic (forward and backward).  All operands are
// [batch, width] fp32 tensors of a few hundred thousand entries, so every kernel here is
// launch-bound; the layouts are chosen for determinism (fixed summation order, fp64 accumulators,
// no float atomics) and, for the scan, for the reference's exact operation order.
#include "mrl_internal.h"
#include "policy_terms.h"

namespace {

using namespace mrl_loss;

constexpr int kScanBlock = 256;
constexpr int kScanChunk = 2048;     // entries of a row staged in LDS per step of the scan
constexpr int kReduceBlock = 1024;

// Sum of one double per thread over a workgroup of kReduceBlock threads, fixed order; every thread
// gets the total.  `lds` holds kReduceBlock / 64 + 1 doubles.
__device__ __forceinline__ double block_sum(double x, double* lds) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int kWaves = kReduceBlock / 64;
    __syncthreads();                     // the previous call's total has been read by everyone
    if (lane == 0) lds[wave] = x;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int w = 0; w < kWaves; ++w) t += lds[w];
        lds[kWaves] = t;
    }
    __syncthreads();
    return lds[kWaves];
}

// ---------------------------------------------------------------------------- KL-penalised rewards
// One workgroup per sample: kld = penalty(old, ref) * mask, rewards = onehot(last response token) *
// score - beta * kld, row_kl = sum(kld * mask) / (sum(mask) + 1e-8).
__global__ __launch_bounds__(256) void kl_rewards_kernel(const float* __restrict__ old_lp,
                                                         const float* __restrict__ ref_lp,
                                                         const void* __restrict__ lens, int ldtype,
                                                         const float* __restrict__ scores, int64_t width, int penalty,
                                                         float beta, float* __restrict__ rewards,
                                                         float* __restrict__ row_kl) {
    __shared__ double part[256 / 64];
    const int64_t i = blockIdx.x;
    const int64_t n = ldtype == MRL_I32 ? (int64_t) reinterpret_cast<const int32_t*>(lens)[i]
                                        : reinterpret_cast<const int64_t*>(lens)[i];
    // python indexing of reward_tensor[i, n - 1]: a zero length lands on the last column
    int64_t hot = n - 1;
    if (hot < 0) hot += width;
    const float score = scores[i];
    Params p = {0.f, 0.f, 0.f, 0.f, 1.f, penalty, 0};
    double acc = 0.0;
    for (int64_t j = threadIdx.x; j < width; j += 256) {
        const int64_t e = i * width + j;
        const float m = j < n ? 1.f : 0.f;
        const Token t = token_terms<false>(old_lp[e], 0.f, false, ref_lp[e], 0.f, p);
        const float kld = t.kl * m;
        const float r = j == hot ? score : 0.f;
        rewards[e] = r - beta * kld;
        if (m != 0.f) acc += (double)(kld * m);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        const double s = part[0] + part[1] + part[2] + part[3];
        const float cnt = (float)(n < 0 ? 0 : (n > width ? width : n));
        row_kl[i] = (float)s / (cnt + 1e-8f);
    }
}

// ---------------------------------------------------------------------------- GAE reverse scan
// One workgroup per sample.  The recurrence lastgaelam = delta_t + (gamma*lam) * lastgaelam is
// evaluated by ONE thread in the reference's order and with its roundings (separate multiply and
// add, no contraction), so advantages and returns are bit-identical to the torch loop; the other
// threads stage the row through LDS in coalesced chunks and write the results.  gl is gamma*lam as
// the host formed it: python multiplies the two in double and torch rounds the product to fp32 once.
__global__ __launch_bounds__(kScanBlock) void gae_scan_kernel(const float* __restrict__ rewards,
                                                              const float* __restrict__ values, int64_t width,
                                                              float gamma, float gl, float* __restrict__ adv,
                                                              float* __restrict__ ret) {
    __shared__ float r_s[kScanChunk];
    __shared__ float v_s[kScanChunk + 1];
    __shared__ float a_s[kScanChunk];
    __shared__ float carry;
    const int64_t base = (int64_t)blockIdx.x * width;
    if (threadIdx.x == 0) carry = 0.f;
    for (int64_t hi = width; hi > 0; hi -= kScanChunk) {
        const int64_t lo = hi > kScanChunk ? hi - kScanChunk : 0;
        const int n = (int)(hi - lo);
        __syncthreads();
        for (int t = threadIdx.x; t < n; t += kScanBlock) {
            r_s[t] = rewards[base + lo + t];
            v_s[t] = values[base + lo + t];
        }
        if (threadIdx.x == 0) v_s[n] = hi < width ? values[base + hi] : 0.f;
        __syncthreads();
        if (threadIdx.x == 0) {
            float last = carry;
            for (int t = n - 1; t >= 0; --t) {
                const float delta = mrl::sub_rn(mrl::add_rn(r_s[t], mrl::mul_rn(gamma, v_s[t + 1])), v_s[t]);
                last = mrl::add_rn(delta, mrl::mul_rn(gl, last));
                a_s[t] = last;
            }
            carry = last;
        }
        __syncthreads();
        for (int t = threadIdx.x; t < n; t += kScanBlock) {
            adv[base + lo + t] = a_s[t];
            ret[base + lo + t] = mrl::add_rn(a_s[t], v_s[t]);
        }
    }
}

// ---------------------------------------------------------------------------- masked whitening
// One workgroup: mean and (Bessel-corrected) variance over the masked entries, then
// out = (x - mean) * rsqrt(var + 1e-8) (+ mean).  Sums in fp64, the scalar arithmetic in fp32 as in
// torch.  info[0] = number of masked entries (sum of the mask).
__global__ __launch_bounds__(kReduceBlock) void masked_whiten_kernel(const float* __restrict__ x,
                                                                    const void* __restrict__ mask, int mdtype,
                                                                    int64_t n, int shift_mean,
                                                                    float* __restrict__ out,
                                                                    double* __restrict__ info) {
    __shared__ double lds[kReduceBlock / 64 + 1];
    double s = 0.0, cnt = 0.0;
    for (int64_t e = threadIdx.x; e < n; e += kReduceBlock) {
        const float m = mask_at(mask, mdtype, nullptr, 0, 0, e, 0);
        cnt += (double)m;
        if (m != 0.f) s += (double)(x[e] * m);
    }
    const double total = block_sum(s, lds);
    const double count = block_sum(cnt, lds);
    const float denom = (float)count + 1e-8f;
    const float mean = (float)total / denom;
    double q = 0.0;
    for (int64_t e = threadIdx.x; e < n; e += kReduceBlock) {
        const float m = mask_at(mask, mdtype, nullptr, 0, 0, e, 0);
        if (m != 0.f) {
            const float c = x[e] - mean;
            q += (double)((c * c) * m);
        }
    }
    const double qsum = block_sum(q, lds);
    float var = (float)qsum / denom;
    const float fc = (float)count;
    if (fc != 1.f) var = var * (fc / (fc - 1.f));
    const float scale = 1.f / sqrtf(var + 1e-8f);
    for (int64_t e = threadIdx.x; e < n; e += kReduceBlock) {
        float w = (x[e] - mean) * scale;
        if (!shift_mean) w += mean;
        out[e] = w;
    }
    if (threadIdx.x == 0) {
        info[0] = count;
        info[1] = (double)mean;
        info[2] = (double)var;
    }
}

// ---------------------------------------------------------------------------- clipped value loss
struct ValueTerm {
    float loss;      // max((vp - ret)^2, (clamp(vp, v - c, v + c) - ret)^2)
    float clipped;   // second operand strictly larger
    float d;         // d loss / d vp
};

__device__ __forceinline__ ValueTerm value_term(float vp, float ret, float v, float c) {
    ValueTerm t;
    const float lo = v - c, hi = v + c;
    const float vc = clampf(vp, lo, hi);
    const float e1 = vp - ret, e2 = vc - ret;
    const float l1 = e1 * e1, l2 = e2 * e2;
    t.loss = torch_max(l1, l2);
    t.clipped = l2 > l1 ? 1.f : 0.f;
    const float d1 = 2.f * e1;
    const float d2 = (vp >= lo && vp <= hi) ? 2.f * e2 : 0.f;
    if (l1 > l2) t.d = d1;
    else if (l2 > l1) t.d = d2;
    else if (l1 == l2) t.d = 0.5f * d1 + 0.5f * d2;
    else t.d = l1 + l2;      // NaN operands propagate
    return t;
}

// out[0] = loss_scale * vf_loss, out[1] = vf_loss = 0.5 * masked_mean(max(l1, l2)), out[2] =
// masked_mean(l2 > l1), out[3] = sum(mask)
__global__ __launch_bounds__(kReduceBlock) void value_loss_fwd_kernel(
    const float* __restrict__ vpreds, const float* __restrict__ returns, const float* __restrict__ values,
    const void* __restrict__ mask, int mdtype, const void* __restrict__ lens, int ldtype, int64_t batch,
    int64_t width, float clip, float loss_scale, float* __restrict__ out) {
    __shared__ double lds[kReduceBlock / 64 + 1];
    double s = 0.0, cf = 0.0, cnt = 0.0;
    const int64_t n = batch * width;
    for (int64_t e = threadIdx.x; e < n; e += kReduceBlock) {
        const int64_t i = e / width, j = e - i * width;
        const float m = mask_at(mask, mdtype, lens, ldtype, i, j, width);
        cnt += (double)m;
        if (m != 0.f) {
            const ValueTerm t = value_term(vpreds[e], returns[e], values[e], clip);
            s += (double)(t.loss * m);
            cf += (double)(t.clipped * m);
        }
    }
    const double ssum = block_sum(s, lds);
    const double csum = block_sum(cf, lds);
    const double count = block_sum(cnt, lds);
    if (threadIdx.x == 0) {
        const float denom = (float)count + 1e-8f;
        const float vf = 0.5f * ((float)ssum / denom);
        out[0] = loss_scale * vf;
        out[1] = vf;
        out[2] = (float)csum / denom;
        out[3] = (float)count;
    }
}

__global__ __launch_bounds__(256) void value_loss_bwd_kernel(
    const float* __restrict__ vpreds, const float* __restrict__ returns, const float* __restrict__ values,
    const void* __restrict__ mask, int mdtype, const void* __restrict__ lens, int ldtype, int64_t batch,
    int64_t width, float clip, float loss_scale, const float* __restrict__ out, const float* __restrict__ upstream,
    float* __restrict__ g_vpreds) {
    const int64_t n = batch * width;
    const float coef = (*upstream) * loss_scale * 0.5f / (out[3] + 1e-8f);
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        const int64_t i = e / width, j = e - i * width;
        const float m = mask_at(mask, mdtype, lens, ldtype, i, j, width);
        float g = 0.f;
        if (m != 0.f) g = coef * m * value_term(vpreds[e], returns[e], values[e], clip).d;
        g_vpreds[e] = g;
    }
}

int check_mask(const char* fn, const void* mask, int mask_dtype, const void* lens, int lens_dtype) {
    MRL_REQUIRE(mask != nullptr || lens != nullptr, MRL_ERR_INVALID_ARG, "%s: neither mask nor response_length given", fn);
    if (mask != nullptr)
        MRL_REQUIRE(mrl::mask_dtype_bytes(mask_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: mask dtype %d", fn, mask_dtype);
    else
        MRL_REQUIRE(mrl::int_dtype_bytes(lens_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: response_length dtype %d", fn,
                    lens_dtype);
    return MRL_OK;
}

}  // namespace

extern "C" int mrl_kl_token_rewards(const float* old_log_prob, const float* ref_log_prob,
                                    const void* response_length, int length_dtype, const float* scores,
                                    int64_t batch, int64_t width, int kl_penalty, float beta, float* rewards,
                                    float* row_kl, void* stream) {
    const char* fn = "mrl_kl_token_rewards";
    MRL_REQUIRE(batch >= 0 && width > 0 && batch <= 0x7fffffffLL, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn,
                (long long)batch, (long long)width);
    MRL_REQUIRE(kl_penalty >= MRL_KL_KL && kl_penalty <= MRL_KL_LOW_VAR, MRL_ERR_INVALID_ARG, "%s: kl_penalty=%d", fn,
                kl_penalty);
    MRL_REQUIRE(mrl::int_dtype_bytes(length_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: response_length dtype %d", fn,
                length_dtype);
    if (batch == 0) return MRL_OK;
    MRL_REQUIRE(old_log_prob && ref_log_prob && response_length && scores && rewards && row_kl, MRL_ERR_INVALID_ARG,
                "%s: NULL pointer", fn);
    hipLaunchKernelGGL(kl_rewards_kernel, dim3((unsigned)batch), dim3(256), 0, mrl::as_stream(stream), old_log_prob,
                       ref_log_prob, response_length, length_dtype, scores, width, kl_penalty, beta, rewards, row_kl);
    return mrl::check_launch(fn);
}

extern "C" int mrl_gae_scan(const float* rewards, const float* values, int64_t batch, int64_t width, float gamma,
                            float gamma_lam, float* advantages, float* returns, void* stream) {
    const char* fn = "mrl_gae_scan";
    MRL_REQUIRE(batch >= 0 && width > 0 && batch <= 0x7fffffffLL, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn,
                (long long)batch, (long long)width);
    if (batch == 0) return MRL_OK;
    MRL_REQUIRE(rewards && values && advantages && returns, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(advantages != rewards && advantages != values && returns != rewards && returns != values &&
                    advantages != returns,
                MRL_ERR_INVALID_ARG, "%s: outputs must not alias the inputs or each other", fn);
    hipLaunchKernelGGL(gae_scan_kernel, dim3((unsigned)batch), dim3(kScanBlock), 0, mrl::as_stream(stream), rewards,
                       values, width, gamma, gamma_lam, advantages, returns);
    return mrl::check_launch(fn);
}

extern "C" int mrl_masked_whiten(const float* x, const void* mask, int mask_dtype, int64_t n, int shift_mean,
                                 float* out, double* info, void* stream) {
    const char* fn = "mrl_masked_whiten";
    MRL_REQUIRE(n >= 0, MRL_ERR_INVALID_ARG, "%s: n=%lld", fn, (long long)n);
    MRL_REQUIRE(mrl::mask_dtype_bytes(mask_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: mask dtype %d", fn, mask_dtype);
    MRL_REQUIRE(info != nullptr, MRL_ERR_INVALID_ARG, "%s: info is NULL", fn);
    MRL_REQUIRE(n == 0 || (x && mask && out), MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    hipLaunchKernelGGL(masked_whiten_kernel, dim3(1), dim3(kReduceBlock), 0, mrl::as_stream(stream), x, mask, mask_dtype,
                       n, shift_mean, out, info);
    return mrl::check_launch(fn);
}

extern "C" int mrl_value_loss_fwd(const float* vpreds, const float* returns, const float* values, const void* mask,
                                  int mask_dtype, const void* response_length, int length_dtype, int64_t batch,
                                  int64_t width, float cliprange_value, float loss_scale, float* out, void* stream) {
    const char* fn = "mrl_value_loss_fwd";
    MRL_REQUIRE(batch >= 0 && width > 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn, (long long)batch,
                (long long)width);
    int rc = check_mask(fn, mask, mask_dtype, response_length, length_dtype);
    if (rc != MRL_OK) return rc;
    MRL_REQUIRE(out != nullptr && (batch == 0 || (vpreds && returns && values)), MRL_ERR_INVALID_ARG, "%s: NULL pointer",
                fn);
    hipLaunchKernelGGL(value_loss_fwd_kernel, dim3(1), dim3(kReduceBlock), 0, mrl::as_stream(stream), vpreds, returns,
                       values, mask, mask_dtype, response_length, length_dtype, batch, width, cliprange_value, loss_scale,
                       out);
    return mrl::check_launch(fn);
}

extern "C" int mrl_value_loss_bwd(const float* vpreds, const float* returns, const float* values, const void* mask,
                                  int mask_dtype, const void* response_length, int length_dtype, int64_t batch,
                                  int64_t width, float cliprange_value, float loss_scale, const float* out,
                                  const float* upstream, float* g_vpreds, void* stream) {
    const char* fn = "mrl_value_loss_bwd";
    MRL_REQUIRE(batch >= 0 && width > 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn, (long long)batch,
                (long long)width);
    int rc = check_mask(fn, mask, mask_dtype, response_length, length_dtype);
    if (rc != MRL_OK) return rc;
    if (batch == 0) return MRL_OK;
    MRL_REQUIRE(vpreds && returns && values && out && upstream && g_vpreds, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    const int64_t n = batch * width;
    const unsigned grid = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    hipLaunchKernelGGL(value_loss_bwd_kernel, dim3(grid), dim3(256), 0, mrl::as_stream(stream), vpreds, returns, values,
                       mask, mask_dtype, response_length, length_dtype, batch, width, cliprange_value, loss_scale, out,
                       upstream, g_vpreds);
    return mrl::check_launch(fn);
}
