// Group-relative advantage normalisation and the DAPO group filter for gfx950.
//
// Both are O(batch) scalar work plus one [batch, width] broadcast store; they exist as kernels so
// that the rewards never leave the device between rollout scoring and the loss.  The advantages are
// a segmented reduction: one wavefront reduces each group of consecutive rewards with shuffles.  fp64 is used
// where the reference uses it; the filter follows numpy's summation order exactly because its
// result is compared with zero.
#include "mrl_internal.h"

namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ float mask_as_float(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case MRL_I64: return (float) reinterpret_cast<const int64_t*>(p)[i];
        case MRL_I32: return (float) reinterpret_cast<const int32_t*>(p)[i];
        case MRL_U8: return (float) reinterpret_cast<const uint8_t*>(p)[i];
        default: return reinterpret_cast<const float*>(p)[i];
    }
}

__device__ __forceinline__ double reward_at(const void* p, int dtype, int64_t i) {
    return dtype == MRL_F64 ? reinterpret_cast<const double*>(p)[i]
                            : (double) reinterpret_cast<const float*>(p)[i];
}

// Segmented reduction over one group of `group` consecutive rewards by ONE wavefront, in fp64 and in a
// fixed order (lane l adds rewards l, l + 64, ... in sequence, then a butterfly of shuffles in which
// both partners form the same sum): mean and unbiased standard deviation, identical in every lane.
// All 64 lanes of the wavefront must call it.
struct GroupMoments {
    double mean, sd;
};

__device__ __forceinline__ double wave_sum_f64(double x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

__device__ __forceinline__ GroupMoments group_moments(const void* rewards, int rdtype, int64_t g0, int64_t group) {
    const int lane = threadIdx.x & 63;
    double part = 0.0;
    for (int64_t q = lane; q < group; q += 64) part += reward_at(rewards, rdtype, g0 + q);
    GroupMoments m;
    m.mean = wave_sum_f64(part) / (double)group;
    part = 0.0;
    for (int64_t q = lane; q < group; q += 64) {
        const double d = reward_at(rewards, rdtype, g0 + q) - m.mean;
        part += d * d;
    }
    m.sd = sqrt(wave_sum_f64(part) / (double)(group - 1));   // group == 1: 0/0 = NaN, like torch.std
    return m;
}

// One workgroup per GROUP: its first wavefront reduces the group's rewards (above), then the four
// wavefronts share the group's rows and write score * mask across each of them.
__global__ __launch_bounds__(kBlock) void group_advantage_kernel(const void* __restrict__ rewards, int rdtype,
                                                                 int64_t group, const void* __restrict__ mask,
                                                                 int mdtype, int64_t width,
                                                                 float* __restrict__ adv, float* __restrict__ ret) {
    __shared__ double moments_s[2];
    const int64_t g0 = (int64_t)blockIdx.x * group;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave == 0) {
        const GroupMoments m = group_moments(rewards, rdtype, g0, group);
        if (lane == 0) {
            moments_s[0] = m.mean;
            moments_s[1] = m.sd;
        }
    }
    __syncthreads();
    const double mean = moments_s[0], sd = moments_s[1];
    for (int64_t q = wave; q < group; q += kBlock / 64) {
        const int64_t i = g0 + q;
        const float score = (float)((reward_at(rewards, rdtype, i) - mean) / (sd + 1e-6));
        for (int64_t j = lane; j < width; j += 64) {
            const float v = score * mask_as_float(mask, mdtype, i * width + j);
            adv[i * width + j] = v;
            if (ret) ret[i * width + j] = v;
        }
    }
}

// One wavefront per group (four groups per workgroup): (r - mean) / (unbiased std + eps), fp64 internally.
__global__ __launch_bounds__(kBlock) void group_standardize_kernel(const void* __restrict__ rewards, int rdtype,
                                                                   int64_t n_groups, int64_t group, double eps,
                                                                   float* __restrict__ out) {
    const int64_t g = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (g >= n_groups) return;                              // whole wavefronts leave together
    const int64_t g0 = g * group;
    const GroupMoments m = group_moments(rewards, rdtype, g0, group);
    for (int64_t q = threadIdx.x & 63; q < group; q += 64)
        out[g0 + q] = (float)((reward_at(rewards, rdtype, g0 + q) - m.mean) / (m.sd + eps));
}

// numpy's arithmetic, one correctly rounded operation at a time (no FMA contraction)
template <typename F> struct Rn;
template <> struct Rn<double> {
    static __device__ __forceinline__ double add(double a, double b) { return mrl::add_rn(a, b); }
    static __device__ __forceinline__ double sub(double a, double b) { return mrl::sub_rn(a, b); }
    static __device__ __forceinline__ double mul(double a, double b) { return mrl::mul_rn(a, b); }
    static __device__ __forceinline__ double div(double a, double b) { return __ddiv_rn(a, b); }
    static __device__ __forceinline__ double root(double a) { return __dsqrt_rn(a); }
};
template <> struct Rn<float> {
    static __device__ __forceinline__ float add(float a, float b) { return mrl::add_rn(a, b); }
    static __device__ __forceinline__ float sub(float a, float b) { return mrl::sub_rn(a, b); }
    static __device__ __forceinline__ float mul(float a, float b) { return mrl::mul_rn(a, b); }
    static __device__ __forceinline__ float div(float a, float b) { return __fdiv_rn(a, b); }
    static __device__ __forceinline__ float root(float a) { return __fsqrt_rn(a); }
};

// numpy's pairwise summation of f(a[i]) over n contiguous elements: plain loop below 8, eight
// interleaved accumulators up to 128, halves (rounded down to a multiple of 8) above.
template <typename F, typename Fn>
__device__ F np_pairwise_sum(const F* a, int64_t n, Fn f) {
    if (n < 8) {
        F res = (F)0;
        for (int64_t i = 0; i < n; ++i) res = Rn<F>::add(res, f(a[i]));
        return res;
    }
    if (n <= 128) {
        F r[8];
        for (int q = 0; q < 8; ++q) r[q] = f(a[q]);
        int64_t i = 8;
        for (; i < n - (n % 8); i += 8)
            for (int q = 0; q < 8; ++q) r[q] = Rn<F>::add(r[q], f(a[i + q]));
        F res = Rn<F>::add(Rn<F>::add(Rn<F>::add(r[0], r[1]), Rn<F>::add(r[2], r[3])),
                           Rn<F>::add(Rn<F>::add(r[4], r[5]), Rn<F>::add(r[6], r[7])));
        for (; i < n; ++i) res = Rn<F>::add(res, f(a[i]));
        return res;
    }
    int64_t n2 = n / 2;
    n2 -= n2 % 8;
    return Rn<F>::add(np_pairwise_sum<F>(a, n2, f), np_pairwise_sum<F>(a + n2, n - n2, f));
}

// One thread per group: numpy.std(group) > 0 or len(group) == 1, written to every row of the group.
template <typename F>
__global__ __launch_bounds__(kBlock) void group_keep_kernel(const F* __restrict__ metric, int64_t n, int64_t group,
                                                            int64_t n_groups, uint8_t* __restrict__ keep) {
    const int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (g >= n_groups) return;
    const int64_t lo = g * group;
    const int64_t len = (lo + group <= n) ? group : (n - lo);
    const F* a = metric + lo;
    // 0 + pairwise(...) as the reduction starts from the additive identity
    const F total = Rn<F>::add((F)0, np_pairwise_sum<F>(a, len, [](F x) { return x; }));
    const F mean = Rn<F>::div(total, (F)len);
    const F ss = Rn<F>::add((F)0, np_pairwise_sum<F>(a, len, [mean](F x) {
                                 const F d = Rn<F>::sub(x, mean);
                                 return Rn<F>::mul(d, d);
                             }));
    const F sd = Rn<F>::root(Rn<F>::div(ss, (F)len));
    const uint8_t k = (sd > (F)0 || len == 1) ? 1 : 0;
    // the reference extends the kept list by a full group even when the last one is short
    for (int64_t q = 0; q < len; ++q) keep[lo + q] = k;
}

}  // namespace

extern "C" int mrl_group_advantage(const void* rewards, int rewards_dtype, int64_t batch, int64_t group,
                                   const void* mask, int mask_dtype, int64_t width, float* advantages,
                                   float* returns, void* stream) {
    const char* fn = "mrl_group_advantage";
    MRL_REQUIRE(rewards_dtype == MRL_F32 || rewards_dtype == MRL_F64, MRL_ERR_UNSUPPORTED,
                "%s: rewards dtype %d (want F32 or F64)", fn, rewards_dtype);
    MRL_REQUIRE(mrl::mask_dtype_bytes(mask_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: mask dtype %d", fn, mask_dtype);
    MRL_REQUIRE(batch >= 0 && width >= 0 && group >= 1, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld group=%lld", fn,
                (long long)batch, (long long)width, (long long)group);
    MRL_REQUIRE(batch % group == 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld is not a multiple of group=%lld", fn,
                (long long)batch, (long long)group);
    MRL_REQUIRE(batch <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: batch exceeds the grid limit", fn);
    if (batch == 0) return MRL_OK;
    MRL_REQUIRE(rewards && (mask || width == 0) && (advantages || width == 0), MRL_ERR_INVALID_ARG, "%s: NULL pointer",
                fn);
    MRL_REQUIRE(mrl::aligned(rewards, rewards_dtype == MRL_F64 ? 8 : 4) &&
                    mrl::aligned(mask, mrl::mask_dtype_bytes(mask_dtype)) && mrl::aligned(advantages, 4) &&
                    mrl::aligned(returns, 4),
                MRL_ERR_MISALIGNED, "%s: misaligned buffer", fn);
    if (width == 0) return MRL_OK;
    hipLaunchKernelGGL(group_advantage_kernel, dim3((unsigned)(batch / group)), dim3(kBlock), 0, mrl::as_stream(stream),
                       rewards, rewards_dtype, group, mask, mask_dtype, width, advantages, returns);
    return mrl::check_launch(fn);
}

extern "C" int mrl_group_keep_mask(const void* metric, int metric_dtype, int64_t n, int64_t group, uint8_t* keep,
                                   void* stream) {
    const char* fn = "mrl_group_keep_mask";
    MRL_REQUIRE(metric_dtype == MRL_F32 || metric_dtype == MRL_F64, MRL_ERR_UNSUPPORTED,
                "%s: metric dtype %d (want F32 or F64)", fn, metric_dtype);
    MRL_REQUIRE(n >= 0 && group >= 1, MRL_ERR_INVALID_ARG, "%s: n=%lld group=%lld", fn, (long long)n, (long long)group);
    if (n == 0) return MRL_OK;
    MRL_REQUIRE(metric && keep, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(metric, metric_dtype == MRL_F64 ? 8 : 4), MRL_ERR_MISALIGNED, "%s: metric misaligned", fn);
    const int64_t n_groups = (n + group - 1) / group;
    const unsigned blocks = (unsigned)((n_groups + kBlock - 1) / kBlock);
    hipStream_t s = mrl::as_stream(stream);
    if (metric_dtype == MRL_F64) {
        hipLaunchKernelGGL(group_keep_kernel<double>, dim3(blocks), dim3(kBlock), 0, s, (const double*)metric, n, group,
                           n_groups, keep);
    } else {
        hipLaunchKernelGGL(group_keep_kernel<float>, dim3(blocks), dim3(kBlock), 0, s, (const float*)metric, n, group,
                           n_groups, keep);
    }
    return mrl::check_launch(fn);
}

extern "C" int mrl_group_standardize(const void* rewards, int rewards_dtype, int64_t n, int64_t group, double eps,
                                     float* out, void* stream) {
    const char* fn = "mrl_group_standardize";
    MRL_REQUIRE(rewards_dtype == MRL_F32 || rewards_dtype == MRL_F64, MRL_ERR_UNSUPPORTED,
                "%s: rewards dtype %d (want F32 or F64)", fn, rewards_dtype);
    MRL_REQUIRE(n >= 0 && group >= 1, MRL_ERR_INVALID_ARG, "%s: n=%lld group=%lld", fn, (long long)n, (long long)group);
    MRL_REQUIRE(n % group == 0, MRL_ERR_INVALID_ARG, "%s: n=%lld is not a multiple of group=%lld", fn, (long long)n,
                (long long)group);
    if (n == 0) return MRL_OK;
    MRL_REQUIRE(rewards && out, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    const int64_t n_groups = n / group;
    MRL_REQUIRE(n_groups <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: too many groups", fn);
    const unsigned blocks = (unsigned)((n_groups + kBlock / 64 - 1) / (kBlock / 64));
    hipLaunchKernelGGL(group_standardize_kernel, dim3(blocks), dim3(kBlock), 0, mrl::as_stream(stream), rewards,
                       rewards_dtype, n_groups, group, eps, out);
    return mrl::check_launch(fn);
}
