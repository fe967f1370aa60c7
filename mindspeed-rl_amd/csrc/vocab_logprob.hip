// Streaming vocabulary sweeps for gfx950: per-row log-softmax gather + entropy + logsumexp
// (forward, one read of the logits) and the fused dlogits (backward, one read + one write).
//
// Mapping: one workgroup of 256 threads (4 wavefronts) per token row.  A row is addressed as
// a run of 16-byte vectors; elements before the first / after the last aligned vector (only
// present for odd vocab sizes or strides) are handled with scalar loads by the first lanes.
// Each thread keeps an online (max, sum exp, sum exp*z) triple in fp32; a rescale happens at
// most once per group of kUnroll vectors and only when the running maximum grows, so the steady
// state costs one convert, one FMA and one v_exp_f32 per element.  Wavefront reduction uses
// cross-lane shuffles, the four wavefronts combine through LDS.
#include <stdlib.h>

#include "mrl_internal.h"
#include "row_sweep.h"
#include "vocab_common.h"

namespace {

using namespace mrl_vocab;

#ifndef MRL_VOCAB_BLOCK
#define MRL_VOCAB_BLOCK 256
#endif
#ifndef MRL_VOCAB_UNROLL
#define MRL_VOCAB_UNROLL 4
#endif
constexpr int kBlock = MRL_VOCAB_BLOCK;
constexpr int kWaves = kBlock / 64;
constexpr int kUnroll = MRL_VOCAB_UNROLL;
// Splits a row of `vocab` elements starting at `row` into head scalars, aligned 16-byte
// vectors and tail scalars.
template <typename T, int kVec>
struct RowSplit {
    int head;       // scalar elements before the first aligned vector
    int n_vec;      // aligned vectors
    int tail_begin; // element index of the first tail scalar
    __device__ __forceinline__ RowSplit(const T* row, int vocab) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(row);
        const int mis = (int)((a % 16) / sizeof(T));
        head = mis ? kVec - mis : 0;
        if (head > vocab) head = vocab;
        n_vec = (vocab - head) / kVec;
        tail_begin = head + n_vec * kVec;
    }
};

template <int DT, typename LabelT, bool kEntropy>
__global__ __launch_bounds__(kBlock) void vocab_fwd_kernel(
    const typename Elem<DT>::T* __restrict__ logits, int64_t row_stride, int vocab,
    const LabelT* __restrict__ labels, const uint8_t* __restrict__ row_active, float inv_t,
    float* __restrict__ logp, float* __restrict__ entropy, float* __restrict__ lse_out) {
    using E = Elem<DT>;
    using T = typename E::T;
    constexpr int kVec = E::kVec;
    __shared__ Stats lds[kWaves];

    const int64_t r = blockIdx.x;
    if (row_active != nullptr && row_active[r] == 0) {
        if (threadIdx.x == 0) {
            logp[r] = 0.f;
            if (entropy) entropy[r] = 0.f;
            if (lse_out) lse_out[r] = 0.f;
        }
        return;
    }
    const T* row = logits + r * row_stride;
    const float k = inv_t * kLog2e;

    // label logit: issued first so that its latency hides behind the sweep
    const int64_t y = (int64_t)labels[r];
    const bool y_ok = (y >= 0) && (y < (int64_t)vocab);
    float z_y = 0.f;
    if (threadIdx.x == 0 && y_ok) z_y = E::load(row + y);

    const RowSplit<T, kVec> sp(row, vocab);
    const u32x4* vec = reinterpret_cast<const u32x4*>(row + sp.head);

    Stats st = {kMaxInit, 0.f, 0.f};
    const int tid = threadIdx.x;

    // full groups of kUnroll vectors per thread: all loads issued before any use
    const int group = kBlock * kUnroll;
    const int n_full = (sp.n_vec / group) * group;
    for (int base = 0; base < n_full; base += group) {
        u32x4 v[kUnroll];
#pragma unroll
        for (int q = 0; q < kUnroll; ++q) v[q] = __builtin_nontemporal_load(vec + base + q * kBlock + tid);
        float z[kUnroll][kVec];
        float vmax = st.m;
#pragma unroll
        for (int q = 0; q < kUnroll; ++q) {
            E::unpack(v[q], z[q]);
#pragma unroll
            for (int i = 0; i < kVec; ++i) vmax = fmaxf(vmax, z[q][i]);
        }
        grow_max<kEntropy>(st, vmax, k);
        const float mk = st.m * k;
#pragma unroll
        for (int q = 0; q < kUnroll; ++q) {
#pragma unroll
            for (int i = 0; i < kVec; ++i) add_one<kEntropy>(st, z[q][i], k, mk);
        }
    }
    // remaining whole vectors
    for (int idx = n_full + tid; idx < sp.n_vec; idx += kBlock) {
        const u32x4 v = __builtin_nontemporal_load(vec + idx);
        float z[kVec];
        E::unpack(v, z);
        float vmax = st.m;
#pragma unroll
        for (int i = 0; i < kVec; ++i) vmax = fmaxf(vmax, z[i]);
        grow_max<kEntropy>(st, vmax, k);
        const float mk = st.m * k;
#pragma unroll
        for (int i = 0; i < kVec; ++i) add_one<kEntropy>(st, z[i], k, mk);
    }
    // head and tail scalars (absent when the row is 16-byte aligned and vocab % kVec == 0)
    {
        const int n_edge = sp.head + (vocab - sp.tail_begin);
        if (tid < n_edge) {
            const int j = tid < sp.head ? tid : sp.tail_begin + (tid - sp.head);
            const float z = E::load(row + j);
            grow_max<kEntropy>(st, z, k);
            add_one<kEntropy>(st, z, k, st.m * k);
        }
    }

    const Stats tot = block_reduce<kEntropy, kWaves>(st, k, lds);
    if (tid == 0) {
        // natural-log units of z' = z * inv_t
        const float lse = (tot.m * k + fast_log2(tot.s)) * kLn2;
        const float picked = y_ok ? z_y * inv_t : tot.m * inv_t;
        logp[r] = picked - lse;
        if (kEntropy) entropy[r] = lse - (tot.u / tot.s) * inv_t;
        if (lse_out) lse_out[r] = lse;
    }
}

// dlogits = e * (c0 + c1 * z) with e = 2^(z*k - lse*log2e), plus g at the label:
//   c0 = inv_t * (-g_lp + g_H * (lse - H)),  c1 = -g_H * inv_t^2
// The row is split by the alignment of the INPUT row; the host only selects this kernel when
// the output row reaches 16-byte alignment at the same element.  Built for DT_OUT == DT_IN and
// for DT_OUT == F32, so one input vector maps to one or two output vectors.
template <int DT_IN, int DT_OUT, typename LabelT, bool kEntropy>
__global__ __launch_bounds__(kBlock) void vocab_bwd_kernel(
    const typename Elem<DT_IN>::T* logits, int64_t row_stride, int vocab,
    const LabelT* __restrict__ labels, float inv_t, const float* __restrict__ lse_in,
    const float* __restrict__ ent_in, const float* __restrict__ g_logp,
    const float* __restrict__ g_entropy, typename Elem<DT_OUT>::T* dlogits, int64_t d_stride) {
    using EI = Elem<DT_IN>;
    using EO = Elem<DT_OUT>;
    using TI = typename EI::T;
    using TO = typename EO::T;
    constexpr int kStep = EI::kVec;
    constexpr int kVecO = EO::kVec;
    static_assert(kStep % kVecO == 0, "an input vector must cover whole output vectors");
    constexpr int kOutPer = kStep / kVecO;

    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    const TI* row = logits + r * row_stride;
    TO* drow = dlogits + r * d_stride;

    const float g_lp = g_logp ? g_logp[r] : 0.f;
    const float g_h = (kEntropy && g_entropy) ? g_entropy[r] : 0.f;
    const bool dead = (g_lp == 0.f) && (g_h == 0.f);

    const float k = inv_t * kLog2e;
    float lse2 = 0.f, c0 = 0.f, c1 = 0.f;
    if (!dead) {
        const float lse = lse_in[r];
        lse2 = lse * kLog2e;
        c0 = -g_lp * inv_t;
        if (kEntropy) {
            c0 = inv_t * (-g_lp + g_h * (lse - ent_in[r]));
            c1 = -g_h * inv_t * inv_t;
        }
    }
    const int64_t y = (int64_t)labels[r];
    const bool y_ok = (y >= 0) && (y < (int64_t)vocab) && !dead;
    const float g_onehot = g_lp * inv_t;

    auto grad_of = [&](float z) -> float {
        const float e = fast_exp2(__builtin_fmaf(z, k, -lse2));
        const float w = kEntropy ? __builtin_fmaf(c1, z, c0) : c0;
        return e * w;
    };

    const RowSplit<TI, kStep> sp(row, vocab);
    const u32x4* ivec = reinterpret_cast<const u32x4*>(row + sp.head);
    u32x4* ovec = reinterpret_cast<u32x4*>(drow + sp.head);
    const bool y_in_body = y_ok && y >= sp.head && y < sp.tail_begin;
    const int y_vec = y_in_body ? (int)((y - sp.head) / kStep) : -1;
    const int y_lane = y_in_body ? (int)((y - sp.head) % kStep) : 0;

    if (dead) {
        const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
        const int n_out = sp.n_vec * kOutPer;
        for (int idx = tid; idx < n_out; idx += kBlock) __builtin_nontemporal_store(zero, ovec + idx);
    } else {
        auto do_vec = [&](int idx, const u32x4& vin) {
            float z[kStep];
            float g[kStep];
            EI::unpack(vin, z);
#pragma unroll
            for (int i = 0; i < kStep; ++i) g[i] = grad_of(z[i]);
            if (idx == y_vec) {
#pragma unroll
                for (int i = 0; i < kStep; ++i)
                    if (i == y_lane) g[i] += g_onehot;
            }
#pragma unroll
            for (int p = 0; p < kOutPer; ++p) {
                float part[kVecO];
#pragma unroll
                for (int i = 0; i < kVecO; ++i) part[i] = g[p * kVecO + i];
                __builtin_nontemporal_store(EO::pack(part), ovec + (int64_t)idx * kOutPer + p);
            }
        };
        const int group = kBlock * kUnroll;
        const int n_full = (sp.n_vec / group) * group;
        for (int base = 0; base < n_full; base += group) {
            u32x4 v[kUnroll];
#pragma unroll
            for (int q = 0; q < kUnroll; ++q) v[q] = __builtin_nontemporal_load(ivec + base + q * kBlock + tid);
#pragma unroll
            for (int q = 0; q < kUnroll; ++q) do_vec(base + q * kBlock + tid, v[q]);
        }
        for (int idx = n_full + tid; idx < sp.n_vec; idx += kBlock) {
            const u32x4 v = __builtin_nontemporal_load(ivec + idx);
            do_vec(idx, v);
        }
    }
    // head and tail scalars
    const int n_edge = sp.head + (vocab - sp.tail_begin);
    if (tid < n_edge) {
        const int j = tid < sp.head ? tid : sp.tail_begin + (tid - sp.head);
        float g = 0.f;
        if (!dead) {
            g = grad_of(EI::load(row + j));
            if (y_ok && (int64_t)j == y) g += g_onehot;
        }
        EO::store(drow + j, g);
    }
}

// Fallback for rows whose input and output are not co-aligned to 16 bytes: scalar accesses.
template <int DT_IN, int DT_OUT, typename LabelT, bool kEntropy>
__global__ __launch_bounds__(kBlock) void vocab_bwd_scalar_kernel(
    const typename Elem<DT_IN>::T* logits, int64_t row_stride, int vocab,
    const LabelT* __restrict__ labels, float inv_t, const float* __restrict__ lse_in,
    const float* __restrict__ ent_in, const float* __restrict__ g_logp,
    const float* __restrict__ g_entropy, typename Elem<DT_OUT>::T* dlogits, int64_t d_stride) {
    using EI = Elem<DT_IN>;
    using EO = Elem<DT_OUT>;
    const int64_t r = blockIdx.x;
    const typename EI::T* row = logits + r * row_stride;
    typename EO::T* drow = dlogits + r * d_stride;
    const float g_lp = g_logp ? g_logp[r] : 0.f;
    const float g_h = (kEntropy && g_entropy) ? g_entropy[r] : 0.f;
    const bool dead = (g_lp == 0.f) && (g_h == 0.f);
    const float k = inv_t * kLog2e;
    float lse2 = 0.f, c0 = 0.f, c1 = 0.f;
    if (!dead) {
        const float lse = lse_in[r];
        lse2 = lse * kLog2e;
        c0 = -g_lp * inv_t;
        if (kEntropy) {
            c0 = inv_t * (-g_lp + g_h * (lse - ent_in[r]));
            c1 = -g_h * inv_t * inv_t;
        }
    }
    const int64_t y = (int64_t)labels[r];
    for (int j = threadIdx.x; j < vocab; j += kBlock) {
        float g = 0.f;
        if (!dead) {
            const float z = EI::load(row + j);
            const float e = fast_exp2(__builtin_fmaf(z, k, -lse2));
            g = e * (kEntropy ? __builtin_fmaf(c1, z, c0) : c0);
            if ((int64_t)j == y) g += g_lp * inv_t;
        }
        EO::store(drow + j, g);
    }
}

// ----------------------------------------------------------------------------- host dispatch
template <int DT, typename LabelT>
int launch_fwd(const void* logits, int64_t n_rows, int vocab, int64_t row_stride, const void* labels,
               const uint8_t* row_active, float inv_t, float* logp, float* entropy, float* lse,
               hipStream_t stream) {
    using T = typename Elem<DT>::T;
    const dim3 grid((unsigned)n_rows), block(kBlock);
    if (entropy) {
        hipLaunchKernelGGL((vocab_fwd_kernel<DT, LabelT, true>), grid, block, 0, stream, (const T*)logits,
                           row_stride, vocab, (const LabelT*)labels, row_active, inv_t, logp, entropy, lse);
    } else {
        hipLaunchKernelGGL((vocab_fwd_kernel<DT, LabelT, false>), grid, block, 0, stream, (const T*)logits,
                           row_stride, vocab, (const LabelT*)labels, row_active, inv_t, logp, entropy, lse);
    }
    return mrl::check_launch("mrl_vocab_logprob_fwd");
}

template <int DT_IN, int DT_OUT, typename LabelT>
int launch_bwd(const void* logits, int64_t n_rows, int vocab, int64_t row_stride, const void* labels,
               float inv_t, const float* lse, const float* ent, const float* g_lp, const float* g_h,
               void* dlogits, int64_t d_stride, bool vector_ok, hipStream_t stream) {
    using TI = typename Elem<DT_IN>::T;
    using TO = typename Elem<DT_OUT>::T;
    const dim3 grid((unsigned)n_rows), block(kBlock);
    const bool with_entropy = (g_h != nullptr);
#define MRL_BWD_LAUNCH(KERNEL, ENT)                                                                     \
    hipLaunchKernelGGL((KERNEL<DT_IN, DT_OUT, LabelT, ENT>), grid, block, 0, stream, (const TI*)logits, \
                       row_stride, vocab, (const LabelT*)labels, inv_t, lse, ent, g_lp, g_h,            \
                       (TO*)dlogits, d_stride)
    if (vector_ok) {
        if (with_entropy) MRL_BWD_LAUNCH(vocab_bwd_kernel, true);
        else MRL_BWD_LAUNCH(vocab_bwd_kernel, false);
    } else {
        if (with_entropy) MRL_BWD_LAUNCH(vocab_bwd_scalar_kernel, true);
        else MRL_BWD_LAUNCH(vocab_bwd_scalar_kernel, false);
    }
#undef MRL_BWD_LAUNCH
    return mrl::check_launch("mrl_vocab_logprob_bwd");
}

int check_common(const char* fn, const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                 int64_t row_stride, const void* labels, int labels_dtype, float inv_t) {
    MRL_REQUIRE(n_rows >= 0 && vocab > 0, MRL_ERR_INVALID_ARG, "%s: n_rows=%lld vocab=%lld", fn,
                (long long)n_rows, (long long)vocab);
    MRL_REQUIRE(n_rows <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: n_rows=%lld exceeds the grid limit", fn,
                (long long)n_rows);
    MRL_REQUIRE(vocab <= (1LL << 30), MRL_ERR_UNSUPPORTED, "%s: vocab=%lld exceeds 2^30", fn, (long long)vocab);
    const int eb = mrl::float_dtype_bytes(logits_dtype);
    MRL_REQUIRE(eb != 0, MRL_ERR_UNSUPPORTED, "%s: logits dtype %d (want F32, BF16 or F16)", fn, logits_dtype);
    MRL_REQUIRE(mrl::int_dtype_bytes(labels_dtype) != 0, MRL_ERR_UNSUPPORTED,
                "%s: labels dtype %d (want I32 or I64)", fn, labels_dtype);
    MRL_REQUIRE(row_stride >= vocab, MRL_ERR_INVALID_ARG, "%s: row_stride=%lld < vocab=%lld", fn,
                (long long)row_stride, (long long)vocab);
    if (n_rows == 0) return MRL_OK;
    MRL_REQUIRE(logits && labels, MRL_ERR_INVALID_ARG, "%s: NULL logits or labels", fn);
    MRL_REQUIRE(mrl::aligned(logits, eb), MRL_ERR_MISALIGNED, "%s: logits not aligned to %d bytes", fn, eb);
    MRL_REQUIRE(mrl::aligned(labels, mrl::int_dtype_bytes(labels_dtype)), MRL_ERR_MISALIGNED,
                "%s: labels misaligned", fn);
    MRL_REQUIRE(inv_t > 0.f && inv_t < 1.0e6f, MRL_ERR_INVALID_ARG, "%s: inv_temperature=%g must be in (0, 1e6)",
                fn, (double)inv_t);
    return MRL_OK;
}

}  // namespace

extern "C" int mrl_vocab_logprob_fwd(const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                                     int64_t row_stride, const void* labels, int labels_dtype,
                                     const uint8_t* row_active, float inv_temperature, float* logp,
                                     float* entropy, float* lse, void* stream) {
    const char* fn = "mrl_vocab_logprob_fwd";
    int rc = check_common(fn, logits, logits_dtype, n_rows, vocab, row_stride, labels, labels_dtype,
                          inv_temperature);
    if (rc != MRL_OK) return rc;
    if (n_rows == 0) return MRL_OK;
    MRL_REQUIRE(logp != nullptr, MRL_ERR_INVALID_ARG, "%s: logp is NULL", fn);
    MRL_REQUIRE(mrl::aligned(logp, 4) && mrl::aligned(entropy, 4) && mrl::aligned(lse, 4), MRL_ERR_MISALIGNED,
                "%s: fp32 outputs misaligned", fn);
    hipStream_t s = mrl::as_stream(stream);
    const int v = (int)vocab;
#define MRL_FWD(DT)                                                                                          \
    (labels_dtype == MRL_I32                                                                                 \
         ? launch_fwd<DT, int32_t>(logits, n_rows, v, row_stride, labels, row_active, inv_temperature, logp, \
                                   entropy, lse, s)                                                          \
         : launch_fwd<DT, int64_t>(logits, n_rows, v, row_stride, labels, row_active, inv_temperature, logp, \
                                   entropy, lse, s))
    switch (logits_dtype) {
        case MRL_F32: return MRL_FWD(MRL_F32);
        case MRL_BF16: return MRL_FWD(MRL_BF16);
        default: return MRL_FWD(MRL_F16);
    }
#undef MRL_FWD
}

extern "C" int mrl_vocab_logprob_bwd(const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                                     int64_t row_stride, const void* labels, int labels_dtype,
                                     float inv_temperature, const float* lse, const float* entropy,
                                     const float* g_logp, const float* g_entropy, void* dlogits,
                                     int dlogits_dtype, int64_t dlogits_row_stride, void* stream) {
    const char* fn = "mrl_vocab_logprob_bwd";
    int rc = check_common(fn, logits, logits_dtype, n_rows, vocab, row_stride, labels, labels_dtype,
                          inv_temperature);
    if (rc != MRL_OK) return rc;
    const int ob = mrl::float_dtype_bytes(dlogits_dtype);
    MRL_REQUIRE(ob != 0, MRL_ERR_UNSUPPORTED, "%s: dlogits dtype %d (want F32, BF16 or F16)", fn, dlogits_dtype);
    MRL_REQUIRE(dlogits_row_stride >= vocab, MRL_ERR_INVALID_ARG, "%s: dlogits_row_stride=%lld < vocab", fn,
                (long long)dlogits_row_stride);
    if (n_rows == 0) return MRL_OK;
    MRL_REQUIRE(dlogits != nullptr, MRL_ERR_INVALID_ARG, "%s: dlogits is NULL", fn);
    MRL_REQUIRE(mrl::aligned(dlogits, ob), MRL_ERR_MISALIGNED, "%s: dlogits misaligned", fn);
    MRL_REQUIRE(lse != nullptr, MRL_ERR_INVALID_ARG, "%s: lse is NULL", fn);
    MRL_REQUIRE(g_entropy == nullptr || entropy != nullptr, MRL_ERR_INVALID_ARG,
                "%s: g_entropy given without the forward's entropy", fn);
    // only same-dtype and fp32-output combinations are built
    MRL_REQUIRE(dlogits_dtype == logits_dtype || dlogits_dtype == MRL_F32, MRL_ERR_UNSUPPORTED,
                "%s: dlogits dtype %d must equal the logits dtype %d or be F32", fn, dlogits_dtype, logits_dtype);
    if (dlogits == logits) {
        MRL_REQUIRE(dlogits_dtype == logits_dtype && dlogits_row_stride == row_stride, MRL_ERR_INVALID_ARG,
                    "%s: in-place backward needs identical dtype and stride", fn);
    } else {
        // partial overlap would corrupt rows that other workgroups still read
        const char* a = (const char*)logits;
        const char* b = (const char*)dlogits;
        const int64_t a_bytes = ((n_rows - 1) * row_stride + vocab) * mrl::float_dtype_bytes(logits_dtype);
        const int64_t b_bytes = ((n_rows - 1) * dlogits_row_stride + vocab) * ob;
        MRL_REQUIRE(a + a_bytes <= b || b + b_bytes <= a, MRL_ERR_INVALID_ARG,
                    "%s: dlogits partially overlaps logits", fn);
    }
    // vector path: every input row and its output row must reach 16-byte alignment at the same
    // element (the kernel splits rows by the input pointer)
    const int ib = mrl::float_dtype_bytes(logits_dtype);
    bool vector_ok;
    {
        const uintptr_t pi = (uintptr_t)logits, po = (uintptr_t)dlogits;
        const int64_t vi = 16 / ib;
        const int64_t mis = (int64_t)((pi % 16) / ib);
        const int64_t head = mis ? vi - mis : 0;
        const bool out_aligned_at_head = ((po + (uintptr_t)(head * ob)) % 16) == 0;
        const bool strides_ok = ((row_stride * ib) % 16 == 0) && ((dlogits_row_stride * ob) % 16 == 0);
        vector_ok = out_aligned_at_head && (strides_ok || n_rows == 1);
    }
    hipStream_t s = mrl::as_stream(stream);
    const int v = (int)vocab;
    // rows from 16 KiB on, same dtype in and out: the streaming kernel (one vector per thread)
    if (dlogits_dtype == logits_dtype &&
        mrl::bwd_chunks_supported(logits_dtype, vocab, logits, row_stride, dlogits, dlogits_row_stride, n_rows)) {
        const mrl::BwdArgs a = {logits, logits_dtype, n_rows, vocab, row_stride, labels, labels_dtype, inv_temperature,
                                lse, entropy, g_logp, g_entropy, dlogits, dlogits_row_stride, s};
        return mrl::launch_bwd_chunks(a);
    }
#define MRL_BWD(DI, DO)                                                                                      \
    (labels_dtype == MRL_I32                                                                                 \
         ? launch_bwd<DI, DO, int32_t>(logits, n_rows, v, row_stride, labels, inv_temperature, lse, entropy, \
                                       g_logp, g_entropy, dlogits, dlogits_row_stride, vector_ok, s)         \
         : launch_bwd<DI, DO, int64_t>(logits, n_rows, v, row_stride, labels, inv_temperature, lse, entropy, \
                                       g_logp, g_entropy, dlogits, dlogits_row_stride, vector_ok, s))
    if (logits_dtype == MRL_F32) return MRL_BWD(MRL_F32, MRL_F32);
    if (logits_dtype == MRL_BF16)
        return dlogits_dtype == MRL_BF16 ? MRL_BWD(MRL_BF16, MRL_BF16) : MRL_BWD(MRL_BF16, MRL_F32);
    return dlogits_dtype == MRL_F16 ? MRL_BWD(MRL_F16, MRL_F16) : MRL_BWD(MRL_F16, MRL_F32);
#undef MRL_BWD
}
