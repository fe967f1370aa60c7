// Fused lm_head + log-prob for gfx950: streams W_vocab x hidden^T tiles through bf16 MFMA and
// keeps an online log-sum-exp per token, so the [T, V] logits are never written to memory.
//
//   logits[t, v] = sum_k hidden[t, k] * W[v, k]        (bf16 operands, fp32 accumulate)
//   lse, logp[label], entropy exactly as the vocabulary sweep computes them, on the fp32 logits
//
// Mapping.  The product runs on the shared tile loop of lmhead_tile.h (256 x 256 tiles, one
// wavefront per SIMD with a 128 x 128 sub-tile of v_mfma_f32_16x16x32_bf16 blocks, operands straight
// from global memory into two LDS stages) with the vocabulary as the MFMA's M and the tokens as its
// N: in the 16x16 result layout a lane then owns ONE token column of each block and 4 vocabulary
// rows, so the softmax statistics of a token accumulate inside a lane; only the four lane quarters
// and the two vocabulary wavefronts have to be combined once, at the very end.  A workgroup owns
// 256 tokens and walks the 256-row vocabulary tiles of its vocabulary group; the groups (8, dealt so
// that the workgroups of one XCD share hidden blocks and weight tiles in its L2) leave per-group
// partial statistics that a small second kernel merges, together with the label logit (one fp32 dot
// product per token).
#include <stdlib.h>

#include <atomic>

#include "lmhead_tile.h"
#include "mrl_internal.h"
#include "vocab_common.h"

// Partial statistics of mrl_lmhead_logprob_fwd_static: device memory that belongs to the library,
// one copy per GPU that runs it, held until the process ends.  In host code this name is only a
// handle for hipGetSymbolAddress; kernels get the address that call returns.
#define MRL_LMHEAD_STATIC_MAX_TOKENS 65536
static __device__ __align__(256) float scratch[(size_t)MRL_LMHEAD_GROUPS * MRL_LMHEAD_STATIC_MAX_TOKENS * 4];

namespace {

using namespace mrl_vocab;

// The tiles of one workgroup: the vocabulary tiles of its group against its block of tokens.  The
// tile loop runs over the flattened (vocabulary tile, k-step) sequence, so the first loads of the
// next tile are in flight during the statistics of the current one.
struct VocabGroupTiles {
    int tile_begin, n_tiles, token_tile;
    __device__ __forceinline__ void coords(int j, int& tm, int& tn) const {
        tm = tile_begin + j;
        tn = token_tile;
    }
};

__global__ __launch_bounds__(mrl_tile::kThreads, 1) void lmhead_fwd_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight, int64_t n_tokens, int vocab, int hdim,
    int n_groups, int tiles_per_group, float k_scale, float* __restrict__ partial) {
    using namespace mrl_tile;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ Stats comb[2][kBlocks][16];       // [token wavefront][token block][lane % 16]

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wv = wave >> 1, wt = wave & 1;
    // Workgroups are dealt round-robin to the 8 XCDs and one round of 256 fills the chip.  The 32
    // workgroups that share an XCD (and its L2) in a round are 4 token tiles x 8 vocabulary groups:
    // the 8 that stream the same hidden block and the 4 that stream the same weight tiles run side
    // by side, so most of both streams hits in L2 (with one vocabulary group per XCD every
    // workgroup re-read its own hidden block from beyond the L2 for each vocabulary tile).
    const int xcd = blockIdx.x & 7, slot = (blockIdx.x >> 3) & 31, round = blockIdx.x >> 8;
    const int group = slot & 7;
    const int64_t ttile = (int64_t)(round * 8 + xcd) * 4 + (slot >> 3);
    const int64_t t0 = ttile * BN;
    if (t0 >= n_tokens) return;                 // padding of the last round
    const int n_vtiles = (vocab + BM - 1) / BM;
    VocabGroupTiles seq;
    seq.tile_begin = group * tiles_per_group;
    seq.n_tiles = max(0, min(seq.tile_begin + tiles_per_group, n_vtiles) - seq.tile_begin);
    seq.token_tile = (int)ttile;

    // a lane holds one token of each of its wavefront's 8 token blocks
    Stats st[kBlocks];
#pragma unroll
    for (int tb = 0; tb < kBlocks; ++tb) st[tb] = {kMaxInit, 0.f, 0.f};

    // online softmax statistics of a tile: per token block a lane holds 8 x 4 vocabulary rows
    auto tile_stats = [&](Accumulators& acc, int tm, int /*tn*/) {
        const int v0 = tm * BM + wv * 128 + 4 * (lane >> 4);       // + 16 vb + r
        const bool ragged = (tm * BM + BM > vocab);
#pragma unroll
        for (int tb = 0; tb < kBlocks; ++tb) {
            if (ragged) {
#pragma unroll
                for (int vb = 0; vb < kBlocks; ++vb)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (v0 + 16 * vb + r >= vocab) acc[vb][tb][r] = kMaxInit;
            }
            float vmax = st[tb].m;
#pragma unroll
            for (int vb = 0; vb < kBlocks; ++vb)
#pragma unroll
                for (int r = 0; r < 4; ++r) vmax = fmaxf(vmax, acc[vb][tb][r]);
            grow_max<true>(st[tb], vmax, k_scale);
            // A lane that has seen no valid vocabulary row yet (the first tile of its group is ragged and
            // ends above its rows) still holds the start value as its maximum: z * k - m * k of the masked
            // entries would then be the rounding residual of two numbers of magnitude 1e30 instead of
            // zero.  With an infinite m * k their exponentials are exactly 0.
            const float mk = st[tb].m > kMaxInit ? st[tb].m * k_scale : __builtin_inff();
#pragma unroll
            for (int vb = 0; vb < kBlocks; ++vb)
#pragma unroll
                for (int r = 0; r < 4; ++r) add_one<true>(st[tb], acc[vb][tb][r], k_scale, mk);
        }
    };
    mfma_tile_loop<false, false, 4>(smem, weight, hdim, vocab, hidden, hdim, (int)n_tokens, hdim, seq, tile_stats);

    // combine the four lane quarters (same token, other vocabulary rows), then the two vocabulary wavefronts
#pragma unroll
    for (int tb = 0; tb < kBlocks; ++tb) {
#pragma unroll
        for (int off = 16; off <= 32; off <<= 1) {
            Stats o;
            o.m = __shfl_xor(st[tb].m, off, 64);
            o.s = __shfl_xor(st[tb].s, off, 64);
            o.u = __shfl_xor(st[tb].u, off, 64);
            st[tb] = merge<true>(st[tb], o, k_scale);
        }
    }
    __syncthreads();
    if (wv == 1 && lane < 16) {
#pragma unroll
        for (int tb = 0; tb < kBlocks; ++tb) comb[wt][tb][lane] = st[tb];
    }
    __syncthreads();
    if (wv == 0 && lane < 16) {
#pragma unroll
        for (int tb = 0; tb < kBlocks; ++tb) {
            const Stats r = merge<true>(st[tb], comb[wt][tb][lane], k_scale);
            const int64_t t = t0 + wt * 128 + tb * 16 + lane;
            if (t < n_tokens) {
                float* p = partial + ((int64_t)group * n_tokens + t) * 4;
                p[0] = r.m;
                p[1] = r.s;
                p[2] = r.u;
                p[3] = 0.f;
            }
        }
    }
}

// One wavefront per token: merges the per-group partial statistics and computes the label logit
// as an fp32 dot product of the token's hidden row with the label's weight row.
template <typename LabelT>
__global__ __launch_bounds__(256) void lmhead_finish_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight, const LabelT* __restrict__ labels,
    const float* __restrict__ partial, int64_t n_tokens, int vocab, int hdim, int n_groups, float inv_t,
    float* __restrict__ logp, float* __restrict__ entropy, float* __restrict__ lse_out) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    const float k = inv_t * kLog2e;
    const int64_t y = (int64_t)labels[t];
    const bool y_ok = (y >= 0) && (y < (int64_t)vocab);
    float dot = 0.f;
    if (y_ok) {
        const uint16_t* hrow = hidden + t * hdim;
        const uint16_t* wrow = weight + y * hdim;
        for (int j = lane * 8; j < hdim; j += 64 * 8) {
            const u32x4 hv = *reinterpret_cast<const u32x4*>(hrow + j);
            const u32x4 wv = *reinterpret_cast<const u32x4*>(wrow + j);
            float a[8], b[8];
            Elem<MRL_BF16>::unpack(hv, a);
            Elem<MRL_BF16>::unpack(wv, b);
#pragma unroll
            for (int i = 0; i < 8; ++i) dot = __builtin_fmaf(a[i], b[i], dot);
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
    if (lane == 0) {
        Stats r = {kMaxInit, 0.f, 0.f};
        for (int g = 0; g < n_groups; ++g) {
            const float* p = partial + ((int64_t)g * n_tokens + t) * 4;
            const Stats o = {p[0], p[1], p[2]};
            r = merge<true>(r, o, k);
        }
        const float lse = (r.m * k + fast_log2(r.s)) * kLn2;
        logp[t] = (y_ok ? dot * inv_t : r.m * inv_t) - lse;
        if (entropy) entropy[t] = lse - (r.u / r.s) * inv_t;
        if (lse_out) lse_out[t] = lse;
    }
}

}  // namespace

extern "C" int64_t mrl_lmhead_workspace_bytes(int64_t n_tokens, int64_t vocab) {
    if (n_tokens < 0 || vocab <= 0) return 0;
    return (int64_t)MRL_LMHEAD_GROUPS * n_tokens * 4 * (int64_t)sizeof(float);
}

// Checks and launches shared by the two forward entry points; `partial` holds
// mrl_lmhead_workspace_bytes(n_tokens, vocab) bytes.
static int lmhead_forward(const char* fn, const void* hidden, const void* weight, int64_t n_tokens, int64_t vocab,
                          int64_t hidden_dim, const void* labels, int labels_dtype, float inv_temperature, float* logp,
                          float* entropy, float* lse, float* partial, hipStream_t s) {
    const int n_groups = MRL_LMHEAD_GROUPS;
    const int n_vtiles = (int)((vocab + mrl_tile::BM - 1) / mrl_tile::BM);
    // a group without tiles (tiny vocabularies) still writes its neutral partials
    const int tiles_per_group = (n_vtiles + n_groups - 1) / n_groups;
    // 256-token tiles, operands straight into two LDS stages (128 KiB of dynamic LDS).  Function
    // attributes belong to a device, so the reservation is made with every launch, on whichever
    // device is current.
    constexpr int kLdsBytes = mrl_tile::kLdsStages;
    const hipError_t attr = hipFuncSetAttribute((const void*)lmhead_fwd_kernel,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    MRL_REQUIRE(attr == hipSuccess, MRL_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", fn, kLdsBytes,
                hipGetErrorString(attr));
    MRL_REQUIRE(256 * hidden_dim * 2 < (1LL << 31) && n_tokens <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED,
                "%s: size out of range", fn);
    const int64_t n_ttiles = (n_tokens + mrl_tile::BN - 1) / mrl_tile::BN;
    const int64_t n_rounds = (n_ttiles + 31) / 32;       // 32 token tiles x 8 groups per round of 256 workgroups
    MRL_REQUIRE(n_rounds * 256 <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: grid too large", fn);
    static_assert(MRL_LMHEAD_GROUPS == 8, "the workgroup mapping assumes 8 vocabulary groups");
    hipLaunchKernelGGL(lmhead_fwd_kernel, dim3((unsigned)(n_rounds * 256)), dim3(mrl_tile::kThreads), kLdsBytes, s,
                       (const uint16_t*)hidden, (const uint16_t*)weight, n_tokens, (int)vocab, (int)hidden_dim,
                       n_groups, tiles_per_group, inv_temperature * kLog2e, partial);
    int rc = mrl::check_launch(fn);
    if (rc != MRL_OK) return rc;
    const dim3 fgrid((unsigned)((n_tokens + 3) / 4)), fblock(256);
    if (labels_dtype == MRL_I32) {
        hipLaunchKernelGGL(lmhead_finish_kernel<int32_t>, fgrid, fblock, 0, s, (const uint16_t*)hidden,
                           (const uint16_t*)weight, (const int32_t*)labels, (const float*)partial, n_tokens, (int)vocab,
                           (int)hidden_dim, n_groups, inv_temperature, logp, entropy, lse);
    } else {
        hipLaunchKernelGGL(lmhead_finish_kernel<int64_t>, fgrid, fblock, 0, s, (const uint16_t*)hidden,
                           (const uint16_t*)weight, (const int64_t*)labels, (const float*)partial, n_tokens, (int)vocab,
                           (int)hidden_dim, n_groups, inv_temperature, logp, entropy, lse);
    }
    return mrl::check_launch(fn);
}

#define MRL_LMHEAD_CHECK_ARGS(fn)                                                                                      \
    MRL_REQUIRE(n_tokens >= 0 && vocab > 0 && hidden_dim > 0, MRL_ERR_INVALID_ARG,                                     \
                "%s: n_tokens=%lld vocab=%lld hidden_dim=%lld", fn, (long long)n_tokens, (long long)vocab,             \
                (long long)hidden_dim);                                                                                \
    MRL_REQUIRE(hidden_dim % mrl_tile::BK == 0, MRL_ERR_UNSUPPORTED, "%s: hidden_dim=%lld must be a multiple of %d", fn, \
                (long long)hidden_dim, mrl_tile::BK);                                                                          \
    MRL_REQUIRE(vocab <= (1LL << 30) && hidden_dim <= (1LL << 20), MRL_ERR_UNSUPPORTED, "%s: size out of range", fn);  \
    MRL_REQUIRE(mrl::int_dtype_bytes(labels_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: labels dtype %d (want I32 or I64)", \
                fn, labels_dtype);                                                                                     \
    MRL_REQUIRE(inv_temperature > 0.f && inv_temperature < 1.0e6f, MRL_ERR_INVALID_ARG,                                \
                "%s: inv_temperature=%g must be in (0, 1e6)", fn, (double)inv_temperature)

extern "C" int mrl_lmhead_logprob_fwd(const void* hidden, const void* weight, int64_t n_tokens, int64_t vocab,
                                      int64_t hidden_dim, const void* labels, int labels_dtype,
                                      float inv_temperature, float* logp, float* entropy, float* lse,
                                      void* workspace, int64_t workspace_bytes, void* stream) {
    const char* fn = "mrl_lmhead_logprob_fwd";
    MRL_LMHEAD_CHECK_ARGS(fn);
    if (n_tokens == 0) return MRL_OK;
    MRL_REQUIRE(hidden && weight && labels && logp && workspace, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(hidden, 16) && mrl::aligned(weight, 16) && mrl::aligned(workspace, 16), MRL_ERR_MISALIGNED,
                "%s: hidden, weight and workspace must be 16-byte aligned", fn);
    MRL_REQUIRE(workspace_bytes >= mrl_lmhead_workspace_bytes(n_tokens, vocab), MRL_ERR_INVALID_ARG,
                "%s: workspace of %lld bytes, need %lld", fn, (long long)workspace_bytes,
                (long long)mrl_lmhead_workspace_bytes(n_tokens, vocab));
    return lmhead_forward(fn, hidden, weight, n_tokens, vocab, hidden_dim, labels, labels_dtype, inv_temperature, logp,
                          entropy, lse, (float*)workspace, mrl::as_stream(stream));
}

// Address of `scratch` on the current device, looked up once per device (each GPU holds its own
// copy of the array at its own address).  NULL and an error message if the lookup fails.
static float* static_scratch(const char* fn) {
    constexpr int kMaxDevices = 64;
    static std::atomic<float*> known[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        mrl::fail(MRL_ERR_LAUNCH, "%s: no current device (hipGetDevice gave %d)", fn, dev);
        return nullptr;
    }
    float* p = known[dev].load(std::memory_order_acquire);
    if (p) return p;
    void* addr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || addr == nullptr) {
        mrl::fail(MRL_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", fn, dev, hipGetErrorString(e));
        return nullptr;
    }
    known[dev].store((float*)addr, std::memory_order_release);
    return (float*)addr;
}

extern "C" int64_t mrl_lmhead_static_max_tokens(void) { return MRL_LMHEAD_STATIC_MAX_TOKENS; }

extern "C" int mrl_lmhead_logprob_fwd_static(const void* hidden, const void* weight, int64_t n_tokens, int64_t vocab,
                                             int64_t hidden_dim, const void* labels, int labels_dtype,
                                             float inv_temperature, float* logp, float* entropy, float* lse,
                                             void* stream) {
    const char* fn = "mrl_lmhead_logprob_fwd_static";
    MRL_LMHEAD_CHECK_ARGS(fn);
    MRL_REQUIRE(n_tokens <= MRL_LMHEAD_STATIC_MAX_TOKENS, MRL_ERR_UNSUPPORTED,
                "%s: n_tokens=%lld exceeds the %d tokens the library's own scratch memory holds; call it on slices of "
                "at most that many tokens, or use mrl_lmhead_logprob_fwd with a workspace",
                fn, (long long)n_tokens, MRL_LMHEAD_STATIC_MAX_TOKENS);
    if (n_tokens == 0) return MRL_OK;
    MRL_REQUIRE(hidden && weight && labels && logp, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(hidden, 16) && mrl::aligned(weight, 16), MRL_ERR_MISALIGNED,
                "%s: hidden and weight must be 16-byte aligned", fn);
    float* partial = static_scratch(fn);
    if (!partial) return MRL_ERR_LAUNCH;
    return lmhead_forward(fn, hidden, weight, n_tokens, vocab, hidden_dim, labels, labels_dtype, inv_temperature, logp,
                          entropy, lse, partial, mrl::as_stream(stream));
}
