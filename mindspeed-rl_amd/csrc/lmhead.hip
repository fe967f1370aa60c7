// Fused lm_head + log-prob for gfx950: streams hidden x W_vocab^T tiles through bf16 MFMA and
// keeps an online log-sum-exp per token, so the [T, V] logits are never written to memory.
//
//   logits[t, v] = sum_k hidden[t, k] * W[v, k]        (bf16 operands, fp32 accumulate)
//   lse, logp[label], entropy exactly as the vocabulary sweep computes them, on the fp32 logits
//
// Mapping.  The product is computed TRANSPOSED, S^T = W_tile x hidden_tile^T with
// v_mfma_f32_32x32x16_bf16: vocabulary rows are the MFMA's M, tokens its N.  In the 32x32 result
// layout a lane then owns ONE token column and 16 vocabulary rows, so the softmax statistics of a
// token accumulate inside a lane; only the two lane halves and the two vocabulary wavefronts have
// to be combined once, at the very end.  A workgroup (256 threads = 2x2 wavefronts) owns 128 tokens
// and walks over the 256-row vocabulary tiles of its vocabulary group; each wavefront computes a
// 128 (vocab) x 64 (token) sub-tile = 4x2 MFMA blocks per 16-wide k-step, operands staged through
// LDS (rows padded to 144 bytes), the next k-step's global loads in flight during the MFMAs.
// Vocabulary groups (gridDim = token tiles x groups, group = blockIdx % groups so that the
// workgroups of one XCD read the same W rows) leave per-group partial statistics that a small
// second kernel merges, together with the label logit (one fp32 dot product per token).
#include <stdlib.h>

#include <atomic>

#include "mrl_internal.h"
#include "vocab_common.h"

// Partial statistics of mrl_lmhead_logprob_fwd_static: device memory that belongs to the library,
// one copy per GPU that runs it, held until the process ends.  In host code this name is only a
// handle for hipGetSymbolAddress; kernels get the address that call returns.
#define MRL_LMHEAD_STATIC_MAX_TOKENS 65536
static __device__ __align__(256) float scratch[(size_t)MRL_LMHEAD_GROUPS * MRL_LMHEAD_STATIC_MAX_TOKENS * 4];

namespace {

using namespace mrl_vocab;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BV = 256;            // vocabulary rows per macro tile
// tokens per macro tile = 64 * kTB: each of the two token wavefronts owns kTB 32-token MFMA blocks
constexpr int BK = 64;             // k elements per LDS stage
constexpr int kLdsStride = BK + 8; // bf16 elements per LDS row: 144 bytes, breaks the bank pattern
constexpr int kChunksPerRow = BK / 8;                          // 16-byte chunks per row and stage
constexpr int kALoads = BV * kChunksPerRow / kThreads;         // 8 chunks per thread

template <int kTB>
__global__ __launch_bounds__(kThreads, (kTB <= 2 ? 2 : 1)) void lmhead_fwd_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight, int64_t n_tokens, int vocab, int hdim,
    int n_groups, int tiles_per_group, float k_scale, float* __restrict__ partial) {
    __shared__ __attribute__((aligned(16))) uint16_t As[BV * kLdsStride];
    constexpr int BT = 64 * kTB;
    constexpr int kBLoads = BT * kChunksPerRow / kThreads;
    __shared__ __attribute__((aligned(16))) uint16_t Bs[BT * kLdsStride];
    __shared__ Stats comb[2][kTB][32];   // [token half][token block][lane % 32]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wv = wave >> 1, wt = wave & 1;
    const int group = blockIdx.x % n_groups;
    const int64_t t0 = (int64_t)(blockIdx.x / n_groups) * BT;
    const int n_vtiles = (vocab + BV - 1) / BV;
    const int tile_begin = group * tiles_per_group;
    const int tile_end = min(tile_begin + tiles_per_group, n_vtiles);

    // global -> LDS staging: chunk c = tid + i*256 covers row c/8, 16-byte column c%8
    const int ld_row = tid >> 3, ld_col = tid & 7;
    // token rows of this workgroup as 32-bit element offsets from the tile base, clamped so that
    // tail rows read valid memory (they are masked on output)
    const uint16_t* b_base = hidden + t0 * hdim;
    int b_off[kBLoads];
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
        int64_t r = ld_row + 32 * i;
        if (t0 + r >= n_tokens) r = n_tokens - 1 - t0;
        b_off[i] = (int)r * hdim + ld_col * 8;
    }

    Stats st[kTB];
#pragma unroll
    for (int tb = 0; tb < kTB; ++tb) st[tb] = {kMaxInit, 0.f, 0.f};

    for (int tile = tile_begin; tile < tile_end; ++tile) {
        const int v0 = tile * BV;
        const uint16_t* a_base = weight + (int64_t)v0 * hdim;
        int a_off[kALoads];
#pragma unroll
        for (int i = 0; i < kALoads; ++i) {
            int r = ld_row + 32 * i;
            if (v0 + r >= vocab) r = vocab - 1 - v0;
            a_off[i] = r * hdim + ld_col * 8;
        }
        floatx16 acc[4][kTB];
#pragma unroll
        for (int vb = 0; vb < 4; ++vb)
#pragma unroll
            for (int tb = 0; tb < kTB; ++tb)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[vb][tb][i] = 0.f;

        u32x4 a_reg[kALoads], b_reg[kBLoads];
#pragma unroll
        for (int i = 0; i < kALoads; ++i) a_reg[i] = *reinterpret_cast<const u32x4*>(a_base + a_off[i]);
#pragma unroll
        for (int i = 0; i < kBLoads; ++i) b_reg[i] = *reinterpret_cast<const u32x4*>(b_base + b_off[i]);

        const int n_ksteps = hdim / BK;
        for (int kstep = 0; kstep < n_ksteps; ++kstep) {
            __syncthreads();                               // the previous stage has been consumed
#pragma unroll
            for (int i = 0; i < kALoads; ++i)
                *reinterpret_cast<u32x4*>(&As[(ld_row + 32 * i) * kLdsStride + ld_col * 8]) = a_reg[i];
#pragma unroll
            for (int i = 0; i < kBLoads; ++i)
                *reinterpret_cast<u32x4*>(&Bs[(ld_row + 32 * i) * kLdsStride + ld_col * 8]) = b_reg[i];
            __syncthreads();
            if (kstep + 1 < n_ksteps) {                    // next stage's loads fly during the MFMAs
                const int off = (kstep + 1) * BK;
#pragma unroll
                for (int i = 0; i < kALoads; ++i) a_reg[i] = *reinterpret_cast<const u32x4*>(a_base + off + a_off[i]);
#pragma unroll
                for (int i = 0; i < kBLoads; ++i) b_reg[i] = *reinterpret_cast<const u32x4*>(b_base + off + b_off[i]);
            }
#pragma unroll
            for (int ks = 0; ks < BK / 16; ++ks) {
                const int koff = ks * 16 + (lane >> 5) * 8;
                bf16x8 af[4], bfr[kTB];
#pragma unroll
                for (int vb = 0; vb < 4; ++vb)
                    af[vb] = *reinterpret_cast<const bf16x8*>(&As[(wv * 128 + vb * 32 + (lane & 31)) * kLdsStride + koff]);
#pragma unroll
                for (int tb = 0; tb < kTB; ++tb)
                    bfr[tb] = *reinterpret_cast<const bf16x8*>(&Bs[(wt * 32 * kTB + tb * 32 + (lane & 31)) * kLdsStride + koff]);
#pragma unroll
                for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                    for (int tb = 0; tb < kTB; ++tb)
                        acc[vb][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[vb], bfr[tb], acc[vb][tb], 0, 0, 0);
            }
        }

        // online softmax statistics of this tile: a lane holds 64 vocabulary rows of each token column
        const bool ragged = (v0 + BV > vocab);
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb) {
            if (ragged) {
#pragma unroll
                for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int v = v0 + wv * 128 + vb * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
                        if (v >= vocab) acc[vb][tb][i] = kMaxInit;
                    }
            }
            float vmax = st[tb].m;
#pragma unroll
            for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                for (int i = 0; i < 16; ++i) vmax = fmaxf(vmax, acc[vb][tb][i]);
            grow_max<true>(st[tb], vmax, k_scale);
            // A lane that has seen no valid vocabulary row yet (the first tile of its group is ragged and
            // ends above its rows) still holds the start value as its maximum: z * k - m * k of the masked
            // entries would then be the rounding residual of two numbers of magnitude 1e30 instead of
            // zero.  With an infinite m * k their exponentials are exactly 0.
            const float mk = st[tb].m > kMaxInit ? st[tb].m * k_scale : __builtin_inff();
#pragma unroll
            for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                for (int i = 0; i < 16; ++i) add_one<true>(st[tb], acc[vb][tb][i], k_scale, mk);
        }
    }

    // combine the two lane halves (same token, other vocabulary rows), then the two vocabulary wavefronts
#pragma unroll
    for (int tb = 0; tb < kTB; ++tb) {
        Stats o;
        o.m = __shfl_xor(st[tb].m, 32, 64);
        o.s = __shfl_xor(st[tb].s, 32, 64);
        o.u = __shfl_xor(st[tb].u, 32, 64);
        st[tb] = merge<true>(st[tb], o, k_scale);
    }
    __syncthreads();
    if (wv == 1 && lane < 32) {
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb) comb[wt][tb][lane] = st[tb];
    }
    __syncthreads();
    if (wv == 0 && lane < 32) {
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb) {
            const Stats r = merge<true>(st[tb], comb[wt][tb][lane], k_scale);
            const int64_t t = t0 + wt * 32 * kTB + tb * 32 + lane;
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

// ------------------------------------------------------------------------------------------
// Second generation of the tile loop: a 512-thread workgroup (2 x 4 wavefronts, one workgroup per
// CU) owns 256 vocabulary rows x 256 tokens, so each wavefront keeps the 128 x 64 sub-tile of the
// kernel above but every staged byte feeds twice the MFMA work.  Operands go from global memory
// straight into LDS (global_load_lds_dwordx4: no staging registers, no ds_write), into one of two
// stage buffers, so the loads of k-step s+1 run during the MFMAs of k-step s and a k-step costs
// ONE barrier.  A direct load puts lane i of a wavefront at LDS byte base + 16 i, which rules out
// padded rows; instead the 16-byte chunks are XOR-swizzled inside each 256-byte pair of rows:
//   physical slot (0..15) = logical slot ^ (pair index & 15),  logical slot = (row & 1) * 8 + chunk
// The 16 lanes that a ds_read_b128 serves together read 16 consecutive rows at one chunk, i.e. 8
// pairs x 2 rows -> 16 different slots -> all 64 banks, no conflict.  The loop runs over the
// flattened (vocabulary tile, k-step) sequence, so the first loads of the next tile are in flight
// during the softmax statistics of the current one.
constexpr int kThreads2 = 512;
constexpr int BT2 = 256;                         // tokens per workgroup
constexpr int kOperandBytes = 256 * BK * 2;      // one operand of one stage: 256 rows x 128 bytes
constexpr int kStageBytes = 2 * kOperandBytes;   // A (weights) then B (hidden)
constexpr int kLdsBytes2 = 2 * kStageBytes;      // two stages

// Global element offset (row * hdim + column, without the k-step) of the chunk that lane `lane`
// of wavefront `wave` brings in with its load j (0..3) of an operand whose tile has `rows_valid`
// rows left (rows beyond are clamped to the last valid one and masked later).
__device__ __forceinline__ int stage_src_offset(int wave, int lane, int j, int hdim, int rows_valid) {
    const int phys_row = (wave * 4 + j) * 8 + (lane >> 3);
    const int pair = phys_row >> 1;
    const int slot = ((phys_row & 1) << 3) | (lane & 7);
    const int logical = slot ^ (pair & 15);
    int row = 2 * pair + (logical >> 3);
    if (row >= rows_valid) row = rows_valid - 1;
    return row * hdim + (logical & 7) * 8;
}

__global__ __launch_bounds__(kThreads2, 1) void lmhead_fwd_kernel_v2(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight, int64_t n_tokens, int vocab, int hdim,
    int n_groups, int tiles_per_group, float k_scale, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ Stats comb[4][2][32];             // [token wavefront][token block][lane % 32]
    constexpr int kTB = 2;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wv = wave >> 2, wt = wave & 3;
    // Workgroups are dealt round-robin to the 8 XCDs and one round of 256 fills the chip.  The 32
    // workgroups that share an XCD (and its L2) in a round are 4 token tiles x 8 vocabulary groups:
    // the 8 that stream the same hidden block and the 4 that stream the same weight tiles run side
    // by side, so most of both streams hits in L2 (with one vocabulary group per XCD every
    // workgroup re-read its own hidden block from beyond the L2 for each vocabulary tile).
    const int xcd = blockIdx.x & 7, slot = (blockIdx.x >> 3) & 31, round = blockIdx.x >> 8;
    const int group = slot & 7;
    const int64_t ttile = (int64_t)(round * 8 + xcd) * 4 + (slot >> 3);
    const int64_t t0 = ttile * BT2;
    if (t0 >= n_tokens) return;                 // padding of the last round
    const int n_vtiles = (vocab + BV - 1) / BV;
    const int tile_begin = group * tiles_per_group;
    const int tile_end = min(tile_begin + tiles_per_group, n_vtiles);
    const int n_ksteps = hdim / BK;

    // sources of this lane's four chunks per operand and stage
    const uint16_t* b_base = hidden + t0 * hdim;
    const int tokens_valid = (int)min((int64_t)BT2, n_tokens - t0);
    int b_off[4], a_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b_off[j] = stage_src_offset(wave, lane, j, hdim, tokens_valid);

    // Buffer (MUBUF) form of the LDS load on purpose: the global_load_lds form is a FLAT instruction
    // that touches two address spaces, and while one is pending the compiler turns every LDS wait
    // into lgkmcnt(0), which would undo the fragment pipeline below.
    const mrl::rsrc_t w_rsrc = mrl::make_rsrc(weight, 0xffffffffu);
    const mrl::rsrc_t h_rsrc = mrl::make_rsrc(b_base, 0xffffffffu);
    auto issue = [&](int tile, int kstep, int buf) {
        const uint32_t a_tile = (uint32_t)(((int64_t)tile * BV * hdim + kstep * BK) * 2);
        const uint32_t b_tile = (uint32_t)(kstep * BK * 2);
        unsigned char* dst = smem + buf * kStageBytes + (wave * 4) * 1024;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (void __attribute__((address_space(3)))*)(dst + j * 1024), 16,
                                                 a_off[j] * 2, a_tile, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(h_rsrc,
                                                 (void __attribute__((address_space(3)))*)(dst + kOperandBytes + j * 1024),
                                                 16, b_off[j] * 2, b_tile, 0, 0);
    };
    auto set_a_rows = [&](int tile) {
        const int rows_valid = min(BV, vocab - tile * BV);
#pragma unroll
        for (int j = 0; j < 4; ++j) a_off[j] = stage_src_offset(wave, lane, j, hdim, rows_valid);
    };

    // fragment addresses: row (lane & 31) of a 32-row block, chunk 2 ks + (lane >> 5)
    const int frag_pair = (lane & 31) >> 1;
    const int frag_slot = (((lane & 1) << 3) | (lane >> 5)) ^ frag_pair;          // ^ (2 ks) per k sub-step
    const int a_frag = (wv * 64) * 256 + frag_pair * 256;                          // + vb * 16 * 256
    const int b_frag = kOperandBytes + (wt * 32) * 256 + frag_pair * 256;          // + tb * 16 * 256

    Stats st[kTB];
#pragma unroll
    for (int tb = 0; tb < kTB; ++tb) st[tb] = {kMaxInit, 0.f, 0.f};

    // The (tile, k-step) stages are numbered 0 .. n_stages-1; stage s lives in buffer s & 1.
    const int n_stages = (tile_end > tile_begin ? tile_end - tile_begin : 0) * n_ksteps;
    int next_tile = tile_begin, next_k = 0;      // the stage that is requested next
    auto issue_next = [&](int buf) {
        if (next_k == 0) set_a_rows(next_tile);
        issue(next_tile, next_k, buf);
        if (++next_k == n_ksteps) {
            next_k = 0;
            ++next_tile;
        }
    };
    struct Frags {
        bf16x8 a[4], b[kTB];
    };
    auto read_frags = [&](Frags& f, const unsigned char* stage, int ks) {
        const int slot_bytes = (frag_slot ^ (2 * ks)) * 16;
#pragma unroll
        for (int vb = 0; vb < 4; ++vb)
            f.a[vb] = *reinterpret_cast<const bf16x8*>(stage + a_frag + vb * 16 * 256 + slot_bytes);
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb)
            f.b[tb] = *reinterpret_cast<const bf16x8*>(stage + b_frag + tb * 16 * 256 + slot_bytes);
    };
    floatx16 acc[4][kTB];
    auto zero_acc = [&]() {
#pragma unroll
        for (int vb = 0; vb < 4; ++vb)
#pragma unroll
            for (int tb = 0; tb < kTB; ++tb)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[vb][tb][i] = 0.f;
    };
    auto mma = [&](const Frags& f) {
#pragma unroll
        for (int vb = 0; vb < 4; ++vb)
#pragma unroll
            for (int tb = 0; tb < kTB; ++tb)
                acc[vb][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[vb], f.b[tb], acc[vb][tb], 0, 0, 0);
    };

    if (n_stages > 0) {
        Frags f0, f1;
        issue_next(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): stage 0 has landed
        __syncthreads();
        if (n_stages > 1) issue_next(1);
        read_frags(f0, smem, 0);
        zero_acc();
        int tile = tile_begin, kstep = 0;
        for (int stage_idx = 0; stage_idx < n_stages; ++stage_idx) {
            const int buf = stage_idx & 1;
            const unsigned char* stage = smem + buf * kStageBytes;
            // software pipeline: the fragments of sub-step ks+1 are requested before the MFMAs of ks
            read_frags(f1, stage, 1);
            __builtin_amdgcn_sched_barrier(0);
            mma(f0);
            __builtin_amdgcn_sched_barrier(0);
            read_frags(f0, stage, 2);
            __builtin_amdgcn_sched_barrier(0);
            mma(f1);
            __builtin_amdgcn_sched_barrier(0);
            read_frags(f1, stage, 3);
            __builtin_amdgcn_sched_barrier(0);
            mma(f0);
            __builtin_amdgcn_sched_barrier(0);
            // The last fragments of this stage are in registers and the next stage has landed: after
            // the barrier this buffer may be overwritten, and the first fragments of the next stage are
            // requested before the last MFMAs of this one are issued.  The barrier and the read are
            // unconditional (after the last stage the read fetches unused bytes of the other buffer): a
            // branch around them would make the wait before the MFMAs cover the new request as well.
            __builtin_amdgcn_s_waitcnt(0x0070);            // vmcnt(0) lgkmcnt(0)
            __syncthreads();
            read_frags(f0, smem + (buf ^ 1) * kStageBytes, 0);
            __builtin_amdgcn_sched_barrier(0);
            mma(f1);
            __builtin_amdgcn_sched_barrier(0);
            // the stage after next goes into the buffer that the barrier has just freed; requested
            // after the MFMAs so that its address arithmetic does not hold them up (measured: 6 % faster
            // than right after the barrier; spreading the requests over the next stage was slower)
            if (stage_idx + 2 < n_stages) issue_next(buf);
            __builtin_amdgcn_sched_barrier(0);
            if (++kstep == n_ksteps) {
                // online softmax statistics of this tile: a lane holds 64 vocabulary rows of each token column
                const int v0 = tile * BV;
                const bool ragged = (v0 + BV > vocab);
#pragma unroll
                for (int tb = 0; tb < kTB; ++tb) {
                    if (ragged) {
#pragma unroll
                        for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                            for (int i = 0; i < 16; ++i) {
                                const int v = v0 + wv * 128 + vb * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
                                if (v >= vocab) acc[vb][tb][i] = kMaxInit;
                            }
                    }
                    float vmax = st[tb].m;
#pragma unroll
                    for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                        for (int i = 0; i < 16; ++i) vmax = fmaxf(vmax, acc[vb][tb][i]);
                    grow_max<true>(st[tb], vmax, k_scale);
                    // no valid vocabulary row seen yet by this lane: see the first-generation kernel
                    const float mk = st[tb].m > kMaxInit ? st[tb].m * k_scale : __builtin_inff();
#pragma unroll
                    for (int vb = 0; vb < 4; ++vb)
#pragma unroll
                        for (int i = 0; i < 16; ++i) add_one<true>(st[tb], acc[vb][tb][i], k_scale, mk);
                }
                zero_acc();
                kstep = 0;
                ++tile;
            }
        }
    }

    // combine the two lane halves (same token, other vocabulary rows), then the two vocabulary wavefronts
#pragma unroll
    for (int tb = 0; tb < kTB; ++tb) {
        Stats o;
        o.m = __shfl_xor(st[tb].m, 32, 64);
        o.s = __shfl_xor(st[tb].s, 32, 64);
        o.u = __shfl_xor(st[tb].u, 32, 64);
        st[tb] = merge<true>(st[tb], o, k_scale);
    }
    __syncthreads();
    if (wv == 1 && lane < 32) {
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb) comb[wt][tb][lane] = st[tb];
    }
    __syncthreads();
    if (wv == 0 && lane < 32) {
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb) {
            const Stats r = merge<true>(st[tb], comb[wt][tb][lane], k_scale);
            const int64_t t = t0 + wt * 64 + tb * 32 + lane;
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

// MRL_LMHEAD_V2=0 selects the first-generation tile loop (a tuning / debugging switch).
bool lmhead_v2_enabled() {
    static const bool on = [] {
        const char* e = getenv("MRL_LMHEAD_V2");
        return !(e && e[0] == '0');
    }();
    return on;
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
    const int n_vtiles = (int)((vocab + BV - 1) / BV);
    const int tiles_per_group = (n_vtiles + n_groups - 1) / n_groups;
    // a group without tiles (tiny vocabularies) still writes its neutral partials
    // the second-generation loop addresses the weights with 32-bit byte offsets
    if (lmhead_v2_enabled() && vocab * hidden_dim * 2 < (1LL << 32)) {
        // 256-token tiles, operands straight into two LDS stages (128 KiB of dynamic LDS)
        static const hipError_t attr = hipFuncSetAttribute((const void*)lmhead_fwd_kernel_v2,
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes2);
        MRL_REQUIRE(attr == hipSuccess, MRL_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", fn, kLdsBytes2,
                    hipGetErrorString(attr));
        const int64_t n_ttiles = (n_tokens + BT2 - 1) / BT2;
        const int64_t n_rounds = (n_ttiles + 31) / 32;       // 32 token tiles x 8 groups per round of 256 workgroups
        MRL_REQUIRE(n_rounds * 256 <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: grid too large", fn);
        static_assert(MRL_LMHEAD_GROUPS == 8, "the workgroup mapping assumes 8 vocabulary groups");
        hipLaunchKernelGGL(lmhead_fwd_kernel_v2, dim3((unsigned)(n_rounds * 256)), dim3(kThreads2), kLdsBytes2, s,
                           (const uint16_t*)hidden, (const uint16_t*)weight, n_tokens, (int)vocab, (int)hidden_dim,
                           n_groups, tiles_per_group, inv_temperature * kLog2e, partial);
    } else {
        // 128-token tiles (4x2 MFMA blocks per wavefront, two workgroups per CU), operands staged through registers
        constexpr int kTokenBlocks = 2;
        const int64_t n_ttiles = (n_tokens + 64 * kTokenBlocks - 1) / (64 * kTokenBlocks);
        MRL_REQUIRE(n_ttiles * n_groups <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: grid too large", fn);
        hipLaunchKernelGGL(lmhead_fwd_kernel<kTokenBlocks>, dim3((unsigned)(n_ttiles * n_groups)), dim3(kThreads), 0, s,
                           (const uint16_t*)hidden, (const uint16_t*)weight, n_tokens, (int)vocab, (int)hidden_dim,
                           n_groups, tiles_per_group, inv_temperature * kLog2e, partial);
    }
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
    MRL_REQUIRE(hidden_dim % BK == 0, MRL_ERR_UNSUPPORTED, "%s: hidden_dim=%lld must be a multiple of %d", fn,         \
                (long long)hidden_dim, BK);                                                                            \
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
