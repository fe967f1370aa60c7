// Row-in-registers vocabulary sweeps for gfx950.
//
// One workgroup of 1024 threads (16 wavefronts, one workgroup per CU) owns one logits row and
// keeps ALL of it in registers: up to 19 16-byte vectors per thread = 311 296 bytes, enough for a
// 152 064-entry bf16 row.  The softmax statistics are taken vector by vector as the data arrives,
// the token's loss gradient follows from them, and dlogits are written from the same registers -
// one HBM read and one HBM write per element for the whole forward + backward of the log-prob /
// policy-loss path.  The requests of a row are issued together (the HBM system serves a row best
// that way) and all accesses are range-checked buffer accesses, so the unrolled bodies contain no
// branch (see mrl_internal.h for why that matters).
//
// fused_sweep_kernel launches one workgroup per row (small batches, or no workspace);
// fused_sweep_persistent_kernel launches one workgroup per CU that takes rows in ticket order and
// requests its next row while it writes the current one.  bwd_chunk_kernel is the split path's backward
// (upstream gradients and the log-sum-exp are inputs, so there is no statistics pass and nothing
// has to stay on chip): a plain stream of one vector per thread.
#include <atomic>

#include "mrl_internal.h"
#include "policy_terms.h"
#include "row_sweep.h"
#include "vocab_common.h"

namespace {

using namespace mrl_vocab;
using namespace mrl_loss;

// Vectors of the next row that are requested early (see fused_sweep_persistent_kernel); build-time
// tuning constants, measured on the 152064-entry bf16 row.  The fused sweep gains 4 % from an early
// burst of 4: its statistics pass then starts without waiting for memory.
#ifndef MRL_SWEEP_HEAD
#define MRL_SWEEP_HEAD 4
#endif
// Workgroup size of the streaming backward (bwd_chunk_kernel): 256 measured best (64: +2 %, 128:
// +14 %, 1024: +8 % in time).
#ifndef MRL_BWD_CHUNK_THREADS
#define MRL_BWD_CHUNK_THREADS 256
#endif

constexpr int kBlock = 1024;
constexpr int kWaves = kBlock / 64;

// Two-level reduction for 16 wavefronts: shuffles inside each wavefront, then the first
// wavefront combines the 16 partials with shuffles again (a serial combine by every thread
// would cost more ALU time than a sixth of the row).
template <bool kEntropy>
__device__ __forceinline__ Stats block_reduce_1024(Stats st, float k, Stats* lds) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        Stats o;
        o.m = __shfl_xor(st.m, off, 64);
        o.s = __shfl_xor(st.s, off, 64);
        o.u = kEntropy ? __shfl_xor(st.u, off, 64) : 0.f;
        st = merge<kEntropy>(st, o, k);
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) lds[wave] = st;
    __syncthreads();
    if (wave == 0) {
        Stats x = lds[lane & (kWaves - 1)];
#pragma unroll
        for (int off = kWaves / 2; off >= 1; off >>= 1) {
            Stats o;
            o.m = __shfl_xor(x.m, off, 64);
            o.s = __shfl_xor(x.s, off, 64);
            o.u = kEntropy ? __shfl_xor(x.u, off, 64) : 0.f;
            x = merge<kEntropy>(x, o, k);
        }
        if (lane == 0) lds[kWaves] = x;
    }
    __syncthreads();
    return lds[kWaves];
}

__device__ __forceinline__ int64_t load_label(const void* labels, int dtype, int64_t r) {
    return dtype == MRL_I32 ? (int64_t) reinterpret_cast<const int32_t*>(labels)[r]
                            : reinterpret_cast<const int64_t*>(labels)[r];
}

struct RowGrad {
    float k;        // inv_t * log2(e)
    float lse2;     // lse * log2(e)
    float c0, c1;   // dlogit = 2^(z k - lse2) * (c0 + c1 z)
    float onehot;   // added at the label
};

template <bool kEntropy>
__device__ __forceinline__ float grad_elem(const RowGrad& g, float z) {
    const float e = fast_exp2(__builtin_fmaf(z, g.k, -g.lse2));
    const float w = kEntropy ? __builtin_fmaf(g.c1, z, g.c0) : g.c0;
    return e * w;
}

// The kernels are instantiated for NV in {4, 8, 12, 16, 19} vectors per thread and the host picks
// the smallest NV that holds the row, so the vectors below kFull are complete for every thread;
// only the last few can reach past the end of the row.
template <int NV>
struct Tail {
    static constexpr int kFull = NV == 19 ? 16 : NV - 4;
};

// Vector q of a row is addressed through a descriptor of its own (the row from byte q * 16 KiB on,
// clamped to empty) with the same per-thread byte offset for every q: the descriptors live in
// scalar registers and cost scalar instructions, where one vector offset per q would cost 19
// vector registers that the row itself needs.
struct RowRef {
    const char* base;   // uniform over the workgroup
    uint32_t bytes;     // 0: nothing is read (loads return zeros) or written
};

__device__ __forceinline__ RowRef row_ref(const void* base, uint32_t bytes) {
    RowRef r = {reinterpret_cast<const char*>(base), bytes};
    return r;
}

__device__ __forceinline__ mrl::rsrc_t vec_rsrc(const RowRef& row, int q) {
    // signed arithmetic on purpose: an unsigned saturating subtraction is selected as a VECTOR
    // instruction, which would make the descriptor non-uniform
    const int skip = q * (kBlock * 16);
    const int rest = (int)row.bytes - skip;
    return mrl::make_rsrc(row.base + skip, (uint32_t)(rest > 0 ? rest : 0));
}

// Keeps the instruction scheduler from moving work of one vector across the work of the next: in
// a fully unrolled, branch-free body it would otherwise unpack many vectors ahead of their use and
// spill the row.
__device__ __forceinline__ void vector_fence() { __builtin_amdgcn_sched_barrier(0); }

__device__ __forceinline__ uint32_t lane_offset() { return (uint32_t)threadIdx.x * 16u; }

// All loads of a row, back to back and without a branch: vectors past the end of the row come back
// as zeros from the range check of the buffer access.
template <int NV>
__device__ __forceinline__ void load_row(u32x4 (&v)[NV], const RowRef& src) {
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        v[q] = mrl::buf_load_nt(vec_rsrc(src, q), lane_offset());
        vector_fence();     // keeps the requests in this order wherever a row is loaded
    }
}

template <int NV>
__device__ __forceinline__ void zero_row(const RowRef& dst) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < NV; ++q) mrl::buf_store_nt(zero, vec_rsrc(dst, q), lane_offset());
}

// Vectors [A, B) of a row: loads, zero stores.
template <int A, int B, int NV>
__device__ __forceinline__ void load_part(u32x4 (&v)[NV], const RowRef& src) {
#pragma unroll
    for (int q = A; q < B; ++q) {
        v[q] = mrl::buf_load_nt(vec_rsrc(src, q), lane_offset());
        vector_fence();
    }
}

template <int A, int B>
__device__ __forceinline__ void zero_part(const RowRef& dst) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = A; q < B; ++q) {
        mrl::buf_store_nt(zero, vec_rsrc(dst, q), lane_offset());
        vector_fence();
    }
}

// Online-softmax statistics of the vectors one thread holds, the careful way: the running maximum is
// brought up to date before every vector, so the exponentials never exceed 1 whatever the logits are
// (infinities and NaN included).  A vector past the end of the row (zeros from the range-checked load)
// is processed like any other and its result discarded, which costs three selects on the few vectors
// that can be affected and keeps the pass free of branches.
template <int DT, int NV, bool kEntropy>
__device__ __forceinline__ Stats thread_stats_careful(const u32x4 (&v)[NV], int n_vec, float k) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    Stats st = {kMaxInit, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        // through an empty asm statement, as in grad_vec: entries that another pass has unpacked
        // must not be kept for this one
        u32x4 x = v[q];
        asm volatile("" : "+v"(x));
        float z[kVec];
        E::unpack(x, z);
        Stats nx = st;
        float vmax = nx.m;
#pragma unroll
        for (int i = 0; i < kVec; ++i) vmax = fmaxf(vmax, z[i]);
        grow_max<kEntropy>(nx, vmax, k);
        const float mk = nx.m * k;
#pragma unroll
        for (int i = 0; i < kVec; ++i) add_one<kEntropy>(nx, z[i], k, mk);
        if (q >= Tail<NV>::kFull) {
            const bool valid = q * kBlock + (int)threadIdx.x < n_vec;
            st.m = valid ? nx.m : st.m;
            st.s = valid ? nx.s : st.s;
            st.u = valid ? nx.u : st.u;
        } else {
            st = nx;
        }
        // pins the running statistics here: without it the scheduler splits the whole unrolled pass
        // into one chain per statistic and parks every exponential in scratch memory in between
        asm volatile("" : "+v"(st.m), "+v"(st.s), "+v"(st.u));
    }
    return st;
}

// A thread's sums may be taken against any reference value in place of the running maximum, as long
// as no exponential overflows: the result (m, s, u) then simply carries that reference as its m, and
// every later merge treats it like a maximum.  An entry of the row is a safe reference from below
// (the largest entry then contributes at least 1), and for ordinary logits it is within a few units
// of the maximum, so nothing comes near the 2^127 an fp32 holds.  Taking the largest entry of the
// thread's first vector saves the maximum over every vector and the rescale that follows it - a
// quarter of the arithmetic of the pass.  If a sum does end up beyond 2^120, infinite or NaN (logits
// that climb by more than 80 above that entry, infinities, NaN), the thread takes its statistics
// once more, carefully.  Which way a thread went depends only on its own entries.
constexpr float kSumLimit = 1.329228e36f;      // 2^120

template <int DT, bool kEntropy>
__device__ __forceinline__ void add_vector(const u32x4& vec, float k, float rk, float& s, float& u) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    float z[kVec];
    E::unpack(vec, z);
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        const float e = fast_exp2(__builtin_fmaf(z[i], k, -rk));
        s += e;
        if (kEntropy) u = __builtin_fmaf(e, z[i], u);
    }
}

template <int DT>
__device__ __forceinline__ float vector_max(const u32x4& vec) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    float z[kVec];
    E::unpack(vec, z);
    float r = z[0];
#pragma unroll
    for (int i = 1; i < kVec; ++i) r = fmaxf(r, z[i]);
    return r;
}

// want_max (uniform over the workgroup): the caller needs the true maximum of the row in m (a label
// outside the vocabulary scores the row maximum), which only the careful pass delivers.
template <int DT, int NV, bool kEntropy>
__device__ __forceinline__ Stats thread_stats(const u32x4 (&v)[NV], int n_vec, float k, bool want_max) {
    Stats st = {kMaxInit, 0.f, 0.f};
    // rows so short that a thread may hold no complete vector at all have nothing to gain
    bool careful = Tail<NV>::kFull == 0 || want_max;
    if (!careful) {
        st.m = vector_max<DT>(v[0]);
        const float rk = st.m * k;
#pragma unroll
        for (int q = 0; q < NV; ++q) {
            float s = st.s, u = st.u;
            add_vector<DT, kEntropy>(v[q], k, rk, s, u);
            if (q >= Tail<NV>::kFull) {
                const bool valid = q * kBlock + (int)threadIdx.x < n_vec;
                st.s = valid ? s : st.s;
                st.u = valid ? u : st.u;
            } else {
                st.s = s;
                st.u = u;
            }
            asm volatile("" : "+v"(st.s), "+v"(st.u));       // as in the careful pass
            // nothing but the two sums links one vector to the next here, so the scheduler would
            // unpack many vectors ahead of their use; keep each vector's work together
            vector_fence();
        }
        careful = !(st.s < kSumLimit);
    }
    if (careful) st = thread_stats_careful<DT, NV, kEntropy>(v, n_vec, k);
    return st;
}

template <int DT, bool kEntropy>
__device__ __forceinline__ u32x4 grad_vec(const u32x4& v, const RowGrad& g) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    // The packed vector is passed through an empty asm statement so that the compiler cannot reuse
    // the unpacked values of the statistics pass: kept alive across both passes they would be a
    // second, four times larger copy of the row, and spill.
    u32x4 x = v;
    asm volatile("" : "+v"(x));
    float z[kVec], d[kVec];
    E::unpack(x, z);
#pragma unroll
    for (int i = 0; i < kVec; ++i) d[i] = grad_elem<kEntropy>(g, z[i]);
    return E::pack(d);
}

// dlogits of vectors [A, B) of the row in registers, stored as they are computed.
template <int DT, bool kEntropy, int A, int B, int NV>
__device__ __forceinline__ void grad_part(const u32x4 (&v)[NV], const RowGrad& g, const RowRef& dst) {
#pragma unroll
    for (int q = A; q < B; ++q) {
        mrl::buf_store_nt(grad_vec<DT, kEntropy>(v[q], g), vec_rsrc(dst, q), lane_offset());
        vector_fence();
    }
}

// The label's entry gets the one-hot term on top of the softmax term.  The thread that has just
// stored the vector holding it re-stores that single entry; for every other thread the byte offset
// is out of range and the hardware drops the store, so there is no branch here either.  Two stores
// of one thread to the same address stay in program order.
template <int DT, bool kEntropy>
__device__ __forceinline__ void store_label_grad(const RowRef& dst, const RowGrad& g, bool y_ok, int64_t y, float z_y) {
    using E = Elem<DT>;
    const bool owner = y_ok && (int)((y / E::kVec) % kBlock) == (int)threadIdx.x;
    const uint32_t off = owner ? (uint32_t)y * (uint32_t)sizeof(typename E::T) : 0x80000000u;
    E::buf_store(mrl::make_rsrc(dst.base, dst.bytes), off, grad_elem<kEntropy>(g, z_y) + g.onehot);
}

struct RowScalars {
    float lp, ent;
    Token t;
    float g_lp, g_h;
};

template <bool kEntropy>
__device__ __forceinline__ RowScalars row_scalars(const Stats& tot, float k, float inv_t, bool y_ok, float z_y,
                                                  const float* __restrict__ ops, int has_old, const Params& p,
                                                  float grad_scale, float m, float& lse) {
    RowScalars s;
    lse = (tot.m * k + fast_log2(tot.s)) * kLn2;
    s.lp = (y_ok ? z_y * inv_t : tot.m * inv_t) - lse;
    s.ent = kEntropy ? lse - (tot.u / tot.s) * inv_t : 0.f;
    s.t = token_terms<true>(s.lp, ops[MRL_OP_OLD], has_old != 0, ops[MRL_OP_REF], ops[MRL_OP_ADV], p);
    const float inv_tok = ops[MRL_OP_INVTOK];
    s.g_lp = grad_scale * m * (ops[MRL_OP_WPG] * s.t.d_pg + p.kl_coef * inv_tok * s.t.d_kl);
    s.g_h = kEntropy ? grad_scale * m * (-p.entropy_coeff * inv_tok) : 0.f;
    return s;
}

template <bool kEntropy>
__device__ __forceinline__ RowGrad row_grad(const RowScalars& s, float k, float inv_t, float lse) {
    RowGrad g;
    g.k = k;
    g.lse2 = lse * kLog2e;
    g.c0 = kEntropy ? inv_t * (-s.g_lp + s.g_h * (lse - s.ent)) : -s.g_lp * inv_t;
    g.c1 = kEntropy ? -s.g_h * inv_t * inv_t : 0.f;
    g.onehot = s.g_lp * inv_t;
    return g;
}

__device__ __forceinline__ void write_row_outputs(int64_t r, const RowScalars& s, float m, float* __restrict__ logp,
                                                  float* __restrict__ entropy, float* __restrict__ row_terms) {
    if (logp) logp[r] = s.lp;
    if (entropy) entropy[r] = s.ent;
    float* out = row_terms + r * S_N;
    out[S_PG] = s.t.pg * m;
    out[S_CLIP] = s.t.clipped * m;
    out[S_PPOKL] = s.t.neg_logr * m;
    out[S_KL] = s.t.kl * m;
    out[S_ENT] = s.ent * m;
    out[S_MASK] = m;
    out[6] = 0.f;
    out[7] = 0.f;
}

__device__ __forceinline__ void write_masked_row_outputs(int64_t r, float* __restrict__ logp,
                                                         float* __restrict__ entropy, float* __restrict__ row_terms) {
    if (logp) logp[r] = 0.f;
    if (entropy) entropy[r] = 0.f;
#pragma unroll
    for (int q = 0; q < S_N; ++q) row_terms[r * S_N + q] = 0.f;
}

template <int DT, int NV, bool kEntropy>
__global__ __launch_bounds__(kBlock) void fused_sweep_kernel(
    const typename Elem<DT>::T* logits, int64_t row_stride, int vocab, const void* __restrict__ labels,
    int labels_dtype, float inv_t, const float* __restrict__ row_ops, int has_old, Params p, float grad_scale,
    const float* __restrict__ grad_scale_dev, typename Elem<DT>::T* dlogits, int64_t d_stride,
    float* __restrict__ logp, float* __restrict__ entropy, float* __restrict__ row_terms) {
    using E = Elem<DT>;
    using T = typename E::T;
    constexpr int kVec = E::kVec;
    __shared__ Stats lds[kWaves + 1];

    if (grad_scale_dev) grad_scale *= *grad_scale_dev;
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    const int n_vec = vocab / kVec;
    const uint32_t row_bytes = (uint32_t)vocab * (uint32_t)sizeof(T);
    const T* row = logits + r * row_stride;
    const RowRef src = row_ref(row, row_bytes);
    const RowRef dst = row_ref(dlogits + r * d_stride, row_bytes);

    const float* ops = row_ops + r * MRL_ROW_OPS;
    const float m = ops[MRL_OP_MASK];
    if (m == 0.f) {                       // not a response token: no gradient, nothing to read
        zero_row<NV>(dst);
        if (tid == 0) write_masked_row_outputs(r, logp, entropy, row_terms);
        return;
    }

    // the whole row: every load is in flight before the first use
    u32x4 v[NV];
    load_row<NV>(v, src);
    const int64_t y = load_label(labels, labels_dtype, r);
    const bool y_ok = (y >= 0) && (y < (int64_t)vocab);
    const float z_y = E::load(row + (y_ok ? y : 0));

    const float k = inv_t * kLog2e;
    const Stats st = thread_stats<DT, NV, kEntropy>(v, n_vec, k, !y_ok);
    const Stats tot = block_reduce_1024<kEntropy>(st, k, lds);

    // row scalars, computed redundantly by every thread (uniform values)
    float lse;
    const RowScalars s = row_scalars<kEntropy>(tot, k, inv_t, y_ok, z_y, ops, has_old, p, grad_scale, m, lse);
    if (tid == 0) write_row_outputs(r, s, m, logp, entropy, row_terms);

    if (s.g_lp == 0.f && s.g_h == 0.f) {
        zero_row<NV>(dst);
    } else {
        const RowGrad g = row_grad<kEntropy>(s, k, inv_t, lse);
#pragma unroll
        for (int q = 0; q < NV; ++q) {
            mrl::buf_store_nt(grad_vec<DT, kEntropy>(v[q], g), vec_rsrc(dst, q), lane_offset());
            vector_fence();
        }
        store_label_grad<DT, kEntropy>(dst, g, y_ok, y, z_y);
    }
}

// ------------------------------------------------------------------------------ row tickets
// The persistent kernel hands out rows through a counter: a workgroup that has finished a row takes
// the next unclaimed one.  With a fixed stride (row r, r + grid, ...) the workgroups drift apart and
// the rows in flight spread over a wide stretch of memory; with tickets the rows in flight are always
// the most recent `grid` consecutive ones, which the HBM system serves about a tenth faster.
// The counter is the first four bytes of the caller's workspace and starts at ZERO: workgroup b
// begins with unit b, and ticket t (the value the fetch-and-add returns) stands for unit
// t + gridDim.x.  So "reset" means "clear": the workspace is zeroed by whoever prepares the sweep
// (the prepare kernel of the loss, or clear_words_kernel below).
__global__ void clear_words_kernel(unsigned long long* p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0ull;
}

// Thread 0 passes its ticket to the workgroup through LDS.  The fences order LDS accesses only and
// the barrier is the bare instruction: __syncthreads() carries a fence over global memory as well,
// which would wait for every outstanding store of the row that was just written.
__device__ __forceinline__ uint32_t broadcast_ticket(uint32_t mine, uint32_t* slot) {
    // every wavefront picks its (unused) result up here, not only the one that passes it on: a
    // result left pending on the other path would make the next fetch-and-add wait for everything
    asm volatile("" : "+v"(mine));
    if (threadIdx.x == 0) *slot = mine;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)*slot);
}

// ------------------------------------------------------------------------------ wide rows
// A row that does not fit the registers of one CU is cut into two halves that two workgroups hold at
// the same time (units 2 r and 2 r + 1 of the ticket order, so the halves of a row are taken by
// workgroups that ask for work one after the other).  Each workgroup publishes a record of its half
// - its statistics and, if the label lies in it, the logit at the label: 16 bytes in the caller's
// workspace, written and read with device-scope atomics only, so that no cache has to be flushed -
// and picks up the other half's before it computes the row's gradient.  A workgroup publishes BEFORE
// it waits, and nothing it does before publishing depends on another workgroup, so waits cannot form
// a cycle; the wait is bounded all the same: when the limit is reached the workgroup reads the other
// half from memory and computes its statistics itself, with the partner's assignment of vectors to
// threads and the same order of operations, so the result is the partner's to the last bit.
//
// In place (dlogits over the logits) the other half may be overwritten by its owner at any time
// AFTER the owner has published: a workgroup waits until its record has reached memory before any of
// its threads stores a gradient.  A workgroup that had to read the other half therefore looks at the
// record once more afterwards: if it is there now, the record is used and what was read is thrown
// away; if it still is not, the owner had not begun to write, and everything read was logits.
struct HalfRecord {
    unsigned long long ms;      // (m, s): never 0, s >= 1 or NaN
    unsigned long long uz;      // (u, logit at the label if it lies in this half, else 1): never 0
};

__device__ __forceinline__ unsigned long long pack2f(float lo, float hi) {
    return (unsigned long long)__float_as_uint(lo) | ((unsigned long long)__float_as_uint(hi) << 32);
}

// Statistics of a stretch of a row streamed from memory by the whole workgroup (the fallback above):
// thread t takes vectors t, t + 1024, ... in this order, as thread_stats does with the vectors a
// thread holds - the same reference, the same sums, the same second attempt - and the reduction is
// the same.  `whole`: every thread has at least one vector and the row maximum is not asked for (what
// makes thread_stats take the short way).
template <int DT, bool kEntropy>
__device__ __forceinline__ Stats stream_stats(const typename Elem<DT>::T* base, int n_vec, float k, bool whole,
                                              Stats* lds) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    const u32x4* vec = reinterpret_cast<const u32x4*>(base);
    Stats st = {kMaxInit, 0.f, 0.f};
    bool careful = !whole;
    if (whole) {
        st.m = vector_max<DT>(__builtin_nontemporal_load(vec + threadIdx.x));
        const float rk = st.m * k;
        for (int idx = threadIdx.x; idx < n_vec; idx += kBlock)
            add_vector<DT, kEntropy>(__builtin_nontemporal_load(vec + idx), k, rk, st.s, st.u);
        careful = !(st.s < kSumLimit);
    }
    if (careful) {
        st = {kMaxInit, 0.f, 0.f};
        for (int idx = threadIdx.x; idx < n_vec; idx += kBlock) {
            float z[kVec];
            E::unpack(__builtin_nontemporal_load(vec + idx), z);
            float vmax = st.m;
#pragma unroll
            for (int i = 0; i < kVec; ++i) vmax = fmaxf(vmax, z[i]);
            grow_max<kEntropy>(st, vmax, k);
            const float mk = st.m * k;
#pragma unroll
            for (int i = 0; i < kVec; ++i) add_one<kEntropy>(st, z[i], k, mk);
        }
    }
    __syncthreads();            // lds may still be read by a slow wavefront of the previous reduction
    return block_reduce_1024<kEntropy>(st, k, lds);
}

// What thread 0 found in the other half's record.
struct Inbox {
    Stats st;
    uint32_t zy_bits;           // fp32 bits of the logit at the label, if the other half holds it
    uint32_t arrived;
};

__device__ __forceinline__ bool read_record(const HalfRecord* rec, unsigned long long& a, unsigned long long& b) {
    if (a == 0) a = __hip_atomic_load(&rec->ms, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (b == 0) b = __hip_atomic_load(&rec->uz, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return a != 0 && b != 0;
}

__device__ __forceinline__ void fill_inbox(Inbox* in, unsigned long long a, unsigned long long b, bool ok) {
    in->st.m = __uint_as_float((uint32_t)a);
    in->st.s = __uint_as_float((uint32_t)(a >> 32));
    in->st.u = __uint_as_float((uint32_t)b);
    in->zy_bits = (uint32_t)(b >> 32);
    in->arrived = ok ? 1u : 0u;
}

// Publishes `mine` (and z_y, the logit at the label, if this half holds it) as half `half` of a row,
// waits (bounded) for the other half and returns the statistics of the whole row, merged in the order
// (first half, second half) by both workgroups; z_y becomes the other half's where that half holds
// the label (zy_there).  rec: the row's two records.  other_base / other_vec: where the other half's
// logits lie; zy_ptr: where the logit at the label lies.
template <int DT, bool kEntropy>
__device__ __forceinline__ Stats exchange_halves(const Stats& mine, int half, HalfRecord* rec, uint32_t spin_limit,
                                                 const typename Elem<DT>::T* other_base, int other_vec, float k,
                                                 bool other_whole, Stats* lds, Inbox* inbox, bool zy_here, bool zy_there,
                                                 const typename Elem<DT>::T* zy_ptr, float& z_y) {
    using E = Elem<DT>;
    if (threadIdx.x == 0) {
        // +0 would make an empty word of (u, z_y) = (0, 0): -0 is the same logit
        const uint32_t zy_word = zy_here ? (__float_as_uint(z_y) == 0u ? 0x80000000u : __float_as_uint(z_y)) : 1u;
        __hip_atomic_store(&rec[half].ms, pack2f(mine.m, mine.s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&rec[half].uz, pack2f(kEntropy ? mine.u : 0.f, __uint_as_float(zy_word)), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        // at most spin_limit polls; with a limit of 0 the record is not looked at here at all, so that
        // the fallback can be exercised deterministically
        unsigned long long a = 0, b = 0;
        bool ok = false;
        for (uint32_t polls = 0; polls < spin_limit && !ok; ++polls) {
            ok = read_record(&rec[half ^ 1], a, b);
            if (!ok) __builtin_amdgcn_s_sleep(4);
        }
        fill_inbox(inbox, a, b, ok);
        // the record has reached memory before any thread of this workgroup stores a gradient
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    Stats other = inbox->st;
    if (inbox->arrived == 0u) {                                  // uniform branch
        other = stream_stats<DT, kEntropy>(other_base, other_vec, k, other_whole, lds);
        if (threadIdx.x == 0) {
            // the logit at the label from the other half, then - once it has arrived - the record again
            uint32_t zy_mem = zy_there ? __float_as_uint(E::load(zy_ptr)) : 0u;
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(zy_mem)::"memory");
            unsigned long long a = 0, b = 0;
            const bool ok = read_record(&rec[half ^ 1], a, b);
            fill_inbox(inbox, a, b, ok);
            if (!ok) inbox->zy_bits = zy_mem;
        }
        __syncthreads();
        if (inbox->arrived != 0u) other = inbox->st;
    }
    if (zy_there) z_y = __uint_as_float(inbox->zy_bits);
    return half == 0 ? merge<kEntropy>(mine, other, k) : merge<kEntropy>(other, mine, k);
}

// Persistent variant of the fused sweep: one workgroup per CU walks rows and, as it turns the
// registers of a row into dlogits, refills them with its NEXT row, so the statistics pass of the next
// row starts on its first vectors while the last are still arriving - the register file never has to
// hold two rows.  The next row is the next unclaimed one (see "row tickets" above), taken while the
// row is being written.
// kWide: the units of work are half rows (see "wide rows" above): unit 2 r is the first
// half_elems entries of row r, unit 2 r + 1 the rest; n_rows then counts units.
template <int DT, int NV, bool kEntropy, bool kWide>
__global__ __launch_bounds__(kBlock) void fused_sweep_persistent_kernel(
    const typename Elem<DT>::T* logits, int64_t row_stride, int vocab, int64_t n_rows,
    const void* __restrict__ labels, int labels_dtype, float inv_t, const float* __restrict__ row_ops, int has_old,
    Params p, float grad_scale, const float* __restrict__ grad_scale_dev, typename Elem<DT>::T* dlogits,
    int64_t d_stride, float* __restrict__ logp, float* __restrict__ entropy, float* __restrict__ row_terms,
    unsigned int* row_ticket, int half_elems, HalfRecord* half_records, uint32_t spin_limit) {
    using E = Elem<DT>;
    using T = typename E::T;
    constexpr int kVec = E::kVec;
    __shared__ Stats lds[kWaves + 1];
    // two slots used in turn: thread 0 may write the ticket of the following row while a slow
    // wavefront has yet to read this one's (one barrier per row separates a slot's reuse)
    __shared__ uint32_t next_row[2];
    __shared__ Inbox inbox;                 // the other half's record (wide rows)

    const int tid = threadIdx.x;
    // bytes and vectors of a unit: the whole row, or its first / second half
    const uint32_t unit_bytes[2] = {(uint32_t)(kWide ? half_elems : vocab) * (uint32_t)sizeof(T),
                                    (uint32_t)(kWide ? vocab - half_elems : 0) * (uint32_t)sizeof(T)};
    const float k = inv_t * kLog2e;
    const int64_t step = gridDim.x;
    if (grad_scale_dev) grad_scale *= *grad_scale_dev;
    // the counter as a 4-byte buffer: only the lane with offset 0 (thread 0) is inside it
    const mrl::rsrc_t ticket = mrl::make_rsrc(row_ticket, 4u);

    // What a workgroup needs to know of the row it fetches next.  A row that is not a response token
    // is never read: its descriptor gets zero bytes, so the (unconditional) loads return zeros
    // without touching memory; the same happens past the last row.
    struct Next {
        int64_t r;              // >= n_rows: none
        int64_t y;
        const T* zy_ptr;
        RowRef row;
    };
    int64_t r = blockIdx.x;
    auto plan = [&](int64_t r2) {
        Next n;
        n.r = r2;
        const bool has = r2 < n_rows;
        const int64_t un = has ? r2 : r;                    // unit
        const int64_t rn = kWide ? (un >> 1) : un;          // row
        const int hn = kWide ? (int)(un & 1) : 0;
        const bool live = has && (row_ops[rn * MRL_ROW_OPS + MRL_OP_MASK] != 0.f);
        const T* nrow = logits + rn * row_stride;
        n.row = row_ref(nrow + (hn ? half_elems : 0), live ? unit_bytes[hn] : 0u);
        n.y = load_label(labels, labels_dtype, rn);
        n.zy_ptr = nrow + ((n.y >= 0 && n.y < (int64_t)vocab) ? n.y : 0);
        return n;
    };

    // The next row is requested in two bursts: its first H vectors once the first H vectors of the
    // current row have been written (they arrive while the rest of the gradient is computed, so the
    // statistics pass of the next row starts without waiting for memory), the others behind the last
    // store.  A larger H costs bandwidth: a row's requests are served best when they are issued
    // together.  The logit at the label comes last; it is not needed before the row is reduced.
    constexpr int H = NV >= 8 ? MRL_SWEEP_HEAD : NV / 2;
    u32x4 v[NV];
    int64_t y = 0;
    uint32_t zy_bits = 0;                   // the logit at the label as loaded; converted where it is used
    if (r < n_rows) {
        const Next first = plan(r);
        y = first.y;
        // the same sequence of operations as one turn of the loop leaves behind (with stores that
        // write nothing), so that the number of operations outstanding at the top of the loop - which
        // the compiler has to assume when it places the waits of the statistics pass - is the same
        // on every path into it
        const RowRef none = row_ref(dlogits, 0u);
        mrl::buf_atomic_add_u32(mrl::make_rsrc(dlogits, 0u), lane_offset(), 0u);
        zero_part<0, H>(none);
        load_part<0, H>(v, first.row);
        zero_part<H, NV>(none);
        mrl::buf_store_b32(0u, mrl::make_rsrc(dlogits, 0u), 0u);
        load_part<H, NV>(v, first.row);
        zy_bits = E::load_bits(first.zy_ptr);
    }
    int parity = 0;
    while (r < n_rows) {
        const int64_t row = kWide ? (r >> 1) : r;
        const int half = kWide ? (int)(r & 1) : 0;
        const int my_first = half ? half_elems : 0;         // first entry of this unit within the row
        const int n_vec = (int)(unit_bytes[half] / 16u);
        const RowRef dst = row_ref(dlogits + row * d_stride + my_first, unit_bytes[half]);
        const float* ops = row_ops + row * MRL_ROW_OPS;
        const float m = ops[MRL_OP_MASK];
        const bool y_ok = (y >= 0) && (y < (int64_t)vocab);
        // the label's entry gets its one-hot term from the unit that holds it
        const int64_t y_here = y - my_first;
        const bool y_mine = y_ok && (!kWide || (y_here >= 0 && y_here < (int64_t)(unit_bytes[half] / sizeof(T))));
        Next nx;
        uint32_t zy_next = 0;

        bool wrote = false;                 // dlogits of row r written and the next row requested
        if (m != 0.f) {
            float z_y = E::from_bits(zy_bits);
            const Stats st = thread_stats<DT, NV, kEntropy>(v, n_vec, k, !y_ok);
            Stats tot = block_reduce_1024<kEntropy>(st, k, lds);
            if (kWide) {
                // the logit at the label as this unit loaded it counts only if the label lies in this
                // half: the other half may already hold gradients when dlogits overwrite the logits
                const int other_first = half ? 0 : half_elems;
                const T* whole = logits + row * row_stride;
                tot = exchange_halves<DT, kEntropy>(tot, half, half_records + row * 2, spin_limit, whole + other_first,
                                                    (int)(unit_bytes[half ^ 1] / 16u), k, Tail<NV>::kFull != 0 && y_ok, lds, &inbox, y_mine,
                                                    y_ok && !y_mine, whole + (y_ok ? y : 0), z_y);
            }
            float lse;
            const RowScalars s = row_scalars<kEntropy>(tot, k, inv_t, y_ok, z_y, ops, has_old, p, grad_scale, m, lse);
            if (tid == 0 && half == 0) write_row_outputs(row, s, m, logp, entropy, row_terms);
            if (s.g_lp != 0.f || s.g_h != 0.f) {
                const RowGrad g = row_grad<kEntropy>(s, k, inv_t, lse);
                // the ticket is asked for ahead of the stores and picked up behind the first H of
                // them: it is older than every store, so waiting for it does not wait for them
                const uint32_t mine = mrl::buf_atomic_add_u32(ticket, lane_offset(), 1u);
                grad_part<DT, kEntropy, 0, H>(v, g, dst);
                nx = plan((int64_t)broadcast_ticket(mine, &next_row[parity]) + step);
                load_part<0, H>(v, nx.row);
                grad_part<DT, kEntropy, H, NV>(v, g, dst);
                store_label_grad<DT, kEntropy>(dst, g, y_mine, y_here, z_y);
                load_part<H, NV>(v, nx.row);
                zy_next = E::load_bits(nx.zy_ptr);
                wrote = true;
            }
        } else if (tid == 0 && half == 0) {
            write_masked_row_outputs(row, logp, entropy, row_terms);
        }
        if (!wrote) {                       // no gradient for this row: zeros, same order of operations
            const uint32_t mine = mrl::buf_atomic_add_u32(ticket, lane_offset(), 1u);
            zero_part<0, H>(dst);
            nx = plan((int64_t)broadcast_ticket(mine, &next_row[parity]) + step);
            load_part<0, H>(v, nx.row);
            zero_part<H, NV>(dst);
            mrl::buf_store_b32(0u, mrl::make_rsrc(dlogits, 0u), 0u);
            load_part<H, NV>(v, nx.row);
            zy_next = E::load_bits(nx.zy_ptr);
        }
        y = nx.y;
        zy_bits = zy_next;
        r = nx.r;
        parity ^= 1;
    }
}

// Backward of the split path as a plain stream: one 16-byte vector per thread, small workgroups that
// retire at once.  The backward needs no whole-row state (the log-sum-exp is an input), so nothing
// has to stay on chip, and this is the access pattern the HBM system serves best: the requests in
// flight always cover one compact, advancing stretch of the logits and of dlogits.  Grid: x walks
// the row in chunks of kThreads vectors, (y, z) number the rows; x is dispatched fastest, so the
// workgroups in flight are neighbours in memory.  A row with no incoming gradient is zero-filled
// without being read; a vector past the end of the row is neither read nor written (range checks).
constexpr int kChunkRowsY = 32768;      // rows per grid.y; grid.z carries the rest

template <int DT, bool kEntropy, int kThreads>
__global__ __launch_bounds__(kThreads) void bwd_chunk_kernel(
    const typename Elem<DT>::T* logits, int64_t row_stride, int vocab, int64_t n_rows,
    const void* __restrict__ labels, int labels_dtype, float inv_t, const float* __restrict__ lse_in,
    const float* __restrict__ ent_in, const float* __restrict__ g_logp, const float* __restrict__ g_entropy,
    typename Elem<DT>::T* dlogits, int64_t d_stride) {
    using E = Elem<DT>;
    using T = typename E::T;
    constexpr int kVec = E::kVec;
    const int64_t r = (int64_t)blockIdx.z * kChunkRowsY + blockIdx.y;
    if (r >= n_rows) return;
    const uint32_t row_bytes = (uint32_t)vocab * (uint32_t)sizeof(T);
    const uint32_t first = blockIdx.x * (uint32_t)kThreads;           // first vector of this workgroup
    const uint32_t off = (first + threadIdx.x) * 16u;
    const mrl::rsrc_t dst = mrl::make_rsrc(dlogits + r * d_stride, row_bytes);
    const float g_lp = g_logp ? g_logp[r] : 0.f;
    const float g_h = (kEntropy && g_entropy) ? g_entropy[r] : 0.f;
    if (g_lp == 0.f && g_h == 0.f) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
        mrl::buf_store_nt(zero, dst, off);
        return;
    }
    const u32x4 v = mrl::buf_load_nt(mrl::make_rsrc(logits + r * row_stride, row_bytes), off);
    const float lse = lse_in[r];
    RowGrad g;
    g.k = inv_t * kLog2e;
    g.lse2 = lse * kLog2e;
    g.c0 = kEntropy ? inv_t * (-g_lp + g_h * (lse - ent_in[r])) : -g_lp * inv_t;
    g.c1 = kEntropy ? -g_h * inv_t * inv_t : 0.f;
    g.onehot = g_lp * inv_t;
    mrl::buf_store_nt(grad_vec<DT, kEntropy>(v, g), dst, off);
    // the entry at the label: written once more, with the one-hot term, by the thread that holds it
    // (stores of one thread to the same address stay in program order)
    const int64_t y = load_label(labels, labels_dtype, r);
    if (y >= 0 && y < (int64_t)vocab) {
        const uint32_t yv = (uint32_t)y / (uint32_t)kVec;
        if (yv >= first && yv < first + (uint32_t)kThreads) {        // uniform over the workgroup
            float z[kVec];
            E::unpack(v, z);
            const int e = (int)((uint32_t)y % (uint32_t)kVec);
            float z_y = z[0];
#pragma unroll
            for (int i = 1; i < kVec; ++i) z_y = (e == i) ? z[i] : z_y;
            const uint32_t y_off = (yv - first == threadIdx.x) ? (uint32_t)y * (uint32_t)sizeof(T) : 0x80000000u;
            E::buf_store(dst, y_off, grad_elem<kEntropy>(g, z_y) + g.onehot);
        }
    }
}

// Conditional in-place rescale: multiplies every row by upstream/applied unless that ratio is 1
// (then every workgroup exits at once; the grid is kept small so that this costs microseconds).
template <int DT>
__global__ __launch_bounds__(256) void scale_rows_kernel(typename Elem<DT>::T* x, int64_t row_stride, int vocab,
                                                         int64_t n_rows, const float* __restrict__ upstream,
                                                         const float* __restrict__ applied) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    const float ratio = *upstream / *applied;
    if (ratio == 1.f) return;
    const int n_vec = vocab / kVec;
    for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) {
        u32x4* vec = reinterpret_cast<u32x4*>(x + r * row_stride);
        for (int idx = threadIdx.x; idx < n_vec; idx += 256) {
            float z[kVec];
            E::unpack(vec[idx], z);
#pragma unroll
            for (int i = 0; i < kVec; ++i) z[i] *= ratio;
            vec[idx] = E::pack(z);
        }
    }
}

// One backward of one buffer in a single launch: the conditional rescale above, then the book-keeping
// of grad_scale_note_kernel.  When nothing is to be moved (the ratio is 1, i.e. the new scale equals
// the old one) workgroup 0 does the book-keeping at once - what it stores over the scale is the value
// every other workgroup reads there anyway - and the others leave.  Otherwise the workgroup that
// finishes last does it (a counter next to the scale tells; every workgroup has read the scale before
// it counts itself, so the last one may overwrite it).
template <int DT>
__global__ __launch_bounds__(256) void scale_rows_note_kernel(typename Elem<DT>::T* x, int64_t row_stride, int vocab,
                                                              int64_t n_rows, const float* __restrict__ upstream,
                                                              float* applied, float* learned, uint32_t* rescales) {
    using E = Elem<DT>;
    constexpr int kVec = E::kVec;
    const float u = *upstream;
    const float was = applied[0];
    const float ratio = u / was;
    if (ratio == 1.f) {
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            applied[0] = u;
            if (learned && u != 0.f && __builtin_isfinite(u)) *learned = u;
        }
        return;
    }
    const int n_vec = vocab / kVec;
    for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) {
        u32x4* vec = reinterpret_cast<u32x4*>(x + r * row_stride);
        for (int idx = threadIdx.x; idx < n_vec; idx += 256) {
            float z[kVec];
            E::unpack(vec[idx], z);
#pragma unroll
            for (int i = 0; i < kVec; ++i) z[i] *= ratio;
            vec[idx] = E::pack(z);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t* done = reinterpret_cast<uint32_t*>(applied) + 1;
        const uint32_t before = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before == gridDim.x - 1) {
            if (rescales) *rescales += 1u;
            applied[0] = u;
            __hip_atomic_store(done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (learned && u != 0.f && __builtin_isfinite(u)) *learned = u;
        }
    }
}

// Book-keeping behind one or more scale_rows_kernel launches: the buffers now carry `upstream`.
__global__ void grad_scale_note_kernel(const float* __restrict__ upstream, float* applied, float* learned,
                                       uint32_t* rescales) {
    if (threadIdx.x != 0) return;
    const float u = *upstream;
    const float was = *applied;
    if (rescales && u / was != 1.f) *rescales += 1u;
    *applied = u;
    // a scale that the next sweep can start from: finite and non-zero
    if (learned && u != 0.f && __builtin_isfinite(u)) *learned = u;
}

// ----------------------------------------------------------------------------- host dispatch
constexpr int kMaxVecPerThread = 19;

inline int pick_nv(int64_t n_vec) {
    const int64_t need = (n_vec + kBlock - 1) / kBlock;
    const int sizes[] = {4, 8, 12, 16, 19};
    for (int s : sizes)
        if (need <= s) return s;
    return 0;
}

// Number of CUs of the current device (one persistent workgroup each); 0 if the query fails.
int cu_count() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return n;
}

// Upper bound of the polls a workgroup spends waiting for the other half of a wide row before it
// computes that half's statistics itself (mrl_set_wide_spin_limit; 0: never look, always compute).
constexpr uint32_t kDefaultSpinLimit = 1u << 18;
std::atomic<uint32_t> g_wide_spin_limit{kDefaultSpinLimit};

constexpr int64_t kWorkspaceHeader = 16;    // the row counter, padded to the alignment of the records

// Rows that go to the persistent workgroups; fewer get one workgroup each.
inline bool wants_persistent(int64_t n_rows, int cus) { return cus > 0 && n_rows > 2 * (int64_t)cus; }

template <int DT, int NV>
int launch_fused(const mrl::FusedArgs& a) {
    using T = typename Elem<DT>::T;
    const dim3 block(kBlock);
    const Params p = {a.clip_lo, a.clip_hi, a.kl_coef, a.entropy_coeff, 1.f, a.kl_penalty, 0};
    unsigned int* counter = reinterpret_cast<unsigned int*>(a.workspace);
    const int cus = cu_count();
    const bool persistent = a.wide || (counter != nullptr && wants_persistent(a.n_rows, cus));
    if (persistent) {
        if (cus < 2) return mrl::fail(MRL_ERR_LAUNCH, "mrl_fused_logprob_loss: cannot query the device");
        // half rows: an even number of workgroups, so that the halves of a row start side by side
        const int64_t units = a.wide ? 2 * a.n_rows : a.n_rows;
        const int64_t want = a.wide ? (cus & ~1) : cus;
        const dim3 pgrid((unsigned)(want < units ? want : units));
        HalfRecord* rec = reinterpret_cast<HalfRecord*>(reinterpret_cast<char*>(a.workspace) + kWorkspaceHeader);
        if (!a.workspace_cleared) {
            const int64_t words = (kWorkspaceHeader + (a.wide ? a.n_rows * 2 * (int64_t)sizeof(HalfRecord) : 0)) / 8;
            hipLaunchKernelGGL(clear_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, a.stream,
                               reinterpret_cast<unsigned long long*>(a.workspace), words);
        }
        const uint32_t spin = g_wide_spin_limit.load(std::memory_order_relaxed);
#define MRL_FUSEDP_LAUNCH(ENT, WIDE)                                                                               \
    hipLaunchKernelGGL((fused_sweep_persistent_kernel<DT, NV, ENT, WIDE>), pgrid, block, 0, a.stream,               \
                       (const T*)a.logits, a.row_stride, (int)a.vocab, units, a.labels, a.labels_dtype, a.inv_t,    \
                       a.row_ops, a.has_old, p, a.grad_scale, a.grad_scale_dev, (T*)a.dlogits, a.d_stride, a.logp,  \
                       a.entropy, a.row_terms, counter, (int)a.half_elems, rec, spin)
        if (a.wide && a.with_entropy) MRL_FUSEDP_LAUNCH(true, true);
        else if (a.wide) MRL_FUSEDP_LAUNCH(false, true);
        else if (a.with_entropy) MRL_FUSEDP_LAUNCH(true, false);
        else MRL_FUSEDP_LAUNCH(false, false);
#undef MRL_FUSEDP_LAUNCH
        return mrl::check_launch("mrl_fused_logprob_loss");
    }
    const dim3 grid((unsigned)a.n_rows);
#define MRL_FUSED_LAUNCH(ENT)                                                                                  \
    hipLaunchKernelGGL((fused_sweep_kernel<DT, NV, ENT>), grid, block, 0, a.stream, (const T*)a.logits,        \
                       a.row_stride, (int)a.vocab, a.labels, a.labels_dtype, a.inv_t, a.row_ops, a.has_old, p, \
                       a.grad_scale, a.grad_scale_dev, (T*)a.dlogits, a.d_stride, a.logp, a.entropy, a.row_terms)
    if (a.with_entropy) MRL_FUSED_LAUNCH(true);
    else MRL_FUSED_LAUNCH(false);
#undef MRL_FUSED_LAUNCH
    return mrl::check_launch("mrl_fused_logprob_loss");
}

#define MRL_NV_SWITCH(FUNC, DT, nv, a)      \
    switch (nv) {                           \
        case 4: return FUNC<DT, 4>(a);      \
        case 8: return FUNC<DT, 8>(a);      \
        case 12: return FUNC<DT, 12>(a);    \
        case 16: return FUNC<DT, 16>(a);    \
        default: return FUNC<DT, 19>(a);    \
    }

template <int DT>
int fused_by_nv(int nv, const mrl::FusedArgs& a) { MRL_NV_SWITCH(launch_fused, DT, nv, a) }

}  // namespace

namespace mrl {

template <int DT, int kThreads>
static int launch_bwd_chunk_n(const BwdArgs& a) {
    using T = typename Elem<DT>::T;
    const int64_t n_vec = a.vocab / Elem<DT>::kVec;
    const int64_t gy = a.n_rows < kChunkRowsY ? a.n_rows : kChunkRowsY;
    const int64_t gz = (a.n_rows + kChunkRowsY - 1) / kChunkRowsY;
    const dim3 grid((unsigned)((n_vec + kThreads - 1) / kThreads), (unsigned)gy, (unsigned)gz);
#define MRL_BWDC_LAUNCH(ENT)                                                                                     \
    hipLaunchKernelGGL((bwd_chunk_kernel<DT, ENT, kThreads>), grid, dim3(kThreads), 0, a.stream, (const T*)a.logits, \
                       a.row_stride, (int)a.vocab, a.n_rows, a.labels, a.labels_dtype, a.inv_t, a.lse, a.entropy,  \
                       a.g_logp, a.g_entropy, (T*)a.dlogits, a.d_stride)
    if (a.g_entropy != nullptr) MRL_BWDC_LAUNCH(true);
    else MRL_BWDC_LAUNCH(false);
#undef MRL_BWDC_LAUNCH
    return check_launch("mrl_vocab_logprob_bwd");
}

// Workgroups of half the size when that leaves at least 3 % fewer lanes idle in a row's last
// chunk (a 38 KiB row is 9.3 chunks of 256 vectors: 2.30 ms against 2.19 ms for 171 174 such rows).
template <int DT>
static int launch_bwd_chunk(const BwdArgs& a) {
    constexpr int kFull = MRL_BWD_CHUNK_THREADS, kHalf = MRL_BWD_CHUNK_THREADS / 2;
    const int64_t n_vec = a.vocab / Elem<DT>::kVec;
    const int64_t idle_full = (n_vec + kFull - 1) / kFull * kFull - n_vec;
    const int64_t idle_half = (n_vec + kHalf - 1) / kHalf * kHalf - n_vec;
    if ((idle_full - idle_half) * 100 >= 3 * n_vec) return launch_bwd_chunk_n<DT, kHalf>(a);
    return launch_bwd_chunk_n<DT, kFull>(a);
}

int launch_bwd_chunks(const BwdArgs& a) {
    switch (a.dtype) {
        case MRL_F32: return launch_bwd_chunk<MRL_F32>(a);
        case MRL_BF16: return launch_bwd_chunk<MRL_BF16>(a);
        default: return launch_bwd_chunk<MRL_F16>(a);
    }
}

bool bwd_chunks_supported(int dtype, int64_t vocab, const void* in, int64_t in_stride, const void* out,
                          int64_t out_stride, int64_t n_rows) {
    const int eb = float_dtype_bytes(dtype);
    if (eb == 0) return false;
    const int64_t per_vec = 16 / eb;
    // rows of whole vectors, at least 16 KiB (below that the loop kernel with one workgroup per row has
    // less to launch), below 2 GiB (32-bit range checks), and a grid.z within its limit
    if (vocab % per_vec != 0 || vocab * eb < 16 * 1024 || vocab * eb >= (1LL << 31)) return false;
    if (n_rows > (int64_t)kChunkRowsY * 65535) return false;
    if (!aligned(in, 16) || !aligned(out, 16)) return false;
    if (n_rows > 1 && ((in_stride * eb) % 16 != 0 || (out_stride * eb) % 16 != 0)) return false;
    return true;
}

bool row_sweep_supported(int dtype, int64_t vocab, const void* in, int64_t in_stride, const void* out,
                         int64_t out_stride, int64_t n_rows) {
    const int eb = float_dtype_bytes(dtype);
    if (eb == 0) return false;
    const int64_t per_vec = 16 / eb;
    if (vocab % per_vec != 0) return false;
    const int64_t n_vec = vocab / per_vec;
    // wider rows: two halves held by two workgroups (see "wide rows")
    if (pick_nv(n_vec) == 0 && pick_nv((n_vec + 1) / 2) == 0) return false;
    if (!aligned(in, 16) || !aligned(out, 16)) return false;
    if (n_rows > 1 && ((in_stride * eb) % 16 != 0 || (out_stride * eb) % 16 != 0)) return false;
    return true;
}

}  // namespace mrl

extern "C" int64_t mrl_fused_max_vocab(int logits_dtype) {
    const int eb = mrl::float_dtype_bytes(logits_dtype);
    if (eb == 0) return 0;
    return 2 * (int64_t)kMaxVecPerThread * kBlock * (16 / eb);      // two workgroups hold a wide row
}

extern "C" int64_t mrl_fused_workspace_bytes(int logits_dtype, int64_t n_rows, int64_t vocab) {
    const int eb = mrl::float_dtype_bytes(logits_dtype);
    if (eb == 0 || n_rows < 0 || vocab <= 0 || vocab % (16 / eb) != 0) return 0;
    const int64_t n_vec = vocab / (16 / eb);
    if (pick_nv(n_vec) != 0) return kWorkspaceHeader;
    if (pick_nv((n_vec + 1) / 2) == 0) return 0;
    return kWorkspaceHeader + n_rows * (int64_t)sizeof(HalfRecord) * 2;
}

extern "C" int64_t mrl_set_wide_spin_limit(int64_t polls) {
    const uint32_t next = polls < 0 ? kDefaultSpinLimit : (uint32_t)(polls > 0xffffffffLL ? 0xffffffffLL : polls);
    return (int64_t)g_wide_spin_limit.exchange(next, std::memory_order_relaxed);
}

extern "C" int mrl_fused_logprob_loss(const void* logits, int logits_dtype, int64_t n_rows, int64_t vocab,
                                      int64_t row_stride, const void* labels, int labels_dtype,
                                      float inv_temperature, const float* row_ops, int has_old, float clip_lo,
                                      float clip_hi, int kl_penalty, float kl_coef, float entropy_coeff,
                                      float grad_scale, const float* grad_scale_dev, void* dlogits,
                                      int64_t dlogits_row_stride, float* logp, float* entropy, float* row_terms,
                                      void* workspace, int64_t workspace_bytes, int workspace_cleared,
                                      void* stream) {
    const char* fn = "mrl_fused_logprob_loss";
    MRL_REQUIRE(n_rows >= 0 && vocab > 0 && n_rows <= 0x3fffffffLL, MRL_ERR_INVALID_ARG, "%s: n_rows=%lld vocab=%lld",
                fn, (long long)n_rows, (long long)vocab);
    const int eb = mrl::float_dtype_bytes(logits_dtype);
    MRL_REQUIRE(eb != 0, MRL_ERR_UNSUPPORTED, "%s: logits dtype %d (want F32, BF16 or F16)", fn, logits_dtype);
    MRL_REQUIRE(mrl::int_dtype_bytes(labels_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: labels dtype %d (want I32 or I64)",
                fn, labels_dtype);
    MRL_REQUIRE(row_stride >= vocab && dlogits_row_stride >= vocab, MRL_ERR_INVALID_ARG, "%s: row stride below vocab",
                fn);
    MRL_REQUIRE(kl_penalty >= MRL_KL_NONE && kl_penalty <= MRL_KL_LOW_VAR, MRL_ERR_INVALID_ARG, "%s: kl_penalty=%d", fn,
                kl_penalty);
    MRL_REQUIRE(inv_temperature > 0.f && inv_temperature < 1.0e6f, MRL_ERR_INVALID_ARG,
                "%s: inv_temperature=%g must be in (0, 1e6)", fn, (double)inv_temperature);
    if (n_rows == 0) return MRL_OK;
    MRL_REQUIRE(logits && labels && row_ops && dlogits && row_terms, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(workspace, 16) && mrl::aligned(grad_scale_dev, 4), MRL_ERR_MISALIGNED,
                "%s: workspace must be 16-byte and grad_scale_dev 4-byte aligned", fn);
    MRL_REQUIRE(mrl::row_sweep_supported(logits_dtype, vocab, logits, row_stride, dlogits, dlogits_row_stride, n_rows),
                MRL_ERR_UNSUPPORTED,
                "%s: needs 16-byte aligned rows, vocab %% %d == 0 and vocab <= %lld for this dtype (got vocab=%lld)", fn,
                16 / eb, (long long)mrl_fused_max_vocab(logits_dtype), (long long)vocab);
    if (dlogits != logits) {
        const char* x = (const char*)logits;
        const char* y = (const char*)dlogits;
        const int64_t xb = ((n_rows - 1) * row_stride + vocab) * eb, yb = ((n_rows - 1) * dlogits_row_stride + vocab) * eb;
        MRL_REQUIRE(x + xb <= y || y + yb <= x, MRL_ERR_INVALID_ARG, "%s: dlogits partially overlaps logits", fn);
    } else {
        MRL_REQUIRE(dlogits_row_stride == row_stride, MRL_ERR_INVALID_ARG, "%s: in-place needs identical strides", fn);
    }
    mrl::FusedArgs a;
    a.logits = logits; a.dtype = logits_dtype; a.n_rows = n_rows; a.vocab = vocab; a.row_stride = row_stride;
    a.labels = labels; a.labels_dtype = labels_dtype; a.inv_t = inv_temperature; a.row_ops = row_ops;
    a.has_old = has_old; a.clip_lo = clip_lo; a.clip_hi = clip_hi; a.kl_penalty = kl_penalty; a.kl_coef = kl_coef;
    a.entropy_coeff = entropy_coeff; a.grad_scale = grad_scale; a.grad_scale_dev = grad_scale_dev;
    a.workspace = workspace; a.workspace_cleared = workspace_cleared != 0; a.dlogits = dlogits; a.d_stride = dlogits_row_stride;
    a.logp = logp; a.entropy = entropy; a.row_terms = row_terms; a.with_entropy = (entropy != nullptr);
    a.stream = mrl::as_stream(stream);
    const int64_t n_vec = vocab / (16 / eb);
    int nv = pick_nv(n_vec);
    a.wide = (nv == 0);
    a.half_elems = 0;
    if (a.wide) {
        a.half_elems = (n_vec + 1) / 2 * (16 / eb);
        nv = pick_nv((n_vec + 1) / 2);
    }
    if (workspace != nullptr || a.wide) {
        const int64_t need = a.wide ? mrl_fused_workspace_bytes(logits_dtype, n_rows, vocab) : kWorkspaceHeader;
        MRL_REQUIRE(workspace != nullptr && workspace_bytes >= need, MRL_ERR_INVALID_ARG,
                    "%s: workspace of %lld bytes, need %lld (rows of this width are cut in two halves that exchange "
                    "their statistics through it)", fn, (long long)(workspace ? workspace_bytes : 0), (long long)need);
    }
    switch (logits_dtype) {
        case MRL_F32: return fused_by_nv<MRL_F32>(nv, a);
        case MRL_BF16: return fused_by_nv<MRL_BF16>(nv, a);
        default: return fused_by_nv<MRL_F16>(nv, a);
    }
}

extern "C" int mrl_scale_rows(void* x, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                              const float* upstream, const float* applied, void* stream) {
    const char* fn = "mrl_scale_rows";
    const int eb = mrl::float_dtype_bytes(dtype);
    MRL_REQUIRE(eb != 0, MRL_ERR_UNSUPPORTED, "%s: dtype %d (want F32, BF16 or F16)", fn, dtype);
    MRL_REQUIRE(n_rows >= 0 && n_rows <= 0x7fffffffLL && vocab > 0 && row_stride >= vocab, MRL_ERR_INVALID_ARG,
                "%s: n_rows=%lld vocab=%lld row_stride=%lld", fn, (long long)n_rows, (long long)vocab,
                (long long)row_stride);
    if (n_rows == 0) return MRL_OK;
    MRL_REQUIRE(x && upstream && applied, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(upstream, 4) && mrl::aligned(applied, 4), MRL_ERR_MISALIGNED,
                "%s: upstream and applied must be 4-byte aligned", fn);
    MRL_REQUIRE(vocab % (16 / eb) == 0 && mrl::aligned(x, 16) && (n_rows == 1 || (row_stride * eb) % 16 == 0),
                MRL_ERR_UNSUPPORTED, "%s: needs 16-byte aligned rows", fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid((unsigned)(n_rows < 4096 ? n_rows : 4096)), block(256);
    switch (dtype) {
        case MRL_F32:
            hipLaunchKernelGGL(scale_rows_kernel<MRL_F32>, grid, block, 0, s, (float*)x, row_stride, (int)vocab,
                               n_rows, upstream, applied);
            break;
        case MRL_BF16:
            hipLaunchKernelGGL(scale_rows_kernel<MRL_BF16>, grid, block, 0, s, (uint16_t*)x, row_stride, (int)vocab,
                               n_rows, upstream, applied);
            break;
        default:
            hipLaunchKernelGGL(scale_rows_kernel<MRL_F16>, grid, block, 0, s, (uint16_t*)x, row_stride, (int)vocab,
                               n_rows, upstream, applied);
            break;
    }
    return mrl::check_launch(fn);
}

extern "C" int mrl_grad_scale_note(const float* upstream, float* applied, float* learned, uint32_t* rescales,
                                   void* stream) {
    const char* fn = "mrl_grad_scale_note";
    MRL_REQUIRE(upstream && applied, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(upstream, 4) && mrl::aligned(applied, 4) && mrl::aligned(learned, 4) &&
                    mrl::aligned(rescales, 4),
                MRL_ERR_MISALIGNED, "%s: pointers must be 4-byte aligned", fn);
    hipLaunchKernelGGL(grad_scale_note_kernel, dim3(1), dim3(64), 0, mrl::as_stream(stream), upstream, applied, learned,
                       rescales);
    return mrl::check_launch(fn);
}

extern "C" int mrl_scale_rows_note(void* x, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                   const float* upstream, float* applied, float* learned, uint32_t* rescales,
                                   void* stream) {
    const char* fn = "mrl_scale_rows_note";
    const int eb = mrl::float_dtype_bytes(dtype);
    MRL_REQUIRE(eb != 0, MRL_ERR_UNSUPPORTED, "%s: dtype %d (want F32, BF16 or F16)", fn, dtype);
    MRL_REQUIRE(n_rows > 0 && n_rows <= 0x7fffffffLL && vocab > 0 && row_stride >= vocab, MRL_ERR_INVALID_ARG,
                "%s: n_rows=%lld vocab=%lld row_stride=%lld", fn, (long long)n_rows, (long long)vocab,
                (long long)row_stride);
    MRL_REQUIRE(x && upstream && applied, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(upstream, 4) && mrl::aligned(applied, 8) && mrl::aligned(learned, 4) &&
                    mrl::aligned(rescales, 4),
                MRL_ERR_MISALIGNED, "%s: applied must be 8-byte, the other scalars 4-byte aligned", fn);
    MRL_REQUIRE(vocab % (16 / eb) == 0 && mrl::aligned(x, 16) && (n_rows == 1 || (row_stride * eb) % 16 == 0),
                MRL_ERR_UNSUPPORTED, "%s: needs 16-byte aligned rows", fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid((unsigned)(n_rows < 2048 ? n_rows : 2048)), block(256);
    switch (dtype) {
        case MRL_F32:
            hipLaunchKernelGGL(scale_rows_note_kernel<MRL_F32>, grid, block, 0, s, (float*)x, row_stride, (int)vocab,
                               n_rows, upstream, applied, learned, rescales);
            break;
        case MRL_BF16:
            hipLaunchKernelGGL(scale_rows_note_kernel<MRL_BF16>, grid, block, 0, s, (uint16_t*)x, row_stride,
                               (int)vocab, n_rows, upstream, applied, learned, rescales);
            break;
        default:
            hipLaunchKernelGGL(scale_rows_note_kernel<MRL_F16>, grid, block, 0, s, (uint16_t*)x, row_stride,
                               (int)vocab, n_rows, upstream, applied, learned, rescales);
            break;
    }
    return mrl::check_launch(fn);
}
