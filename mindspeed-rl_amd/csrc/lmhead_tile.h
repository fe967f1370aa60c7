// The tile loop of the lm_head matrix products on the bf16 matrix cores of gfx950, shared by the plain
// products (lmhead_gemm.hip) and by the fused lm_head + log-prob forward (lmhead.hip), which differ in
// what they do with a finished 256 x 256 tile of fp32 results.
//
//     tile[n][m] = sum_k A[m][k] * B[n][k]
//
// A workgroup of 256 threads (2 x 2 wavefronts, one per SIMD, wavefront tile 128 x 128 = 8 x 8 blocks of
// v_mfma_f32_16x16x32_bf16 in 256 accumulator registers) walks a sequence of tiles; operands go from
// global memory straight into LDS (buffer_load ... lds) into two 64 KiB stages of 64 k each,
// XOR-swizzled 16-byte chunks, and the loop runs over the flattened (tile, k-step) sequence, so the
// first loads of the next tile are in flight while the current one is finished.  At the board's power
// limit the 16x16x32 MFMA runs the same flops about 18 % faster than 32x32x16.
//
// An operand is k-contiguous ([rows, K]) or "k-major" ([K, rows] with the rows contiguous, kATrans /
// kBTrans): its fragments (8 consecutive k per lane) then come out of ds_read_b64_tr_b16, the LDS read
// of gfx950 that transposes 4 x 4 blocks of 16-bit entries across lanes, and rows of k beyond K read as
// zero through the range check of the buffer descriptor, so K needs no padding there.
#pragma once

#include "mrl_internal.h"

namespace mrl_tile {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Wavefront layout of the 256 x 256 tile: 2 wavefronts along m (128 rows of A each) by 2 along n
// (128 rows of B each); a wavefront owns 8 x 8 MFMA blocks of 16 x 16.
constexpr int kWavesN = 2;
constexpr int kWaves = 2 * kWavesN;
constexpr int kThreads = 64 * kWaves;
constexpr int kBlocks = 8;                       // 16-row blocks of A, and of B, per wavefront
constexpr int kLoadsPerWave = 32 / kWaves;       // 8-row groups of an operand that a wavefront brings in
constexpr int BM = 256;                          // rows of A per tile
constexpr int BN = 256;                          // rows of B per tile
constexpr int BK = 64;                           // k elements per LDS stage
constexpr int kOperandBytes = 256 * BK * 2;      // one operand of one stage: 256 rows x 128 bytes
constexpr int kStageBytes = 2 * kOperandBytes;   // A then B
constexpr int kLdsStages = 2 * kStageBytes;      // two stages

// Element offset (row * ld + column, without the k-step) of the chunk that lane `lane` of wavefront
// `wave` brings in with its load j (0..7) of an operand tile with `rows_valid` rows left (rows beyond
// are clamped to the last valid one; their products are never stored).  Physical slot of a 16-byte
// chunk inside its 256-byte pair of rows: logical slot ^ (pair & 15), logical = (row & 1) * 8 + chunk.
__device__ __forceinline__ int64_t stage_src_offset(int wave, int lane, int j, int64_t ld, int rows_valid) {
    const int phys_row = (wave * kLoadsPerWave + j) * 8 + (lane >> 3);
    const int pair = phys_row >> 1;
    const int slot = ((phys_row & 1) << 3) | (lane & 7);
    const int logical = slot ^ (pair & 15);
    int row = 2 * pair + (logical >> 3);
    if (row >= rows_valid) row = rows_valid - 1;
    return (int64_t)row * ld + (logical & 7) * 8;
}

// The same for a k-major operand [K, rows].  Its stage is cut into 4 column blocks of 64 rows of the
// operand; a column block holds its 64 k-rows at a pitch of 128 bytes (8 KiB), and load j of a
// wavefront fills 1 KiB with 8 k-rows of one column block, 8 lanes per 128-byte line as for the
// k-contiguous operand.  Inside a k-row the four 32-byte segments (16 rows of the operand, what one
// fragment read takes from it) are permuted: byte offset ^ (f(k) << 5), f(k) = (k >> 1 & 1) |
// ((k >> 3 & 1) << 1); with the bank half that k & 1 selects, the 8 k-rows that half a wavefront
// reads at a time fall on different banks.  Rows at or beyond `rows_valid` (a multiple of 8) are
// clamped to the last valid chunk.
__device__ __forceinline__ int tr_swizzle(int k) { return (((k >> 1) & 1) | (((k >> 3) & 1) << 1)) << 5; }
__device__ __forceinline__ int64_t stage_src_offset_kmajor(int wave, int lane, int j, int64_t ld, int rows_valid) {
    const int q = wave * kLoadsPerWave + j;
    const int k = 8 * (q & 7) + (lane >> 3);
    const int byte = ((lane & 7) * 16) ^ tr_swizzle(k);
    int row = (q >> 3) * 64 + (byte >> 1);
    if (row >= rows_valid) row = rows_valid - 8;
    return (int64_t)k * ld + row;
}


typedef floatx4 Accumulators[kBlocks][kBlocks];

// Runs the workgroup's tiles.  `smem`: kLdsStages bytes of LDS, 16-byte aligned (more is the caller's).
// `seq`: n_tiles and coords(j, tm, tn), the tile coordinates (in units of 256 rows of A and of B) of the
// j-th tile of this workgroup, uniform over the workgroup.  `epilogue(acc, tm, tn)` is called with the
// finished tile: wavefront (wv, wt) = (wave / 2, wave % 2) holds rows wv * 128 .. + 127 of A (m) and
// wt * 128 .. + 127 of B (n); acc[vb][tb] is the 16 x 16 block at m = 16 vb, n = 16 tb of it, of which a
// lane holds column n = lane & 15 and rows m = 4 (lane >> 4) .. + 3.  Rows of a ragged last tile beyond
// M or N hold products of clamped operand rows: the epilogue must skip them.  K % 64 == 0 unless an
// operand is k-major.  kEarly (0..4): how many of a stage's 16 requests go out early, see the schedule
// below.  Every thread of the workgroup must call this (it contains barriers).
template <bool kATrans, bool kBTrans, int kEarly, typename Seq, typename Epilogue>
__device__ __forceinline__ void mfma_tile_loop(unsigned char* smem, const uint16_t* __restrict__ A, int64_t lda, int M,
                                               const uint16_t* __restrict__ B, int64_t ldb, int N, int K, const Seq& seq,
                                               Epilogue&& epilogue) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wv = wave / kWavesN, wt = wave % kWavesN;
    const int n_tiles = seq.n_tiles;
    if (n_tiles <= 0) return;
    const int n_ksteps = (K + BK - 1) / BK;           // a last partial step only with k-major operands

    // ---- loader state: the tile whose stages are being requested
    int load_j = 0;                                   // index into the workgroup's tile sequence
    int load_k = 0;
    int a_off[kLoadsPerWave], b_off[kLoadsPerWave];
    mrl::rsrc_t a_rsrc, b_rsrc;
    int load_tm = 0, load_tn = 0;
    // A k-major operand takes a descriptor per stage: its base moves by 64 k-rows (which may be more
    // than the 4 GiB that an offset can span), and its range ends with row K, so that the k-rows of a
    // last partial step read as zero.
    auto set_load_stage = [&]() {
        const int k0 = load_k * BK;
        const int64_t k_rows = min(BK, K - k0);
        if (kATrans)
            a_rsrc = mrl::make_rsrc(A + (int64_t)k0 * lda + (int64_t)load_tm * BM,
                                    (uint32_t)((k_rows * lda - (int64_t)load_tm * BM) * 2));
        if (kBTrans)
            b_rsrc = mrl::make_rsrc(B + (int64_t)k0 * ldb + (int64_t)load_tn * BN,
                                    (uint32_t)((k_rows * ldb - (int64_t)load_tn * BN) * 2));
    };
    auto set_load_tile = [&](int j) {
        seq.coords(j, load_tm, load_tn);
        const int rows_a = min(BM, M - load_tm * BM), rows_b = min(BN, N - load_tn * BN);
#pragma unroll
        for (int i = 0; i < kLoadsPerWave; ++i) {
            a_off[i] = (int)((kATrans ? stage_src_offset_kmajor(wave, lane, i, lda, rows_a)
                                      : stage_src_offset(wave, lane, i, lda, rows_a)) * 2);
            b_off[i] = (int)((kBTrans ? stage_src_offset_kmajor(wave, lane, i, ldb, rows_b)
                                      : stage_src_offset(wave, lane, i, ldb, rows_b)) * 2);
        }
        // one descriptor per tile: byte offsets inside a tile stay below 2^32 for any operand size
        if (!kATrans) a_rsrc = mrl::make_rsrc(A + (int64_t)load_tm * BM * lda, 0xffffffffu);
        if (!kBTrans) b_rsrc = mrl::make_rsrc(B + (int64_t)load_tn * BN * ldb, 0xffffffffu);
        set_load_stage();
    };
    // request i (0..15) of the stage being requested: the wavefront's 8 groups of A, then of B
    auto issue_one = [&](int buf, int i) {
        const uint32_t k_bytes = (uint32_t)(load_k * BK * 2);
        unsigned char* dst = smem + buf * kStageBytes + (wave * kLoadsPerWave) * 1024;
        if (i < kLoadsPerWave)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (void __attribute__((address_space(3)))*)(dst + i * 1024), 16,
                                                 a_off[i], kATrans ? 0u : k_bytes, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                b_rsrc, (void __attribute__((address_space(3)))*)(dst + kOperandBytes + (i - kLoadsPerWave) * 1024), 16,
                b_off[i - kLoadsPerWave], kBTrans ? 0u : k_bytes, 0, 0);
    };
    // After the last stage of the last tile the requests go on (the schedule below has no branches):
    // they fetch valid bytes of the last tile into a buffer that nobody reads any more.
    auto stage_issued = [&]() {
        if (++load_k == n_ksteps) {
            load_k = 0;
            if (++load_j < n_tiles) set_load_tile(load_j);
            else set_load_stage();
        } else {
            set_load_stage();
        }
    };

    // Fragment addresses.  A lane reads row (lane & 15) of a 16-row block (8 row pairs, 2 KiB), chunk
    // 4 ks + (lane >> 4) of its 8: inside the block its pair is (lane >> 1) & 7, the pair's low bits
    // are ((block & 1) << 3) | that, and the physical slot is the logical one XOR those bits.
    int frag_off[2][2];                                   // [block parity][k sub-step of 32]
#pragma unroll
    for (int par = 0; par < 2; ++par)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int pair_in_block = (lane >> 1) & 7;
            const int slot = ((((lane & 1) ^ par) << 3) | ((4 * ks + (lane >> 4)) ^ pair_in_block));
            frag_off[par][ks] = pair_in_block * 256 + slot * 16;
        }
    // The same for a k-major operand: k-row 32 ks + 8 (lane >> 4) + 4 r + ((lane >> 2) & 3) for the two
    // reads r = 0, 1 of a fragment, 8 bytes at row 16 block + 4 (lane & 3) of it (column block
    // block >> 2, segment block & 3 of the k-row); after the transposing read, lane i of each 16 holds
    // row 16 block + i for 4 consecutive k.
    int tr_off[4];                                        // [block & 3]
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int g = lane >> 4, kk = (lane >> 2) & 3;
        tr_off[j] = (8 * g + kk) * 128 + ((j * 32) ^ tr_swizzle(8 * g + kk)) + (lane & 3) * 8;
    }
    // A k-contiguous operand's fragments are ordinary 16-byte loads (the compiler waits for them); a k-major
    // operand's arrive as the two 8-byte halves that the asm reads below deliver, and stay two values until
    // `landed` has passed them through the loop's own wait (members that a product does not use fold away).
    typedef long long2v __attribute__((ext_vector_type(2)));
    struct Frags {
        bf16x8 a[kBlocks], b[kBlocks];
        long a_lo[kBlocks], a_hi[kBlocks], b_lo[kBlocks], b_hi[kBlocks];
    };
    // fragment of 16-row block `blk` (0..15 inside the tile) of an operand whose stage starts at `op`
    auto read_kcontig = [&](const unsigned char* op, int blk, int ks) {
        return *reinterpret_cast<const bf16x8*>(op + blk * 2048 + frag_off[blk & 1][ks]);
    };
    // The transposing read goes out as inline assembly: through the builtin the compiler cannot tell it
    // from an access to the bytes that the requests in flight are writing and waits for all of them
    // (vmcnt(0)) before every read.  The price: it does not wait for the result either - the loop
    // below does (lgkmcnt(0) before a sub-step consumes fragments read during the one before), and
    // `landed` makes that wait the point where the halves become usable values: whatever the compiler does
    // with them (join them in place, or copy them) it can only do behind the wait.
    const unsigned smem_lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
    auto read_kmajor = [&](const unsigned char* op, int blk, int ks, long& lo, long& hi) {
        const unsigned addr = smem_lds + (unsigned)(op - smem) + (blk >> 2) * 8192 + ks * (32 * 128) + tr_off[blk & 3];
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(addr) : "memory");
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:512" : "=v"(hi) : "v"(addr) : "memory");
    };
    auto join = [](long lo, long hi) {
        long2v both;
        both[0] = lo;
        both[1] = hi;
        return __builtin_bit_cast(bf16x8, both);
    };
    // placed right behind the wait for a fragment set: every half of the set is an input and an output of an
    // empty statement there, so no use of it (and no copy of it) can be scheduled ahead of the wait
    auto landed = [&](Frags& f) {
        static_assert(kBlocks == 8, "the operand lists below name 8 fragments");
        if (kATrans)
            asm volatile("" : "+v"(f.a_lo[0]), "+v"(f.a_hi[0]), "+v"(f.a_lo[1]), "+v"(f.a_hi[1]), "+v"(f.a_lo[2]),
                              "+v"(f.a_hi[2]), "+v"(f.a_lo[3]), "+v"(f.a_hi[3]), "+v"(f.a_lo[4]), "+v"(f.a_hi[4]),
                              "+v"(f.a_lo[5]), "+v"(f.a_hi[5]), "+v"(f.a_lo[6]), "+v"(f.a_hi[6]), "+v"(f.a_lo[7]),
                              "+v"(f.a_hi[7]));
        if (kBTrans)
            asm volatile("" : "+v"(f.b_lo[0]), "+v"(f.b_hi[0]), "+v"(f.b_lo[1]), "+v"(f.b_hi[1]), "+v"(f.b_lo[2]),
                              "+v"(f.b_hi[2]), "+v"(f.b_lo[3]), "+v"(f.b_hi[3]), "+v"(f.b_lo[4]), "+v"(f.b_hi[4]),
                              "+v"(f.b_lo[5]), "+v"(f.b_hi[5]), "+v"(f.b_lo[6]), "+v"(f.b_hi[6]), "+v"(f.b_lo[7]),
                              "+v"(f.b_hi[7]));
    };
    // read r (0..15) of a fragment set, in the order the MFMAs need them: a0, all of b, a1..a7
    auto read1 = [&](Frags& f, const unsigned char* stage, int ks, int r) {
        const bool is_a = r == 0 || r > kBlocks;
        const int blk = r == 0 ? 0 : (r <= kBlocks ? r - 1 : r - kBlocks);
        if (is_a) {
            if (kATrans) read_kmajor(stage, wv * kBlocks + blk, ks, f.a_lo[blk], f.a_hi[blk]);
            else f.a[blk] = read_kcontig(stage, wv * kBlocks + blk, ks);
        } else {
            if (kBTrans) read_kmajor(stage + kOperandBytes, wt * kBlocks + blk, ks, f.b_lo[blk], f.b_hi[blk]);
            else f.b[blk] = read_kcontig(stage + kOperandBytes, wt * kBlocks + blk, ks);
        }
    };
    floatx4 acc[kBlocks][kBlocks];
    auto zero_acc = [&]() {
#pragma unroll
        for (int vb = 0; vb < kBlocks; ++vb)
#pragma unroll
            for (int tb = 0; tb < kBlocks; ++tb)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[vb][tb][i] = 0.f;
    };
    // Empty statements that demand every accumulator in the accumulator half of the register file:
    // placed after the zeroing and before the store, they keep the allocator from spreading the 64
    // four-register values over both halves (and copying them around inside the k loop).
    auto pin_acc = [&]() {
#pragma unroll
        for (int vb = 0; vb < kBlocks; ++vb)
#pragma unroll
            for (int tb = 0; tb < kBlocks; ++tb) asm volatile("" : "+a"(acc[vb][tb]));
    };
    auto mfma1 = [&](const Frags& f, int i) {
        const int vb = i / kBlocks, tb = i % kBlocks;
        const bf16x8 a = kATrans ? join(f.a_lo[vb], f.a_hi[vb]) : f.a[vb];
        const bf16x8 b = kBTrans ? join(f.b_lo[tb], f.b_hi[tb]) : f.b[tb];
        acc[vb][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[vb][tb], 0, 0, 0);
    };

    // One wavefront per SIMD: memory instructions are placed between the MFMAs of the same instruction
    // stream (an MFMA holds the matrix pipe for 16 cycles, other instructions issue meanwhile).  A
    // stage s (buffer s & 1) is two sub-steps of 64 MFMAs, each on a fragment set that was read during
    // the sub-step before:
    //   sub-step 0: MFMAs on G0 | reads G1 (s, k 32..63)  | the last kEarly requests of stage s+1
    //   wait for own requests and reads, barrier: stage s+1 has landed, buffer s & 1 is free
    //   sub-step 1: MFMAs on G1 | reads G0 (s+1, k 0..31) | the first 16 - kEarly requests of stage s+2
    //                                                        (into buffer s & 1)
    // How the 16 requests of a stage are best placed depends on the caller's tile order, measured at
    // 32 768 x 152 064 x 3584: the plain products (panels of tiles) want all of them in sub-step 1, one
    // every 4 MFMAs, so that each has a whole sub-step (1 us) before the barrier that needs it (4 of them
    // in sub-step 0: -4 %, 8: -11 %; twice or three times as dense right after the barrier: -1 .. -7 %);
    // the fused forward (a workgroup walks the vocabulary with one block of tokens) wants 4 of them in
    // sub-step 0 (0: -15 %, 2: -3 %, 8: -9 %).
#define MRL_SB __builtin_amdgcn_sched_barrier(0)
    constexpr int kMfmas = kBlocks * kBlocks, kReads = 2 * kBlocks, kLoads = 2 * kLoadsPerWave;
    static_assert(kMfmas == 64 && kReads == 16 && kLoads == 16, "the schedule below is written for these counts");
    static_assert(kEarly >= 0 && kEarly <= 4, "at most 4 early requests");
    constexpr int kLate = kLoads - kEarly, kLateEvery = kEarly == 0 ? 4 : 5;
    Frags G0, G1;
    set_load_tile(0);
#pragma unroll
    for (int i = 0; i < kLoads; ++i) issue_one(0, i);
    stage_issued();
    __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): stage 0 has landed
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kReads; ++r) read1(G0, smem, 0, r);
#pragma unroll
    for (int i = 0; i < kLate; ++i) issue_one(1, i);
    if (kEarly == 0) stage_issued();
    int stage_idx = 0;
    for (int mine = 0; mine < n_tiles; ++mine) {
        zero_acc();
        pin_acc();
        for (int kstep = 0; kstep < n_ksteps; ++kstep, ++stage_idx) {
            const int buf = stage_idx & 1;
            const unsigned char* stage = smem + buf * kStageBytes;
            const unsigned char* other = smem + (buf ^ 1) * kStageBytes;
            MRL_SB;
            if (kATrans || kBTrans) __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0): G0 has arrived
            landed(G0);
            MRL_SB;
#pragma unroll
            for (int i = 0; i < kMfmas; ++i) {
                mfma1(G0, i);
                MRL_SB;
                if (i % 3 == 0 && i / 3 < kReads) {
                    read1(G1, stage, 1, i / 3);
                    MRL_SB;
                }
                if (kEarly > 0 && i % 6 == 1 && i / 6 < kEarly) {
                    issue_one(buf ^ 1, kLate + i / 6);
                    MRL_SB;
                }
            }
            if (kEarly > 0) stage_issued();
            __builtin_amdgcn_s_waitcnt(0x0070);        // vmcnt(0) lgkmcnt(0)
            landed(G1);
            asm volatile("s_barrier" ::: "memory");
            MRL_SB;
#pragma unroll
            for (int i = 0; i < kMfmas; ++i) {
                mfma1(G1, i);
                MRL_SB;
                if (i % 3 == 0 && i / 3 < kReads) {
                    read1(G0, other, 0, i / 3);
                    MRL_SB;
                }
                if (i % kLateEvery == kLateEvery - (kEarly == 0 ? 1 : 4) && i / kLateEvery < kLate) {
                    issue_one(buf, i / kLateEvery);
                    MRL_SB;
                }
            }
            if (kEarly == 0) stage_issued();
        }
        pin_acc();
        int tm, tn;
        seq.coords(mine, tm, tn);
        epilogue(acc, tm, tn);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                // nothing is in flight into LDS when the workgroup ends
#undef MRL_SB
}

}  // namespace mrl_tile
