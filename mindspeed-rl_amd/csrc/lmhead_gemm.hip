// bf16 matrix products of the lm_head training step for gfx950: operands go from global memory
// straight into LDS (buffer_load ... lds), two 64 KiB stages, XOR-swizzled 16-byte chunks,
// v_mfma_f32_16x16x32_bf16 (at the board's power limit this shape runs about 18 % faster than the
// same flops as 32x32x16), memory instructions placed between the MFMAs of one instruction stream.
//
// One kernel covers the three products of the step, because each of them can be put in the form
//
//     out[n][m] (+)= sum_k A[m][k] * B[n][k]          A: [M, K], B: [N, K], both with k contiguous
//
// (the MFMA's M is the fast dimension of the output: in the 16x16 result layout a lane owns ONE
// column n and 4 consecutive rows m, i.e. 8 contiguous bytes of bf16 or 16 of fp32):
//
//     logits[t][v]  = sum_h W[v][h]      * hidden[t][h]      A = W,         B = hidden chunk
//     dHidden[t][h] = sum_v W[v][h]      * dlogits[t][v]     A = W (k-major), B = dlogits chunk
//     dW[v][h]     += sum_t hidden[t][h]   * dlogits[t][v]     A = hidden,    B = dlogits chunk, both k-major
//
// An operand may also be given "k-major", as [K, rows] with the rows contiguous (kATrans / kBTrans):
// its stage is then 64 k-rows by 256 rows of the operand in LDS, and the fragments (8 consecutive k per lane) come
// out of ds_read_b64_tr_b16, the LDS read of gfx950 that transposes 4 x 4 blocks of 16-bit entries
// across lanes.  dHidden uses it for W, dW for both operands, hidden [t][h] and dlogits [t][v] as they lie;
// rows of k beyond K read as zero through the range check of the buffer descriptor, so K needs no padding there.
//
// Work distribution: one persistent 256-thread workgroup per CU (2 x 2 wavefronts, one per SIMD,
// wavefront tile 128 x 128 in 256 accumulator registers) walks output tiles of 256 x 256.  Tiles are
// numbered so that 32 consecutive numbers are 8 tiles along m by 4 along n, and the 32 workgroups
// that share an XCD (and its L2) take 32 consecutive numbers at a time: the 4 that stream the same A
// tile and the 8 that stream the same B tile run side by side (see tile_coords for the order of the
// groups of 32).  The loop runs over the flattened (tile, k-step) sequence of a workgroup, so the
// first loads of its next tile are in flight while the current one is stored.
#include <stdlib.h>

#include "lmhead_gemm.h"
#include "mrl_internal.h"
#include "vocab_common.h"

namespace {

using namespace mrl_vocab;

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
constexpr int kLdsTurn = 32 * 1024;              // where the wavefronts turn their result blocks (store_tile)
constexpr int kLdsBytes = kLdsStages + kLdsTurn;
constexpr int kTilesAlongN = 4;                  // tiles along n in a group of consecutive tile numbers

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

struct TileGrid {
    int tiles_m, tiles_n, panel_m;
    int64_t total;
};

// Tile number -> (tile along m, tile along n).  Tiles are numbered panel by panel, a panel being
// panel_m tiles along m by all tiles along n; inside a panel consecutive numbers walk m first inside
// a group of 4 tiles along n (4 consecutive numbers are one tile of A with 4 tiles of B), and the groups
// walk along n.  With panel_m = 8 the 32 workgroups of an XCD hold 8 (m) x 4 (n) tiles and the 8 XCDs
// 8 x 32; with 32 an XCD still holds 8 x 4 and the chip 32 x 8, which fetches less from beyond the L2
// (B is passed over a quarter as often).
// A workgroup keeps its tile of A from one of its tiles to the next.
__device__ __forceinline__ void tile_coords(const TileGrid& g, int64_t t, int& tm, int& tn) {
    const int64_t per_panel = (int64_t)g.panel_m * g.tiles_n;
    const int p = (int)(t / per_panel);
    const int idx = (int)(t - (int64_t)p * per_panel);
    const int pm = min(g.panel_m, g.tiles_m - p * g.panel_m);   // rows of tiles in this panel
    const int ng = idx / (pm * kTilesAlongN);
    const int rem = idx - ng * (pm * kTilesAlongN);
    const int width = min(kTilesAlongN, g.tiles_n - ng * kTilesAlongN);
    tm = p * g.panel_m + rem / width;
    tn = ng * kTilesAlongN + rem % width;
}

// kAccumulate: out is fp32 and the product is added to it; else out is bf16 and overwritten.
// kATrans / kBTrans: the operand is k-major, [K, M] or [K, N]; else [M, K] or [N, K].
template <bool kAccumulate, bool kATrans, bool kBTrans>
__global__ __launch_bounds__(kThreads, 1) void gemm_kernel(const uint16_t* __restrict__ A, int64_t lda, int M,
                                                              const uint16_t* __restrict__ B, int64_t ldb, int N, int K,
                                                              void* __restrict__ out, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wv = wave / kWavesN, wt = wave % kWavesN;

    TileGrid grid;
    grid.tiles_m = (M + BM - 1) / BM;
    grid.tiles_n = (N + BN - 1) / BN;
    grid.total = (int64_t)grid.tiles_m * grid.tiles_n;
    // panels of 8 rows of tiles line up with the 8 x 4 blocks of an XCD; tall products take 32
    grid.panel_m = grid.tiles_m >= 64 ? 32 : 8;
    // workgroups are dealt round-robin to the 8 XCDs: the gridDim / 8 workgroups of an XCD take
    // consecutive tile numbers
    const int per_xcd = gridDim.x >> 3;
    const int64_t first_tile = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    const int64_t tile_stride = gridDim.x;
    if (first_tile >= grid.total) return;
    const int my_tiles = (int)((grid.total - 1 - first_tile) / tile_stride) + 1;
    const int n_ksteps = (K + BK - 1) / BK;           // a last partial step only with k-major operands

    // ---- loader state: the tile whose stages are being requested
    int64_t load_tile = first_tile;
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
    auto set_load_tile = [&](int64_t t) {
        tile_coords(grid, t, load_tm, load_tn);
        const int rows_a = min(BM, M - load_tm * BM), rows_b = min(BN, N - load_tn * BN);
#pragma unroll
        for (int j = 0; j < kLoadsPerWave; ++j) {
            a_off[j] = (int)((kATrans ? stage_src_offset_kmajor(wave, lane, j, lda, rows_a)
                                      : stage_src_offset(wave, lane, j, lda, rows_a)) * 2);
            b_off[j] = (int)((kBTrans ? stage_src_offset_kmajor(wave, lane, j, ldb, rows_b)
                                      : stage_src_offset(wave, lane, j, ldb, rows_b)) * 2);
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
            load_tile += tile_stride;
            if (load_tile < grid.total) set_load_tile(load_tile);
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
    struct Frags {
        bf16x8 a[kBlocks], b[kBlocks];
    };
    // fragment of 16-row block `blk` (0..15 inside the tile) of an operand whose stage starts at `op`
    auto read_kcontig = [&](const unsigned char* op, int blk, int ks) {
        return *reinterpret_cast<const bf16x8*>(op + blk * 2048 + frag_off[blk & 1][ks]);
    };
    // The transposing read goes out as inline assembly: through the builtin the compiler cannot tell it
    // from an access to the bytes that the requests in flight are writing and waits for all of them
    // (vmcnt(0)) before every read.  The price: it does not wait for the result either - the loop
    // below does (lgkmcnt(0) before a sub-step consumes fragments read during the one before).
    const unsigned smem_lds = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
    auto read_kmajor = [&](const unsigned char* op, int blk, int ks) {
        typedef long long2v __attribute__((ext_vector_type(2)));
        const unsigned addr = smem_lds + (unsigned)(op - smem) + (blk >> 2) * 8192 + ks * (32 * 128) + tr_off[blk & 3];
        long2v both;
        long lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(addr) : "memory");
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:512" : "=v"(hi) : "v"(addr) : "memory");
        both[0] = lo;
        both[1] = hi;
        return __builtin_bit_cast(bf16x8, both);
    };
    // read r (0..15) of a fragment set, in the order the MFMAs need them: a0, all of b, a1..a7
    auto read1 = [&](Frags& f, const unsigned char* stage, int ks, int r) {
        const bool is_a = r == 0 || r > kBlocks;
        const int blk = r == 0 ? 0 : (r <= kBlocks ? r - 1 : r - kBlocks);
        if (is_a)
            f.a[blk] = kATrans ? read_kmajor(stage, wv * kBlocks + blk, ks) : read_kcontig(stage, wv * kBlocks + blk, ks);
        else
            f.b[blk] = kBTrans ? read_kmajor(stage + kOperandBytes, wt * kBlocks + blk, ks)
                               : read_kcontig(stage + kOperandBytes, wt * kBlocks + blk, ks);
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
        acc[vb][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.a[vb], f.b[tb], acc[vb][tb], 0, 0, 0);
    };
    // The finished tile.  A lane holds column n = lane & 15 of each 16 x 16 block and rows
    // 4 (lane >> 4) .. + 3 of it: stored like that, a store instruction would touch 16 output rows with
    // 8 or 16 bytes each.  Each wavefront therefore turns its blocks through a private 8 KiB of LDS:
    // [64 n][128 bytes of m] at a time (4 blocks along n by 4 along m for bf16, by 2 for fp32), 16-byte
    // chunks XOR-swizzled by the row pair, written in the MFMA layout and read back as 8 lanes x 16 bytes
    // per output row, so that every store covers whole 128-byte lines.
    unsigned char* turn = smem + kLdsStages + wave * (kLdsTurn / kWaves);
    auto store_tile = [&](int64_t t) {
        int tm, tn;
        tile_coords(grid, t, tm, tn);
        const int row_w = lane & 15, quarter = lane >> 4;        // writer: its n, its run of 4 m inside the block
        const int row_r = lane >> 3, chunk_r = lane & 7;          // reader: n within a group of 8, 16-byte chunk
        constexpr int kMPerPass = kAccumulate ? 2 : 4;            // 32 fp32 or 64 bf16 entries of m are 128 bytes
#pragma unroll
        for (int tb0 = 0; tb0 < kBlocks; tb0 += 4) {
            const int n0 = tn * BN + wt * 128 + tb0 * 16;
#pragma unroll
            for (int vb0 = 0; vb0 < kBlocks; vb0 += kMPerPass) {
                const int m0 = tm * BM + wv * 128 + vb0 * 16;
#pragma unroll
                for (int tbi = 0; tbi < 4; ++tbi) {
                    const int row = tbi * 16 + row_w;
                    unsigned char* line = turn + row * 128;
                    const int key = (row >> 1) & 7;
#pragma unroll
                    for (int vbi = 0; vbi < kMPerPass; ++vbi) {
                        const floatx4& c = acc[vb0 + vbi][tb0 + tbi];
                        if (kAccumulate) {
                            *reinterpret_cast<float4*>(line + (((vbi * 4 + quarter) ^ key) * 16)) =
                                make_float4(c[0], c[1], c[2], c[3]);
                        } else {
                            uint2 w;
                            w.x = Elem<MRL_BF16>::pack2(c[0], c[1]);
                            w.y = Elem<MRL_BF16>::pack2(c[2], c[3]);
                            *reinterpret_cast<uint2*>(line + (((vbi * 2 + (quarter >> 1)) ^ key) * 16) + (quarter & 1) * 8) = w;
                        }
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);            // lgkmcnt(0): the slice is written
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    const int row = g * 8 + row_r;
                    const u32x4 v =
                        *reinterpret_cast<const u32x4*>(turn + row * 128 + ((chunk_r ^ ((row >> 1) & 7)) * 16));
                    const int n = n0 + row;
                    const int m = m0 + chunk_r * (kAccumulate ? 4 : 8);
                    if (n < N && m < M) {                      // M % 8 == 0: a chunk is inside or outside
                        if (kAccumulate) {
                            float4* p = reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + (int64_t)n * ldo + m);
                            float4 c = *p;
                            c.x += __uint_as_float(v.x);
                            c.y += __uint_as_float(v.y);
                            c.z += __uint_as_float(v.z);
                            c.w += __uint_as_float(v.w);
                            *p = c;
                        } else {
                            *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(out) + (int64_t)n * ldo + m) = v;
                        }
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);            // the slice has been read: it may be rewritten
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // One wavefront per SIMD: memory instructions are placed between the MFMAs of the same instruction
    // stream (an MFMA holds the matrix pipe for 16 cycles, other instructions issue meanwhile).  A
    // stage s (buffer s & 1) is two sub-steps of 64 MFMAs, each on a fragment set that was read during
    // the sub-step before:
    //   sub-step 0: MFMAs on G0 | reads G1 (s, k 32..63)  | requests 12..15 of stage s+1
    //   wait for own requests and reads, barrier: stage s+1 has landed, buffer s & 1 is free
    //   sub-step 1: MFMAs on G1 | reads G0 (s+1, k 0..31) | requests 0..11 of stage s+2 (into buffer s & 1)
#define MRL_SB __builtin_amdgcn_sched_barrier(0)
    constexpr int kMfmas = kBlocks * kBlocks, kReads = 2 * kBlocks, kLoads = 2 * kLoadsPerWave;
    static_assert(kMfmas == 64 && kReads == 16 && kLoads == 16, "the schedule below is written for these counts");
    Frags G0, G1;
    set_load_tile(load_tile);
#pragma unroll
    for (int i = 0; i < kLoads; ++i) issue_one(0, i);
    stage_issued();
    __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): stage 0 has landed
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kReads; ++r) read1(G0, smem, 0, r);
#pragma unroll
    for (int i = 0; i < 12; ++i) issue_one(1, i);
    int stage_idx = 0;
    for (int mine = 0; mine < my_tiles; ++mine) {
        zero_acc();
        pin_acc();
        for (int kstep = 0; kstep < n_ksteps; ++kstep, ++stage_idx) {
            const int buf = stage_idx & 1;
            const unsigned char* stage = smem + buf * kStageBytes;
            const unsigned char* other = smem + (buf ^ 1) * kStageBytes;
            MRL_SB;
            if (kATrans || kBTrans) __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0): G0 has arrived
            MRL_SB;
#pragma unroll
            for (int i = 0; i < kMfmas; ++i) {
                mfma1(G0, i);
                MRL_SB;
                if (i % 3 == 0 && i / 3 < kReads) {
                    read1(G1, stage, 1, i / 3);
                    MRL_SB;
                }
                if (i % 6 == 1 && i / 6 < 4) {
                    issue_one(buf ^ 1, 12 + i / 6);
                    MRL_SB;
                }
            }
            stage_issued();
            __builtin_amdgcn_s_waitcnt(0x0070);        // vmcnt(0) lgkmcnt(0)
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
                if (i % 5 == 1 && i / 5 < 12) {
                    issue_one(buf, i / 5);
                    MRL_SB;
                }
            }
        }
        pin_acc();
        store_tile(first_tile + (int64_t)mine * tile_stride);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                // nothing is in flight into LDS when the workgroup ends
#undef MRL_SB
}

int persistent_grid() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return n & ~7;          // a whole number of workgroups per XCD
}

}  // namespace

namespace mrl {

template <bool kAccumulate, bool kATrans, bool kBTrans>
static int launch_gemm(const char* fn, int grid, const void* a, int64_t lda, int64_t m, const void* b, int64_t ldb, int64_t n,
                       int64_t k, void* out, int64_t ldo, hipStream_t stream) {
    static const hipError_t attr = hipFuncSetAttribute((const void*)gemm_kernel<kAccumulate, kATrans, kBTrans>,
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    MRL_REQUIRE(attr == hipSuccess, MRL_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS", fn, kLdsBytes);
    hipLaunchKernelGGL((gemm_kernel<kAccumulate, kATrans, kBTrans>), dim3((unsigned)grid), dim3(kThreads), kLdsBytes, stream,
                       (const uint16_t*)a, lda, (int)m, (const uint16_t*)b, ldb, (int)n, (int)k, out, ldo);
    return check_launch(fn);
}

int gemm_bf16(const char* fn, const void* a, int64_t lda, int64_t m, bool a_kmajor, const void* b, int64_t ldb, int64_t n,
              bool b_kmajor, int64_t k, void* out, int64_t ldo, bool accumulate_f32, hipStream_t stream) {
    MRL_REQUIRE(m > 0 && n > 0 && k > 0 && m % 8 == 0, MRL_ERR_UNSUPPORTED, "%s: product of m=%lld n=%lld k=%lld (m must be a multiple of 8)",
                fn, (long long)m, (long long)n, (long long)k);
    MRL_REQUIRE(m <= 0x7fffffffLL && n <= 0x7fffffffLL && k <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: size out of range",
                fn);
    const int64_t k_steps = (k + BK - 1) / BK * BK;        // what a k-contiguous operand is read up to
    MRL_REQUIRE((a_kmajor || b_kmajor) || k % BK == 0, MRL_ERR_UNSUPPORTED,
                "%s: k=%lld must be a multiple of %d when no operand is k-major", fn, (long long)k, BK);
    MRL_REQUIRE(!b_kmajor || n % 8 == 0, MRL_ERR_UNSUPPORTED, "%s: n=%lld must be a multiple of 8 for a k-major b", fn,
                (long long)n);
    MRL_REQUIRE(lda >= (a_kmajor ? m : k_steps) && ldb >= (b_kmajor ? n : k_steps) && ldo >= m && lda % 8 == 0 &&
                    ldb % 8 == 0 && ldo % 8 == 0,
                MRL_ERR_INVALID_ARG, "%s: leading dimensions lda=%lld ldb=%lld ldo=%lld", fn, (long long)lda, (long long)ldb,
                (long long)ldo);
    // what one buffer descriptor has to span: a tile of 256 rows, or a stage of 64 k-rows
    MRL_REQUIRE(256 * lda * 2 < (1LL << 31) && 256 * ldb * 2 < (1LL << 31), MRL_ERR_UNSUPPORTED,
                "%s: 256 rows of an operand must stay below 2 GiB", fn);
    MRL_REQUIRE(aligned(a, 16) && aligned(b, 16) && aligned(out, 16), MRL_ERR_MISALIGNED,
                "%s: operands must be 16-byte aligned", fn);
    const int grid = persistent_grid();
    MRL_REQUIRE(grid >= 8, MRL_ERR_LAUNCH, "%s: cannot query the device", fn);
    if (!a_kmajor && !b_kmajor && !accumulate_f32)
        return launch_gemm<false, false, false>(fn, grid, a, lda, m, b, ldb, n, k, out, ldo, stream);
    if (a_kmajor && !b_kmajor && !accumulate_f32)
        return launch_gemm<false, true, false>(fn, grid, a, lda, m, b, ldb, n, k, out, ldo, stream);
    if (a_kmajor && b_kmajor && accumulate_f32)
        return launch_gemm<true, true, true>(fn, grid, a, lda, m, b, ldb, n, k, out, ldo, stream);
    MRL_REQUIRE(false, MRL_ERR_UNSUPPORTED, "%s: this combination of operand layouts is not built", fn);
    return MRL_ERR_UNSUPPORTED;
}

}  // namespace mrl

// ------------------------------------------------------------------------------------------ C ABI
extern "C" int mrl_lmhead_logits(const void* hidden, const void* weight, int64_t n_tokens, int64_t vocab,
                                 int64_t hidden_dim, void* logits, int64_t logits_row_stride, void* stream) {
    const char* fn = "mrl_lmhead_logits";
    MRL_REQUIRE(n_tokens >= 0 && vocab > 0 && hidden_dim > 0, MRL_ERR_INVALID_ARG,
                "%s: n_tokens=%lld vocab=%lld hidden_dim=%lld", fn, (long long)n_tokens, (long long)vocab,
                (long long)hidden_dim);
    MRL_REQUIRE(hidden_dim % BK == 0 && vocab % 8 == 0 && logits_row_stride % 8 == 0, MRL_ERR_UNSUPPORTED,
                "%s: hidden_dim=%lld must be a multiple of %d, vocab=%lld and the row stride of 8", fn, (long long)hidden_dim, BK,
                (long long)vocab);
    MRL_REQUIRE(logits_row_stride >= vocab, MRL_ERR_INVALID_ARG, "%s: logits_row_stride below vocab", fn);
    if (n_tokens == 0) return MRL_OK;
    MRL_REQUIRE(hidden && weight && logits, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    return mrl::gemm_bf16(fn, weight, hidden_dim, vocab, false, hidden, hidden_dim, n_tokens, false, hidden_dim, logits,
                          logits_row_stride, false, mrl::as_stream(stream));
}

extern "C" int mrl_lmhead_logprob_bwd(const void* hidden, const void* weight, const void* dlogits,
                                      int64_t dlogits_row_stride, int64_t n_tokens, int64_t vocab, int64_t hidden_dim,
                                      void* d_hidden, float* d_weight, void* stream) {
    const char* fn = "mrl_lmhead_logprob_bwd";
    MRL_REQUIRE(n_tokens >= 0 && vocab > 0 && hidden_dim > 0, MRL_ERR_INVALID_ARG,
                "%s: n_tokens=%lld vocab=%lld hidden_dim=%lld", fn, (long long)n_tokens, (long long)vocab,
                (long long)hidden_dim);
    MRL_REQUIRE(hidden_dim % 8 == 0 && vocab % 8 == 0, MRL_ERR_UNSUPPORTED,
                "%s: hidden_dim=%lld and vocab=%lld must be multiples of 8", fn, (long long)hidden_dim, (long long)vocab);
    MRL_REQUIRE(dlogits_row_stride % BK == 0 && dlogits_row_stride >= vocab, MRL_ERR_INVALID_ARG,
                "%s: dlogits_row_stride=%lld must be a multiple of %d and at least vocab (the padding columns must hold "
                "zeros)", fn, (long long)dlogits_row_stride, BK);
    if (n_tokens == 0) return MRL_OK;
    MRL_REQUIRE(hidden && weight && dlogits && d_hidden && d_weight, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    hipStream_t s = mrl::as_stream(stream);
    // dHidden[t][h] = sum_v W[v][h] * dlogits[t][v]: the weight as it lies is the k-major operand; its rows
    // beyond vocab read as zero, dlogits is read up to the next multiple of 64 columns
    int rc = mrl::gemm_bf16(fn, weight, hidden_dim, hidden_dim, true, dlogits, dlogits_row_stride, n_tokens, false, vocab,
                            d_hidden, hidden_dim, false, s);
    if (rc != MRL_OK) return rc;
    // dW[v][h] += sum_t hidden[t][h] * dlogits[t][v]: both operands k-major as they lie, any n_tokens
    return mrl::gemm_bf16(fn, hidden, hidden_dim, hidden_dim, true, dlogits, dlogits_row_stride, vocab, true, n_tokens,
                          d_weight, hidden_dim, true, s);
}
