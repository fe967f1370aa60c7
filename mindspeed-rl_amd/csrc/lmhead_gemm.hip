// bf16 matrix products of the lm_head training step for gfx950 on the shared tile loop (lmhead_tile.h).
//
// One kernel covers the three products of the step, because each of them can be put in the form
//
//     out[n][m] (+)= sum_k A[m][k] * B[n][k]
//
// (the MFMA's M is the fast dimension of the output: in the 16x16 result layout a lane owns ONE
// column n and 4 consecutive rows m, i.e. 8 contiguous bytes of bf16 or 16 of fp32):
//
//     logits[t][v]  = sum_h W[v][h]      * hidden[t][h]      A = W,           B = hidden chunk
//     dHidden[t][h] = sum_v W[v][h]      * dlogits[t][v]     A = W (k-major), B = dlogits chunk
//     dW[v][h]     += sum_t hidden[t][h] * dlogits[t][v]     A = hidden,      B = dlogits chunk, both k-major
//
// so the backward reads hidden, W and dlogits as they lie: no transposed copies.
//
// Work distribution: one persistent workgroup per CU walks output tiles of 256 x 256.  Tiles are
// numbered so that 32 consecutive numbers are 8 tiles along m by 4 along n, and the 32 workgroups
// that share an XCD (and its L2) take 32 consecutive numbers at a time: the 4 that stream the same A
// tile and the 8 that stream the same B tile run side by side (see tile_coords for the order of the
// groups of 32).
#include <stdlib.h>

#include "lmhead_gemm.h"
#include "lmhead_tile.h"
#include "mrl_internal.h"
#include "vocab_common.h"

namespace {

using namespace mrl_vocab;
using namespace mrl_tile;

constexpr int kLdsTurn = 32 * 1024;              // where the wavefronts turn their result blocks (store_tile)
constexpr int kLdsBytes = kLdsStages + kLdsTurn;
constexpr int kTilesAlongN = 4;                  // tiles along n in a group of consecutive tile numbers

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

// The tiles of one workgroup: number first + j * stride.
struct StridedTiles {
    TileGrid grid;
    int64_t first, stride;
    int n_tiles;
    __device__ __forceinline__ void coords(int j, int& tm, int& tn) const { tile_coords(grid, first + j * stride, tm, tn); }
};

// kAccumulate: out is fp32 and the product is added to it; else out is bf16 and overwritten.
// kATrans / kBTrans: the operand is k-major, [K, M] or [K, N]; else [M, K] or [N, K].
template <bool kAccumulate, bool kATrans, bool kBTrans>
__global__ __launch_bounds__(kThreads, 1) void gemm_kernel(const uint16_t* __restrict__ A, int64_t lda, int M,
                                                           const uint16_t* __restrict__ B, int64_t ldb, int N, int K,
                                                           void* __restrict__ out, int64_t ldo) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wv = wave / kWavesN, wt = wave % kWavesN;

    StridedTiles seq;
    seq.grid.tiles_m = (M + BM - 1) / BM;
    seq.grid.tiles_n = (N + BN - 1) / BN;
    seq.grid.total = (int64_t)seq.grid.tiles_m * seq.grid.tiles_n;
    // panels of up to 8 rows of tiles (8 x 4 blocks per XCD), tall products up to 32; all panels the same
    // height (14 rows of tiles as 7 + 7 measured 1.7 % faster than as 8 + 6)
    const int panel_cap = seq.grid.tiles_m >= 64 ? 32 : 8;
    const int n_panels = (seq.grid.tiles_m + panel_cap - 1) / panel_cap;
    seq.grid.panel_m = (seq.grid.tiles_m + n_panels - 1) / n_panels;
    // workgroups are dealt round-robin to the 8 XCDs: the gridDim / 8 workgroups of an XCD take
    // consecutive tile numbers
    const int per_xcd = gridDim.x >> 3;
    seq.first = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    seq.stride = gridDim.x;
    seq.n_tiles = seq.first < seq.grid.total ? (int)((seq.grid.total - 1 - seq.first) / seq.stride) + 1 : 0;

    // The finished tile.  A lane holds column n = lane & 15 of each 16 x 16 block and rows
    // 4 (lane >> 4) .. + 3 of it: stored like that, a store instruction would touch 16 output rows with
    // 8 or 16 bytes each.  Each wavefront therefore turns its blocks through a private 8 KiB of LDS:
    // [64 n][128 bytes of m] at a time (4 blocks along n by 4 along m for bf16, by 2 for fp32), 16-byte
    // chunks XOR-swizzled by the row pair, written in the MFMA layout and read back as 8 lanes x 16 bytes
    // per output row, so that every store covers whole 128-byte lines.
    unsigned char* turn = smem + kLdsStages + wave * (kLdsTurn / kWaves);
    auto store_tile = [&](mrl_tile::Accumulators& acc, int tm, int tn) {
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

    mfma_tile_loop<kATrans, kBTrans, 0>(smem, A, lda, M, B, ldb, N, K, seq, store_tile);
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
    // function attributes belong to a device: reserved with every launch, on whichever device is current
    const hipError_t attr = hipFuncSetAttribute((const void*)gemm_kernel<kAccumulate, kATrans, kBTrans>,
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
