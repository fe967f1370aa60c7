// Version, per-thread error message and the calibration copy kernel of libmrl_hip.so.
#include <stdarg.h>
#include <string.h>

#include "mrl_internal.h"

namespace mrl {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_error[0] = '\0'; }

}  // namespace mrl

namespace {

// One 16-byte load and one 16-byte store per thread per iteration, grid-stride.
__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                   int64_t n_vec) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n_vec; i += step) {
        u32x4 v = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(v, dst + i);
    }
}


// Bandwidth probes with the access pattern of the sweeps: one workgroup of 1024 threads per row of
// `row_vec` 16-byte vectors.  They give the practical ceilings the kernels are measured against.
constexpr int kProbeBlock = 1024;
constexpr int kProbeMaxVec = 19;

// read-only: every vector is loaded and folded into a value that is (never) written
__global__ __launch_bounds__(kProbeBlock) void probe_read_kernel(const u32x4* __restrict__ src, int64_t row_vec,
                                                                 unsigned* __restrict__ sink) {
    const u32x4* row = src + (int64_t)blockIdx.x * row_vec;
    unsigned acc = 0;
    for (int64_t i = threadIdx.x; i < row_vec; i += kProbeBlock) {
        const u32x4 v = __builtin_nontemporal_load(row + i);
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

__global__ __launch_bounds__(kProbeBlock) void probe_write_kernel(u32x4* __restrict__ dst, int64_t row_vec) {
    u32x4* row = dst + (int64_t)blockIdx.x * row_vec;
    const u32x4 v = {1u, 2u, 3u, 4u};
    for (int64_t i = threadIdx.x; i < row_vec; i += kProbeBlock) __builtin_nontemporal_store(v, row + i);
}

// copy with the whole row in registers: all loads of a workgroup are issued before its stores;
// range-checked buffer accesses keep the body free of branches
__global__ __launch_bounds__(kProbeBlock) void probe_copy_kernel(const u32x4* __restrict__ src,
                                                                 u32x4* __restrict__ dst, int row_vec) {
    const mrl::rsrc_t s = mrl::make_rsrc(src + (int64_t)blockIdx.x * row_vec, (uint32_t)row_vec * 16u);
    const mrl::rsrc_t d = mrl::make_rsrc(dst + (int64_t)blockIdx.x * row_vec, (uint32_t)row_vec * 16u);
    u32x4 v[kProbeMaxVec];
#pragma unroll
    for (int q = 0; q < kProbeMaxVec; ++q) v[q] = mrl::buf_load_nt(s, (uint32_t)(q * kProbeBlock + threadIdx.x) * 16u);
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kProbeMaxVec; ++q) mrl::buf_store_nt(v[q], d, (uint32_t)(q * kProbeBlock + threadIdx.x) * 16u);
}

// The same three streams with the pattern the HBM system serves best: small workgroups that each
// touch ONE vector per thread and retire, so that the requests in flight at any moment cover one
// compact, advancing stretch of memory.  These are the ceilings of the machine rather than of the
// row-per-workgroup pattern.
__global__ __launch_bounds__(1024) void stream_read_kernel(const u32x4* __restrict__ src, int64_t n_vec,
                                                           unsigned* __restrict__ sink) {
    const int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    if (i >= n_vec) return;
    const u32x4 v = __builtin_nontemporal_load(src + i);
    if ((v.x ^ v.y ^ v.z ^ v.w) == 0x9e3779b9u) sink[0] = v.x;
}

__global__ __launch_bounds__(256) void stream_write_kernel(u32x4* __restrict__ dst, int64_t n_vec) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const u32x4 v = {1u, 2u, 3u, 4u};
    if (i < n_vec) dst[i] = v;
}

__global__ __launch_bounds__(64) void stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                         int64_t n_vec) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i < n_vec) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

}  // namespace

extern "C" int mrl_version(void) { return MRL_VERSION; }

extern "C" const char* mrl_last_error(void) { return mrl::g_error; }

extern "C" int mrl_copy_bytes(const void* src, void* dst, int64_t n_bytes, void* stream) {
    MRL_REQUIRE(src && dst, MRL_ERR_INVALID_ARG, "mrl_copy_bytes: NULL pointer");
    MRL_REQUIRE(n_bytes >= 0 && n_bytes % 16 == 0, MRL_ERR_INVALID_ARG,
                "mrl_copy_bytes: n_bytes=%lld must be a non-negative multiple of 16", (long long)n_bytes);
    MRL_REQUIRE(mrl::aligned(src, 16) && mrl::aligned(dst, 16), MRL_ERR_MISALIGNED,
                "mrl_copy_bytes: pointers must be 16-byte aligned");
    if (n_bytes == 0) return MRL_OK;
    const int64_t n_vec = n_bytes / 16;
    int64_t blocks = (n_vec + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, mrl::as_stream(stream),
                       (const u32x4*)src, (u32x4*)dst, n_vec);
    return mrl::check_launch("mrl_copy_bytes");
}

extern "C" int mrl_bandwidth_probe(int mode, const void* src, void* dst, int64_t n_rows, int64_t row_bytes,
                                   void* stream) {
    const char* fn = "mrl_bandwidth_probe";
    MRL_REQUIRE(mode >= 0 && mode <= 5, MRL_ERR_INVALID_ARG,
                "%s: mode=%d (0 read, 1 write, 2 copy by rows; 3 read, 4 write, 5 copy streaming)", fn, mode);
    MRL_REQUIRE(n_rows >= 0 && n_rows <= 0x7fffffffLL && row_bytes > 0 && row_bytes % 16 == 0, MRL_ERR_INVALID_ARG,
                "%s: n_rows=%lld row_bytes=%lld (row_bytes must be a positive multiple of 16)", fn, (long long)n_rows,
                (long long)row_bytes);
    MRL_REQUIRE(row_bytes / 16 <= (int64_t)kProbeMaxVec * kProbeBlock, MRL_ERR_UNSUPPORTED,
                "%s: row_bytes=%lld exceeds %d bytes", fn, (long long)row_bytes, kProbeMaxVec * kProbeBlock * 16);
    if (n_rows == 0) return MRL_OK;
    MRL_REQUIRE((mode == 1 || mode == 4 || src != nullptr) && dst != nullptr, MRL_ERR_INVALID_ARG, "%s: NULL pointer",
                fn);
    MRL_REQUIRE(mrl::aligned(src, 16) && mrl::aligned(dst, 16), MRL_ERR_MISALIGNED, "%s: pointers must be 16-byte aligned",
                fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid((unsigned)n_rows), block(kProbeBlock);
    const int64_t row_vec = row_bytes / 16;
    const int64_t n_vec = n_rows * row_vec;
    if (mode >= 3) {
        const int64_t per = mode == 3 ? 1024 : (mode == 4 ? 256 : 64);
        const int64_t blocks = (n_vec + per - 1) / per;
        MRL_REQUIRE(blocks <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: %lld bytes are too many for one launch", fn,
                    (long long)(n_vec * 16));
        const dim3 sgrid((unsigned)blocks);
        if (mode == 3) {
            hipLaunchKernelGGL(stream_read_kernel, sgrid, dim3(1024), 0, s, (const u32x4*)src, n_vec, (unsigned*)dst);
        } else if (mode == 4) {
            hipLaunchKernelGGL(stream_write_kernel, sgrid, dim3(256), 0, s, (u32x4*)dst, n_vec);
        } else {
            hipLaunchKernelGGL(stream_copy_kernel, sgrid, dim3(64), 0, s, (const u32x4*)src, (u32x4*)dst, n_vec);
        }
        return mrl::check_launch(fn);
    }
    if (mode == 0) {
        hipLaunchKernelGGL(probe_read_kernel, grid, block, 0, s, (const u32x4*)src, row_vec, (unsigned*)dst);
    } else if (mode == 1) {
        hipLaunchKernelGGL(probe_write_kernel, grid, block, 0, s, (u32x4*)dst, row_vec);
    } else {
        hipLaunchKernelGGL(probe_copy_kernel, grid, block, 0, s, (const u32x4*)src, (u32x4*)dst, (int)row_vec);
    }
    return mrl::check_launch(fn);
}
