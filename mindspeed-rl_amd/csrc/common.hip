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
